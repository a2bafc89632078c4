#!/usr/bin/env python3
"""Benchmark of the HIP hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--only NAME]

A "step" is one pass of the headline workload over one batch of synthetic input that is already
resident in HBM: BASELINE config 2, the fused conv2d + bias + ReLU (f32, N32 C64->128 56x56 3x3 s1 p1).
The single JSON line printed at the end carries that workload as `value` and lists every other
BASELINE configuration (f32 GEMM 512^3, bf16 GEMM 4096^3 and 16x4096x4096, attention S2048 causal and
non-causal, the decoder stack) under `workloads`, each with its own roofline figures.

Timing: W untimed warm-up steps, then exactly K steps bracketed by a device synchronisation on both
sides (wall clock) and by HIP events recorded on the stream the kernels are launched on (kernel time).
The defaults (W = 50, K = 200) time the kernels in the sustained regime: under bf16 MFMA load on random
data the chip settles at a lower clock than it starts with (and a cold chip ramps up), so a handful of
steps measures neither.  Every workload carries a `cpu_baseline`: the C restatement of the reference's
CPU path (oracle/) timed on the host cores of the same box, on a bounded sample that is stated with it;
a reported baseline, never part of `value`.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Published MI355X peaks the roofline fractions are priced against.
PEAK_TFLOPS = {"f32": 157.3, "bf16": 2500.0}
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch; FETCH_SIZE
# scaled x2.0 and WRITE_SIZE x1.0, the factors a streaming kernel of known size gives on this chip).  The
# summaries live in profiles/dominant_kernels_counters.md; workloads not listed there report null.
MEASURED_TRAFFIC_BYTES = {
    "conv2d_bias_relu_f32_n32_c64to128_56x56_k3s1p1": (14291 * 2 + 50176) * 1024,
    "conv2d_grad_input_f32_n32_c64to128_56x56_k3s1p1": ((32964 + 660) * 2 + 25088 + 288) * 1024,
    "conv2d_grad_weight_f32_n32_c64to128_56x56_k3s1p1": ((44170 + 36161) * 2 + 72288 + 288) * 1024,
    "gemm_bf16_f32acc_4096x4096x4096": (98511 * 2 + 65536) * 1024,
    "gemm_bf16_f32acc_4096x4096x4096_prepacked_rhs": (98406 * 2 + 65536) * 1024,
    "gemm_bf16_f32acc_16x4096x4096": ((16927 + 1045) * 2 + 2048 + 256) * 1024,
    "gemm_bf16_f32acc_16x4096x4096_prepacked_rhs": (16924 * 2 + 256) * 1024,
    "attention_f32_b8_h16_s2048_d64_noncausal": (98379 * 2 + 65536) * 1024,
    "attention_f32_b8_h16_s2048_d64_causal": (138815 * 2 + 65537) * 1024,
    "attention_f32_attn_bias_c1_s2048_d64": ((10840 + 4260) * 2 + 8448 + 512) * 1024,
    "attention_f32_attn_bias_c16_s1024_d64": ((49240 + 8484) * 2 + 16896 + 4096) * 1024,
    "gemm_f32_100352x128x576_conv_equivalent": (136982 * 2 + 50176) * 1024,
    "gemm_f32_4096x4096x4096": (196708 * 2 + 65536) * 1024,
    "gemm_f32_512x512x512": (4646 * 2 + 1024) * 1024,
    "attention_bf16_b16_h8_s1024_d64_causal": (25124 * 2 + 16384) * 1024,
    "layer_norm_f32_to_bf16_16384x512": (16432 * 2 + 16384) * 1024,
    "row_softmax_f32_16384x512": (16408 * 2 + 32768) * 1024,
    "gelu_backward_f32_16384x512": (32788 * 2 + 32768) * 1024,
    "scale_f32_16384x512": (16394 * 2 + 32768) * 1024,
    "sum_axis0_f32_16384x512": ((16401 + 527) * 2 + 512 + 2) * 1024,
}


def log(*items):
    print(*items, file=sys.stderr, flush=True)


class Timer:
    def __init__(self, hip):
        self.hip = hip
        self.stream = hip.Stream()
        self.start, self.stop = hip.Event(), hip.Event()

    def run(self, step, warmup, steps):
        """Returns (wall ms per step, event ms per step)."""
        for _ in range(warmup):
            step(self.stream)
        self.stream.synchronize()
        self.hip.device_synchronize()
        self.start.record(self.stream)
        t0 = time.perf_counter()
        for _ in range(steps):
            step(self.stream)
        self.stop.record(self.stream)
        self.stream.synchronize()
        self.hip.device_synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / steps
        return wall, self.start.elapsed_ms(self.stop) / steps


def roofline(bound, dtype, flops, bytes_, ms):
    if bound == "mfma":
        achieved = flops / (ms * 1e-3) / 1e12
        peak = PEAK_TFLOPS[dtype]
        return {"bound": "mfma", "achieved": round(achieved, 3), "peak": peak, "unit": "TFLOP/s",
                "frac": round(achieved / peak, 4), "traffic": None}
    achieved = bytes_ / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(achieved / PEAK_HBM_GBS, 4), "traffic": None}


def entry(name, dtype, flops, bytes_, bound, wall_ms, event_ms, extra=None):
    out = {"workload": name, "dtype": dtype, "flops_per_step": flops, "min_bytes_per_step": bytes_,
           "ms_per_step": round(wall_ms, 5), "kernel_ms_per_step": round(event_ms, 5),
           "gflops": round(flops / (wall_ms * 1e-3) / 1e9, 1),
           "roofline": roofline(bound, "bf16" if dtype == "bf16" else "f32", flops, bytes_, event_ms)}
    out["roofline"]["traffic"] = MEASURED_TRAFFIC_BYTES.get(name)
    if extra:
        out.update(extra)
    return out


# ---- workloads (BASELINE.json configs) ---------------------------------------------------------------

def wl_conv2d(hip, inputs, timer, warmup, steps):
    batch, c_in, h, w, c_out = 32, 64, 56, 56, 128
    x = inputs.normal(inputs.seed_for(2, 0), batch * c_in * h * w)
    wt = inputs.normal(inputs.seed_for(2, 1), c_out * c_in * 9, 0.0, math.sqrt(2.0 / (c_in * 9)))
    b = inputs.uniform(inputs.seed_for(2, 2), c_out, -0.1, 0.1)
    d_x, d_w, d_b = (hip.DeviceBuffer.from_array(a) for a in (x, wt, b))
    d_out = hip.DeviceBuffer(batch * c_out * h * w * 4)
    geom = ((3, 3), (1, 1), (1, 1), (1, 1))

    def step(stream):
        hip.conv2d_bias_act_f32_dev(batch, c_in, h, w, c_out, *geom, 1, d_x, d_w, d_b, d_out, stream)

    wall, ev = timer.run(step, warmup, steps)
    flops = 2 * batch * c_out * h * w * c_in * 9
    bytes_ = 4 * (x.size + wt.size + b.size + batch * c_out * h * w)
    return entry("conv2d_bias_relu_f32_n32_c64to128_56x56_k3s1p1", "f32", flops, bytes_, "mfma", wall, ev), \
        (x, wt, b, geom, (batch, c_in, h, w, c_out))


def wl_conv2d_backward(hip, inputs, timer, warmup, steps, which):
    """Gradients of config 2's convolution: grad_input (adjoint convolution) or grad_weight (reduction over
    batch and pixels); both cost the forward's FLOPs."""
    batch, c_in, h, w, c_out = 32, 64, 56, 56, 128
    x = inputs.normal(inputs.seed_for(2, 0), batch * c_in * h * w)
    wt = inputs.normal(inputs.seed_for(2, 1), c_out * c_in * 9, 0.0, math.sqrt(2.0 / (c_in * 9)))
    g = inputs.normal(inputs.seed_for(2, 3), batch * c_out * h * w)
    d_x, d_w, d_g = (hip.DeviceBuffer.from_array(a) for a in (x, wt, g))
    geom = ((3, 3), (1, 1), (1, 1), (1, 1))
    if which == "grad_input":
        d_out = hip.DeviceBuffer(x.nbytes)
        step = lambda stream: hip.conv2d_grad_input_f32_dev(batch, c_in, h, w, c_out, *geom, d_g, d_w, d_out, stream)
        bytes_ = 4 * (g.size + wt.size + x.size)
    else:
        d_out = hip.DeviceBuffer(wt.nbytes)
        step = lambda stream: hip.conv2d_grad_weight_f32_dev(batch, c_in, h, w, c_out, *geom, d_x, d_g, 1.0 / batch,
                                                             d_out, stream)
        bytes_ = 4 * (g.size + wt.size + x.size)
    wall, ev = timer.run(step, warmup, steps)
    flops = 2 * batch * c_out * h * w * c_in * 9
    return entry(f"conv2d_{which}_f32_n32_c64to128_56x56_k3s1p1", "f32", flops, bytes_, "mfma", wall, ev)


def wl_gemm_f32(hip, inputs, timer, warmup, steps, m, n, k, name):
    a = inputs.uniform(inputs.seed_for(1, 0), m * k, -1.0, 1.0)
    b = inputs.uniform(inputs.seed_for(1, 1), k * n, -1.0, 1.0)
    d_a, d_b = hip.DeviceBuffer.from_array(a), hip.DeviceBuffer.from_array(b)
    d_c = hip.DeviceBuffer(m * n * 4)

    def step(stream):
        hip.gemm_f32_dev(m, n, k, 1.0, False, d_a, d_b, d_c, stream)

    wall, ev = timer.run(step, warmup, steps)
    return entry(name, "f32", 2 * m * n * k, 4 * (m * k + k * n + m * n), "mfma", wall, ev)


def wl_gemm_bf16(hip, inputs, timer, warmup, steps, m, n, k, name, bound, packed=False):
    """bf16 operands, f32 accumulation and output.  `packed`: B handed over as its (n, k) transpose (PackedB's
    layout), packed once outside the timed region as a weight would be.

    The HBM-bound (skinny) shapes cycle through ten copies of B, 320 MiB in all: a single 32 MiB B stays in the
    256 MiB memory-side cache from one launch to the next, and a loop over it measures that cache, not HBM (a decode
    loop reads a different weight matrix with every GEMM).  The cache-resident time is reported beside it."""
    a = inputs.to_bf16(inputs.normal(inputs.seed_for(4, 0 if m == n else 2), m * k, 0.0, 0.02))
    b = inputs.to_bf16(inputs.normal(inputs.seed_for(4, 1), k * n, 0.0, 0.02))
    d_a = hip.DeviceBuffer.from_array(a)
    d_c = hip.DeviceBuffer(m * n * 4)
    copies = 10 if bound == "hbm" else 1
    if packed:
        d_b = hip.DeviceBuffer.from_array(b)
        rhs = []
        for _ in range(copies):
            rhs.append(hip.DeviceBuffer(k * n * 2))
            hip.pack_rhs_bf16_dev(k, n, d_b, rhs[-1])
        hip.device_synchronize()
    else:
        rhs = [hip.DeviceBuffer.from_array(b) for _ in range(copies)]
    turn = [0]

    def step(stream, rotate=True):
        d_rhs = rhs[turn[0] % copies if rotate else 0]
        turn[0] += 1
        if packed:
            hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, 0, d_a, d_rhs, None, None, d_c, None, stream)
        else:
            hip.gemm_bf16_f32acc_dev(m, n, k, d_a, d_rhs, d_c, stream)

    wall, ev = timer.run(step, warmup, steps)
    extra = None
    if copies > 1:
        _, resident = timer.run(lambda stream: step(stream, rotate=False), warmup, steps)
        extra = {"rhs_copies_cycled": copies, "kernel_ms_per_step_rhs_cache_resident": round(resident, 5)}
    return entry(name, "bf16", 2 * m * n * k, 2 * (m * k + k * n) + 4 * m * n, bound, wall, ev, extra)


def wl_attention(hip, inputs, timer, warmup, steps, causal):
    contexts, seq, dim = 128, 2048, 64
    count = contexts * seq * dim
    q, k, v = (inputs.normal(inputs.seed_for(3, i), count) for i in range(3))
    d_q, d_k, d_v = (hip.DeviceBuffer.from_array(a) for a in (q, k, v))
    d_o = hip.DeviceBuffer(count * 4)

    def step(stream):
        hip.attention_f32_dev(contexts, seq, dim, 0.125, causal, d_q, d_k, d_v, None, None, d_o, stream)

    wall, ev = timer.run(step, warmup, steps)
    flops = 4 * dim * contexts * (seq * (seq + 1) // 2 if causal else seq * seq)
    name = "attention_f32_b8_h16_s2048_d64_" + ("causal" if causal else "noncausal")
    return entry(name, "f32", flops, 4 * 4 * count, "mfma", wall, ev)


def wl_attention_bias(hip, inputs, timer, warmup, steps, contexts, seq):
    """Attention with a per-query bias matrix, the form the reference's only in-tree Rust caller uses (one context
    per head with an attn_bias kernel matrix, crates/st-nn/src/z_rba/attention.rs:586-595): general kernel."""
    dim = 64
    count = contexts * seq * dim
    q, k, v = (inputs.normal(inputs.seed_for(3, i), count) for i in range(3))
    bias = inputs.normal(inputs.seed_for(3, 5), contexts * seq * seq, 0.0, 0.5)
    d_q, d_k, d_v, d_b = (hip.DeviceBuffer.from_array(a) for a in (q, k, v, bias))
    d_o = hip.DeviceBuffer(count * 4)

    def step(stream):
        hip.attention_f32_dev(contexts, seq, dim, 0.125, False, d_q, d_k, d_v, None, d_b, d_o, stream)

    wall, ev = timer.run(step, warmup, steps)
    flops = 4 * dim * contexts * seq * seq
    return entry(f"attention_f32_attn_bias_c{contexts}_s{seq}_d64", "f32", flops, 4 * (4 * count + bias.size), "mfma",
                 wall, ev)


def wl_attention_bf16(hip, inputs, timer, warmup, steps):
    """The decoder's attention on its own: batch 16, 8 heads, seq 1024, head_dim 64, causal, bf16 operands read
    in place from a fused (tokens, 3*512) projection."""
    batch, heads, seq, dim = 16, 8, 1024, 64
    width = heads * dim
    qkv = inputs.to_bf16(inputs.normal(inputs.seed_for(5, 2), batch * seq * 3 * width))
    d_qkv = hip.DeviceBuffer.from_array(qkv)
    d_out = hip.DeviceBuffer(batch * seq * width * 2)

    def step(stream):
        hip.attention_bf16_dev(batch, heads, seq, dim, 0.125, True, d_qkv, d_qkv.at(width * 2), d_qkv.at(width * 4),
                               3 * width, d_out, width, stream)

    wall, ev = timer.run(step, warmup, steps)
    flops = 4 * dim * batch * heads * (seq * (seq + 1) // 2)
    return entry("attention_bf16_b16_h8_s1024_d64_causal", "bf16", flops, 2 * 4 * batch * seq * width, "mfma", wall, ev)


def wl_decoder(hip, inputs, timer, warmup, steps):
    vocab, d, heads, layers, ff, batch, seq = 256, 512, 8, 6, 2048, 16, 1024
    count = hip.Decoder.weight_count(vocab, d, heads, layers, ff)
    weights = inputs.normal(inputs.seed_for(5, 0), count, 0.0, 0.02)
    tokens = inputs.tokens(inputs.seed_for(5, 1), batch * seq, vocab)
    dec = hip.Decoder(vocab, d, heads, layers, ff, batch, seq, 1e-5, weights)
    d_tok = hip.DeviceBuffer.from_array(tokens)
    d_logits = hip.DeviceBuffer(batch * seq * vocab * 4)

    def step(stream):
        dec.forward_dev(d_tok, d_logits, stream)

    wall, ev = timer.run(step, warmup, steps)
    T = batch * seq
    hd = d // heads
    per_layer = 3 * 2 * T * d * d + 2 * T * d * d + 4 * hd * batch * heads * (seq * (seq + 1) // 2) + 2 * 2 * T * d * ff
    flops = layers * per_layer + 2 * T * d * vocab
    out = entry("decoder_bf16_v256_d512_h8_l6_ff2048_b16_s1024", "bf16", flops, 0, "mfma", wall, ev,
                {"tokens_per_s": round(T / (wall * 1e-3), 1)})
    dec.destroy()
    return out


def wl_rowops(hip, inputs, timer, warmup, steps):
    """HBM-bound tensor utilities at the decoder's activation shape (16384 x 512 f32, 32 MiB): bytes are the
    algorithmic reads + writes of each op."""
    rows, cols = 16384, 512
    n = rows * cols
    x = inputs.normal(inputs.seed_for(5, 3), n)
    d_x, d_y = hip.DeviceBuffer.from_array(x), hip.DeviceBuffer(n * 4)
    d_g = hip.DeviceBuffer.from_array(inputs.normal(inputs.seed_for(5, 4), n))
    ones = hip.DeviceBuffer.from_array(np.ones(cols, np.float32))
    d_16, d_cols = hip.DeviceBuffer(n * 2), hip.DeviceBuffer(cols * 4)
    ops = [
        ("layer_norm_f32_to_bf16", 6 * n, lambda st: hip.layer_norm_f32_dev(rows, cols, d_x, None, ones, ones, 1e-5, None, d_16, st)),
        ("row_softmax_f32", 8 * n, lambda st: hip.row_softmax_f32_dev(rows, cols, d_x, d_y, st)),
        ("gelu_backward_f32", 12 * n, lambda st: hip.gelu_backward_f32_dev(n, d_x, d_g, d_y, st)),
        ("scale_f32", 8 * n, lambda st: hip.scale_f32_dev(n, d_x, 0.5, d_y, st)),
        ("sum_axis0_f32", 4 * n, lambda st: hip.sum_axis0_f32_dev(rows, cols, d_x, 1.0, d_cols, st)),
    ]
    out = []
    for name, bytes_, step in ops:
        wall, ev = timer.run(step, warmup, steps)
        out.append(entry(f"{name}_16384x512", "f32", 0, bytes_, "hbm", wall, ev))
    return out


def wl_lopsided(hip, inputs, timer, warmup, steps):
    """Shapes outside the BASELINE configs whose dispatch has kernels of its own: matrix x vector (a stream over A: the
    f32 matrix is 1 GiB, the bf16 one 512 MiB, both beyond the 256 MiB memory-side cache), a product of few output tiles
    with a long k (k-sliced over workgroups), softmax over rows of 100000 values (each row cut into segments over the grid), and thousands
    of short attention windows.  All HBM-bound; bytes are the algorithmic reads + writes."""
    out = []
    m = k = 16384
    d_a = hip.DeviceBuffer(m * k * 4)
    d_a.zero()
    d_x = hip.DeviceBuffer.from_array(inputs.uniform(inputs.seed_for(1, 2), k, -1.0, 1.0))
    d_y = hip.DeviceBuffer(m * 4)
    wall, ev = timer.run(lambda st: hip.gemm_f32_dev(m, 1, k, 1.0, False, d_a, d_x, d_y, st), warmup, steps)
    out.append(entry(f"gemv_f32_{m}x1x{k}", "f32", 2 * m * k, 4 * (m * k + k + m), "hbm", wall, ev))
    d_x16 = hip.DeviceBuffer.from_array(inputs.to_bf16(inputs.uniform(inputs.seed_for(1, 2), k, -1.0, 1.0)))
    wall, ev = timer.run(lambda st: hip.gemm_bf16_f32acc_dev(m, 1, k, d_a, d_x16, d_y, st), warmup, steps)
    out.append(entry(f"gemv_bf16_{m}x1x{k}", "bf16", 2 * m * k, 2 * (m * k + k) + 4 * m, "hbm", wall, ev))
    # the same stored matrix read as k x m: A^T x, the gradient of the product above with respect to x
    wall, ev = timer.run(lambda st: hip.gemm_f32_dev(m, 1, k, 1.0, True, d_a, d_x, d_y, st), warmup, steps)
    out.append(entry(f"gemv_f32_lhs_transposed_{m}x1x{k}", "f32", 2 * m * k, 4 * (m * k + k + m), "hbm", wall, ev))
    m2, n2, k2 = 64, 64, 100000
    d_c = hip.DeviceBuffer(m2 * n2 * 4)
    wall, ev = timer.run(lambda st: hip.gemm_f32_dev(m2, n2, k2, 1.0, False, d_a, d_a, d_c, st), warmup, steps)
    out.append(entry(f"gemm_f32_{m2}x{n2}x{k2}_k_sliced", "f32", 2 * m2 * n2 * k2, 4 * (m2 * k2 + k2 * n2 + m2 * n2), "hbm", wall, ev))
    rows, cols = 100, 100000
    d_in = hip.DeviceBuffer.from_array(inputs.normal(inputs.seed_for(5, 5), rows * cols))
    d_out = hip.DeviceBuffer(rows * cols * 4)
    wall, ev = timer.run(lambda st: hip.row_softmax_f32_dev(rows, cols, d_in, d_out, st), warmup, steps)
    out.append(entry(f"row_softmax_f32_{rows}x{cols}", "f32", 0, 8 * rows * cols, "hbm", wall, ev))
    # windowed attention: 16384 contexts of 16 positions, head size 64 (a wavefront per context)
    ctx, seq, dim = 16384, 16, 64
    n = ctx * seq * dim
    d_q, d_o = hip.DeviceBuffer(n * 4), hip.DeviceBuffer(n * 4)
    d_q.zero()
    wall, ev = timer.run(lambda st: hip.attention_f32_dev(ctx, seq, dim, 0.125, False, d_q, d_q, d_q, None, None, d_o, st),
                         warmup, steps)
    out.append(entry(f"attention_f32_{ctx}_windows_of_{seq}x{dim}", "f32", 4 * ctx * seq * seq * dim, 16 * n, "hbm", wall, ev))
    return out


def wl_calibration(hip, inputs, timer, warmup, steps):
    """Plain streaming kernel of known traffic (f32 -> bf16 rounding of 64 Mi values: 256 MiB read, 128 MiB
    written).  It anchors the FETCH_SIZE / WRITE_SIZE counters and shows the HBM rate a trivial kernel reaches."""
    count = 64 * 1024 * 1024
    d_src = hip.DeviceBuffer(count * 4)
    d_src.zero()
    d_dst = hip.DeviceBuffer(count * 2)

    def step(stream):
        hip.f32_to_bf16_dev(count, d_src, d_dst, stream)

    wall, ev = timer.run(step, warmup, steps)
    return entry("calibration_f32_to_bf16_64mi", "f32", 0, count * 6, "hbm", wall, ev)


# ---- CPU baselines: the C restatement of the reference's CPU path, timed on the host cores of this box ------------

def _cpu(flops, seconds, cores, sample):
    return {"value": round(flops / seconds / 1e9, 3), "unit": "GFLOP/s", "cores": cores, "kind": "port", "sample": sample}


def cpu_baseline_conv(conv_inputs, passes=5):
    """Conv2d::forward_cpu, single-threaded as the reference's contraction is (conv.rs:297-323), on full passes
    of config 2; the median pass is reported."""
    from oracle import oracle
    x, wt, b, geom, (batch, c_in, h, w, c_out) = conv_inputs
    seconds = []
    for _ in range(passes):
        t0 = time.perf_counter()
        oracle.conv2d_bias_act_f32(batch, c_in, h, w, c_out, *geom, oracle.ACT_RELU, x, wt, b, threads=1)
        seconds.append(time.perf_counter() - t0)
    median = sorted(seconds)[len(seconds) // 2]
    return _cpu(2 * batch * c_out * h * w * c_in * 9, median, 1,
                f"{passes} full passes of config 2 ({batch} images each), single thread, {sum(seconds):.1f} s in all, "
                f"median pass {median:.2f} s; host has {os.cpu_count()} logical CPUs")


def cpu_baselines(inputs):
    """One bounded sample per remaining configuration; returns {workload name: cpu_baseline}."""
    from oracle import oracle
    cores = min(16, os.cpu_count() or 1)
    out = {}

    def timed(fn, repeat=1):
        best = None
        for _ in range(repeat):
            t0 = time.perf_counter()
            fn()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        return best

    # config 1: all cores over row tiles, as rayon does in cpu_dense.rs:226-236
    a = inputs.uniform(inputs.seed_for(1, 0), 512 * 512, -1.0, 1.0)
    b = inputs.uniform(inputs.seed_for(1, 1), 512 * 512, -1.0, 1.0)
    sec = timed(lambda: oracle.gemm_f32(512, 512, 512, a, b, threads=cores), repeat=20)
    out["gemm_f32_512x512x512"] = _cpu(2 * 512 ** 3, sec, cores, f"full 512^3, best of 20 passes, {cores} threads over row tiles")
    # config 3: single thread as fused_attention_cpu is (pure.rs:11860-11916); 2 of 128 contexts, scaled
    q, k, v = (inputs.normal(inputs.seed_for(3, i), 2 * 2048 * 64) for i in range(3))
    for causal in (False, True):
        sec = timed(lambda: oracle.attention_f32(2, 2048, 64, 0.125, q, k, v, causal=causal))
        flops = 4 * 64 * 2 * (2048 * 2049 // 2 if causal else 2048 * 2048)
        out["attention_f32_b8_h16_s2048_d64_" + ("causal" if causal else "noncausal")] = _cpu(
            flops, sec, 1, f"2 of 128 contexts, single thread, {sec:.2f} s (the full config would take {sec * 64:.0f} s)")
    # config 4: all cores over rows; 128 of 4096 rows of A for the square shape, the whole skinny shape
    a16 = inputs.to_bf16(inputs.normal(inputs.seed_for(4, 0), 128 * 4096, 0.0, 0.02))
    b16 = inputs.to_bf16(inputs.normal(inputs.seed_for(4, 1), 4096 * 4096, 0.0, 0.02))
    sec = timed(lambda: oracle.gemm_bf16_f32acc(128, 4096, 4096, a16, b16, threads=cores), repeat=3)
    square = _cpu(2 * 128 * 4096 * 4096, sec, cores, f"128 of 4096 rows of A, best of 3, {cores} threads ({sec:.2f} s; full: {sec * 32:.0f} s)")
    out["gemm_bf16_f32acc_4096x4096x4096"] = square
    out["gemm_bf16_f32acc_4096x4096x4096_prepacked_rhs"] = square
    sec = timed(lambda: oracle.gemm_bf16_f32acc(16, 4096, 4096, a16[:16 * 4096], b16, threads=cores), repeat=5)
    out["gemm_bf16_f32acc_16x4096x4096"] = _cpu(2 * 16 * 4096 * 4096, sec, cores, f"full shape, best of 5, {cores} threads")
    out["gemm_bf16_f32acc_16x4096x4096_prepacked_rhs"] = out["gemm_bf16_f32acc_16x4096x4096"]
    # matrix x vector: 2048 of the 16384 rows, all cores over rows
    av = inputs.uniform(inputs.seed_for(1, 3), 2048 * 16384, -1.0, 1.0)
    xv = inputs.uniform(inputs.seed_for(1, 2), 16384, -1.0, 1.0)
    sec = timed(lambda: oracle.gemm_f32(2048, 1, 16384, av, xv, threads=cores), repeat=3)
    out["gemv_f32_16384x1x16384"] = _cpu(2 * 2048 * 16384, sec, cores, f"2048 of 16384 rows, best of 3, {cores} threads")
    # config 5: one layer (+ embedding, final norm, head) on one of 16 sequences, single thread, scaled
    vocab, d, heads, ff, seq = 256, 512, 8, 2048, 1024
    weights = inputs.normal(inputs.seed_for(5, 0), oracle.decoder_weight_count(vocab, d, heads, 1, ff), 0.0, 0.02)
    tokens = inputs.tokens(inputs.seed_for(5, 1), seq, vocab)
    sec = timed(lambda: oracle.decoder_forward(vocab, d, heads, 1, ff, 1, seq, 1e-5, weights, tokens))
    hd = d // heads
    layer = 3 * 2 * seq * d * d + 2 * seq * d * d + 4 * hd * heads * (seq * (seq + 1) // 2) + 2 * 2 * seq * d * ff
    out["decoder_bf16_v256_d512_h8_l6_ff2048_b16_s1024"] = _cpu(
        layer + 2 * seq * d * vocab, sec, 1,
        f"1 of 6 layers on 1 of 16 sequences, single thread, {sec:.2f} s (the full config would take about {sec * 96:.0f} s)")
    return out


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=200)
    parser.add_argument("--warmup", type=int, default=50)
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--only", default=None, help="run only the headline plus workloads whose name contains this")
    args = parser.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (every op shards into independent "
              "units: GEMM by row blocks, conv by image, attention by context, the decoder by batch). "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    from spiraltorch_amd import hip, inputs
    hip.init()  # raises when libsthip.so or the device is missing: there is no fallback to measure
    props = hip.device_properties(0)
    log("device:", props)
    timer = Timer(hip)

    headline, conv_inputs = wl_conv2d(hip, inputs, timer, args.warmup, args.steps)
    log(json.dumps(headline))
    others = []
    # Side workloads: the same sustained protocol, scaled down for the kernels that last a millisecond.
    warm, steps = max(2, min(args.warmup, 50)), max(5, min(args.steps, 200))
    long_warm, long_steps = max(2, warm // 5), max(5, steps // 5)
    plan = [
        ("conv2d_grad_input", lambda: wl_conv2d_backward(hip, inputs, timer, warm, steps, "grad_input")),
        ("conv2d_grad_weight", lambda: wl_conv2d_backward(hip, inputs, timer, warm, steps, "grad_weight")),
        ("gemm_f32_512", lambda: wl_gemm_f32(hip, inputs, timer, warm, steps, 512, 512, 512, "gemm_f32_512x512x512")),
        ("gemm_f32_4096", lambda: wl_gemm_f32(hip, inputs, timer, long_warm, long_steps, 4096, 4096, 4096,
                                               "gemm_f32_4096x4096x4096")),
        ("gemm_f32_conv_equivalent", lambda: wl_gemm_f32(hip, inputs, timer, warm, steps, 100352, 128, 576,
                                                         "gemm_f32_100352x128x576_conv_equivalent")),
        ("gemm_bf16_4096", lambda: wl_gemm_bf16(hip, inputs, timer, warm, steps, 4096, 4096, 4096,
                                                "gemm_bf16_f32acc_4096x4096x4096", "mfma")),
        ("gemm_bf16_4096_prepacked", lambda: wl_gemm_bf16(hip, inputs, timer, warm, steps, 4096, 4096, 4096,
                                                          "gemm_bf16_f32acc_4096x4096x4096_prepacked_rhs", "mfma", True)),
        ("gemm_bf16_skinny", lambda: wl_gemm_bf16(hip, inputs, timer, warm, steps, 16, 4096, 4096,
                                                  "gemm_bf16_f32acc_16x4096x4096", "hbm")),
        ("gemm_bf16_skinny_prepacked", lambda: wl_gemm_bf16(hip, inputs, timer, warm, steps, 16, 4096, 4096,
                                                            "gemm_bf16_f32acc_16x4096x4096_prepacked_rhs", "hbm", True)),
        ("attention_noncausal", lambda: wl_attention(hip, inputs, timer, long_warm, long_steps, False)),
        ("attention_causal", lambda: wl_attention(hip, inputs, timer, long_warm, long_steps, True)),
        ("attention_bias", lambda: [wl_attention_bias(hip, inputs, timer, warm, steps, 1, 2048),
                                    wl_attention_bias(hip, inputs, timer, long_warm, long_steps, 16, 1024)]),
        ("attention_bf16", lambda: wl_attention_bf16(hip, inputs, timer, warm, steps)),
        ("decoder", lambda: wl_decoder(hip, inputs, timer, long_warm, long_steps)),
        ("rowops", lambda: wl_rowops(hip, inputs, timer, warm, steps)),
        ("lopsided", lambda: wl_lopsided(hip, inputs, timer, long_warm, long_steps)),
        ("calibration", lambda: wl_calibration(hip, inputs, timer, long_warm, long_steps)),
    ]
    for name, fn in plan:
        if args.only and args.only not in name:
            continue
        result = fn()
        for item in (result if isinstance(result, list) else [result]):
            others.append(item)

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline_conv(conv_inputs)
        log(json.dumps(cpu))
        per_workload = cpu_baselines(inputs)
        for item in others:
            if item["workload"] in per_workload:
                item["cpu_baseline"] = per_workload[item["workload"]]
            elif item["workload"].startswith("conv2d_grad"):
                item["cpu_baseline"] = dict(cpu, sample="the forward pass of the same layer (the reference's backward runs "
                                                         "the same contraction sizes): " + cpu["sample"])
    for item in others:
        log(json.dumps(item))

    line = {
        "metric": "GFLOP/s and % of MFMA roofline (GEMM, conv, attention) on 1 MI355X; value = fused conv2d+bias+ReLU",
        "value": headline["gflops"],
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": headline["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": headline["workload"], "batch": 32, "c_in": 64, "c_out": 128, "hw": 56, "kernel": 3,
                   "resident": "HBM"},
        "roofline": headline["roofline"],
        "cpu_baseline": cpu,
        "device": {"arch": props["arch"], "compute_units": props["compute_units"], "clock_khz": props["clock_khz"]},
        "workloads": others,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
