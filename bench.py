#!/usr/bin/env python3
"""Benchmark of the HIP hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-sustained] [--only NAME] [--all] [--probes]

A "step" is one pass of the headline workload over one batch of synthetic input that is already
resident in HBM: BASELINE config 2, the fused conv2d + bias + ReLU (f32, N32 C64->128 56x56 3x3 s1 p1).
The single JSON line printed at the end (kept well below 16 KB) carries that workload as `value` and one
compact row per other BASELINE configuration (f32 GEMM 512^3, bf16 GEMM 4096^3 and 16x4096x4096,
attention S2048 causal and non-causal, the decoder stack, and the backward / biased forms of the same
kernels) under `workloads`, each with its own roofline figures and CPU baseline.  `--all` adds the
workloads that are no BASELINE configuration (row utilities, lopsided shapes, the counter calibration
stream); those are printed as JSON lines on stderr only.

Timing: W untimed warm-up steps, then exactly K steps bracketed by a device synchronisation on both
sides (wall clock) and by HIP events recorded on the stream the kernels are launched on (kernel time).
That first measurement, at the W and K given, is what `value`, `ms_per_step` and every row's `roofline`
report.  A cold chip ramps its clock up and, under bf16 MFMA load on random data, then settles lower, so
a handful of steps and a long loop measure different regimes: every workload is therefore timed a second
time with 50 warm-up + 200 timed steps (10 + 40 for the kernels that last a millisecond) and that figure
is reported beside the first under `sustained`.  Every workload carries a `cpu_baseline`: the C
restatement of the reference's CPU path (oracle/) timed on the host cores of the same box, on a bounded
sample that is stated with it; a reported baseline, never part of `value`.
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
    "conv2d_grad_weight_f32_n32_c64to128_56x56_k3s1p1": ((44801 + 12109) * 2 + 24192 + 288) * 1024,
    "conv2d_bias_relu_bf16_f32acc_n32_c64to128_56x56_k3s1p1": ((12703 + 8123) * 2 + 13600 + 50176) * 1024,
    "gemm_bf16_f32acc_4096x4096x4096": (98511 * 2 + 65536) * 1024,
    "gemm_bf16_f32acc_4096x4096x4096_prepacked_rhs": (98406 * 2 + 65536) * 1024,
    "gemm_bf16_f32acc_16x4096x4096": ((16927 + 1045) * 2 + 2048 + 256) * 1024,
    "gemm_bf16_f32acc_16x4096x4096_prepacked_rhs": (16924 * 2 + 256) * 1024,
    "attention_f32_b8_h16_s2048_d64_noncausal": (98379 * 2 + 65536) * 1024,
    "attention_f32_b8_h16_s2048_d64_causal": (134572 * 2 + 65547) * 1024,
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


SUSTAINED_WARMUP, SUSTAINED_STEPS = 50, 200


class Timer:
    """Times a step function under two protocols: the one asked for on the command line (W warm-up steps, K timed
    steps) and the sustained one (50 + 200; a fifth of both for workloads flagged `long`, whose steps last about a
    millisecond)."""

    def __init__(self, hip, warmup, steps, sustained=True):
        self.hip = hip
        self.stream = hip.Stream()
        self.start, self.stop = hip.Event(), hip.Event()
        self.warmup, self.steps, self.sustained = warmup, steps, sustained

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

    def protocols(self, long, headline=False):
        """((warmup, steps) as asked, (warmup, steps) sustained).  The headline runs exactly the W and K given; side
        workloads cap them at the sustained protocol's, and `long` ones take a fifth once K exceeds 40."""
        if headline:
            first = (self.warmup, self.steps)
        else:
            first = (max(2, min(self.warmup, SUSTAINED_WARMUP)), max(5, min(self.steps, SUSTAINED_STEPS)))
            if long and first[1] > 40:
                first = (max(2, first[0] // 5), first[1] // 5)
        second = (SUSTAINED_WARMUP // 5, SUSTAINED_STEPS // 5) if long else (SUSTAINED_WARMUP, SUSTAINED_STEPS)
        return first, second

    def measure(self, step, long=False, headline=False):
        """Returns (wall ms, event ms, sustained) where sustained = {"warmup", "steps", "kernel_ms_per_step"}: the
        second protocol's figure, measured after the first (the same numbers when the two protocols coincide)."""
        first, second = self.protocols(long, headline)
        wall, ev = self.run(step, *first)
        if not self.sustained:
            return wall, ev, None
        ev2 = ev if first == second else self.run(step, *second)[1]
        return wall, ev, {"warmup": second[0], "steps": second[1], "kernel_ms_per_step": round(ev2, 5)}


def roofline(bound, dtype, flops, bytes_, ms):
    if bound == "mfma":
        achieved = flops / (ms * 1e-3) / 1e12
        peak = PEAK_TFLOPS[dtype]
        return {"bound": "mfma", "achieved": round(achieved, 3), "peak": peak, "unit": "TFLOP/s",
                "frac": round(achieved / peak, 4), "traffic": None}
    achieved = bytes_ / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(achieved / PEAK_HBM_GBS, 4), "traffic": None}


def entry(name, dtype, flops, bytes_, bound, wall_ms, event_ms, extra=None, sustained=None):
    kind = "bf16" if dtype == "bf16" else "f32"
    out = {"workload": name, "dtype": dtype, "flops_per_step": flops, "min_bytes_per_step": bytes_,
           "ms_per_step": round(wall_ms, 5), "kernel_ms_per_step": round(event_ms, 5),
           "gflops": round(flops / (wall_ms * 1e-3) / 1e9, 1),
           "roofline": roofline(bound, kind, flops, bytes_, event_ms)}
    out["roofline"]["traffic"] = MEASURED_TRAFFIC_BYTES.get(name)
    if sustained:
        again = roofline(bound, kind, flops, bytes_, sustained["kernel_ms_per_step"])
        out["sustained"] = dict(sustained, achieved=again["achieved"], frac=again["frac"])
    if extra:
        out.update(extra)
    return out


def compact(item):
    """The row of the final JSON line for one workload: what identifies it, its time, its roofline object, the
    sustained figure and the CPU baseline; the per-step flop and byte counts stay on the stderr lines."""
    row = {"workload": item["workload"], "dtype": item["dtype"], "kernel_ms_per_step": item["kernel_ms_per_step"],
           "gflops": item["gflops"], "roofline": item["roofline"]}
    if "sustained" in item:
        row["sustained"] = {"kernel_ms_per_step": item["sustained"]["kernel_ms_per_step"], "frac": item["sustained"]["frac"]}
    for key in ("tokens_per_s", "kernel_ms_per_step_rhs_cache_resident", "cpu_baseline"):
        if key in item:
            row[key] = item[key]
    return row


# ---- workloads (BASELINE.json configs) ---------------------------------------------------------------

def wl_conv2d(hip, inputs, timer):
    batch, c_in, h, w, c_out = 32, 64, 56, 56, 128
    x = inputs.normal(inputs.seed_for(2, 0), batch * c_in * h * w)
    wt = inputs.normal(inputs.seed_for(2, 1), c_out * c_in * 9, 0.0, math.sqrt(2.0 / (c_in * 9)))
    b = inputs.uniform(inputs.seed_for(2, 2), c_out, -0.1, 0.1)
    d_x, d_w, d_b = (hip.DeviceBuffer.from_array(a) for a in (x, wt, b))
    d_out = hip.DeviceBuffer(batch * c_out * h * w * 4)
    geom = ((3, 3), (1, 1), (1, 1), (1, 1))

    def step(stream):
        hip.conv2d_bias_act_f32_dev(batch, c_in, h, w, c_out, *geom, 1, d_x, d_w, d_b, d_out, stream)

    wall, ev, sus = timer.measure(step, headline=True)
    flops = 2 * batch * c_out * h * w * c_in * 9
    bytes_ = 4 * (x.size + wt.size + b.size + batch * c_out * h * w)
    return entry("conv2d_bias_relu_f32_n32_c64to128_56x56_k3s1p1", "f32", flops, bytes_, "mfma", wall, ev, sustained=sus), \
        (x, wt, b, geom, (batch, c_in, h, w, c_out))


def wl_conv2d_bf16(hip, inputs, timer):
    """Config 2's layer on bf16-rounded operands (bf16 NCHW images and OIHW weights, f32 accumulation, f32 output): the
    implicit GEMM on the bf16 matrix cores, priced against the bf16 peak.  The timed step includes the copy of the images
    into the padded channels-last layout the kernel works on and the re-layout of the weights."""
    batch, c_in, h, w, c_out = 32, 64, 56, 56, 128
    x = inputs.to_bf16(inputs.normal(inputs.seed_for(2, 0), batch * c_in * h * w))
    wt = inputs.to_bf16(inputs.normal(inputs.seed_for(2, 1), c_out * c_in * 9, 0.0, math.sqrt(2.0 / (c_in * 9))))
    b = inputs.uniform(inputs.seed_for(2, 2), c_out, -0.1, 0.1)
    d_x, d_w, d_b = (hip.DeviceBuffer.from_array(a) for a in (x, wt, b))
    d_out = hip.DeviceBuffer(batch * c_out * h * w * 4)
    geom = ((3, 3), (1, 1), (1, 1), (1, 1))

    def step(stream):
        hip.conv2d_bias_act_bf16_dev(batch, c_in, h, w, c_out, *geom, 1, d_x, d_w, d_b, d_out, None, stream)

    wall, ev, sus = timer.measure(step)
    flops = 2 * batch * c_out * h * w * c_in * 9
    bytes_ = 2 * (x.size + wt.size) + 4 * (b.size + batch * c_out * h * w)
    return entry("conv2d_bias_relu_bf16_f32acc_n32_c64to128_56x56_k3s1p1", "bf16", flops, bytes_, "mfma", wall, ev, sustained=sus)


def wl_conv2d_backward(hip, inputs, timer, which):
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
    wall, ev, sus = timer.measure(step)
    flops = 2 * batch * c_out * h * w * c_in * 9
    return entry(f"conv2d_{which}_f32_n32_c64to128_56x56_k3s1p1", "f32", flops, bytes_, "mfma", wall, ev, sustained=sus)


def wl_gemm_f32(hip, inputs, timer, m, n, k, name, long=False):
    a = inputs.uniform(inputs.seed_for(1, 0), m * k, -1.0, 1.0)
    b = inputs.uniform(inputs.seed_for(1, 1), k * n, -1.0, 1.0)
    d_a, d_b = hip.DeviceBuffer.from_array(a), hip.DeviceBuffer.from_array(b)
    d_c = hip.DeviceBuffer(m * n * 4)

    def step(stream):
        hip.gemm_f32_dev(m, n, k, 1.0, False, d_a, d_b, d_c, stream)

    wall, ev, sus = timer.measure(step, long=long)
    return entry(name, "f32", 2 * m * n * k, 4 * (m * k + k * n + m * n), "mfma", wall, ev, sustained=sus)


def wl_gemm_bf16(hip, inputs, timer, m, n, k, name, bound, packed=False):
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

    wall, ev, sus = timer.measure(step)
    extra = None
    if copies > 1:
        _, resident = timer.run(lambda stream: step(stream, rotate=False), SUSTAINED_WARMUP, SUSTAINED_STEPS)
        extra = {"rhs_copies_cycled": copies, "kernel_ms_per_step_rhs_cache_resident": round(resident, 5)}
    return entry(name, "bf16", 2 * m * n * k, 2 * (m * k + k * n) + 4 * m * n, bound, wall, ev, extra, sustained=sus)


def wl_attention(hip, inputs, timer, causal):
    contexts, seq, dim = 128, 2048, 64
    count = contexts * seq * dim
    q, k, v = (inputs.normal(inputs.seed_for(3, i), count) for i in range(3))
    d_q, d_k, d_v = (hip.DeviceBuffer.from_array(a) for a in (q, k, v))
    d_o = hip.DeviceBuffer(count * 4)

    def step(stream):
        hip.attention_f32_dev(contexts, seq, dim, 0.125, causal, d_q, d_k, d_v, None, None, d_o, stream)

    wall, ev, sus = timer.measure(step, long=True)
    flops = 4 * dim * contexts * (seq * (seq + 1) // 2 if causal else seq * seq)
    name = "attention_f32_b8_h16_s2048_d64_" + ("causal" if causal else "noncausal")
    return entry(name, "f32", flops, 4 * 4 * count, "mfma", wall, ev, sustained=sus)


def wl_attention_bias(hip, inputs, timer, contexts, seq):
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

    wall, ev, sus = timer.measure(step)
    flops = 4 * dim * contexts * seq * seq
    return entry(f"attention_f32_attn_bias_c{contexts}_s{seq}_d64", "f32", flops, 4 * (4 * count + bias.size), "mfma",
                 wall, ev, sustained=sus)


def wl_attention_bf16(hip, inputs, timer):
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

    wall, ev, sus = timer.measure(step)
    flops = 4 * dim * batch * heads * (seq * (seq + 1) // 2)
    return entry("attention_bf16_b16_h8_s1024_d64_causal", "bf16", flops, 2 * 4 * batch * seq * width, "mfma", wall, ev,
                 sustained=sus)


def wl_decoder(hip, inputs, timer):
    vocab, d, heads, layers, ff, batch, seq = 256, 512, 8, 6, 2048, 16, 1024
    count = hip.Decoder.weight_count(vocab, d, heads, layers, ff)
    weights = inputs.normal(inputs.seed_for(5, 0), count, 0.0, 0.02)
    tokens = inputs.tokens(inputs.seed_for(5, 1), batch * seq, vocab)
    dec = hip.Decoder(vocab, d, heads, layers, ff, batch, seq, 1e-5, weights)
    d_tok = hip.DeviceBuffer.from_array(tokens)
    d_logits = hip.DeviceBuffer(batch * seq * vocab * 4)

    def step(stream):
        dec.forward_dev(d_tok, d_logits, stream)

    wall, ev, sus = timer.measure(step, long=True)
    T = batch * seq
    hd = d // heads
    per_layer = 3 * 2 * T * d * d + 2 * T * d * d + 4 * hd * batch * heads * (seq * (seq + 1) // 2) + 2 * 2 * T * d * ff
    flops = layers * per_layer + 2 * T * d * vocab
    out = entry("decoder_bf16_v256_d512_h8_l6_ff2048_b16_s1024", "bf16", flops, 0, "mfma", wall, ev,
                {"tokens_per_s": round(T / (wall * 1e-3), 1)}, sustained=sus)
    dec.destroy()
    return out


def wl_rowops(hip, inputs, timer):
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
        wall, ev, sus = timer.measure(step)
        out.append(entry(f"{name}_16384x512", "f32", 0, bytes_, "hbm", wall, ev, sustained=sus))
    return out


def fill_tiled(buf, block):
    """Fills a device buffer with repeated copies of a seeded host block (a 1 GiB operand from a 64 MiB block: random
    bits everywhere, generated in a second)."""
    step = block.nbytes
    for offset in range(0, buf.nbytes, step):
        part = block if offset + step <= buf.nbytes else block.ravel().view(np.uint8)[:buf.nbytes - offset]
        buf.upload(part, offset)


def wl_lopsided(hip, inputs, timer):
    """Shapes outside the BASELINE configs whose dispatch has kernels of its own: matrix x vector (a stream over A: the
    f32 matrix is 1 GiB, the bf16 one 512 MiB, both beyond the 256 MiB memory-side cache), a product of few output tiles
    with a long k (k-sliced over workgroups), softmax over rows of 100000 values (each row cut into segments over the grid), and thousands
    of short attention windows.  All HBM-bound; bytes are the algorithmic reads + writes.  Operands are seeded random
    values like every other workload's (the big matrices repeat a 64 MiB block)."""
    out = []
    m = k = 16384
    block = inputs.uniform(inputs.seed_for(1, 3), 16 * 1024 * 1024, -1.0, 1.0)
    d_a = hip.DeviceBuffer(m * k * 4)
    fill_tiled(d_a, block)
    d_a16 = hip.DeviceBuffer(m * k * 2)
    fill_tiled(d_a16, inputs.to_bf16(block))
    d_x = hip.DeviceBuffer.from_array(inputs.uniform(inputs.seed_for(1, 2), k, -1.0, 1.0))
    d_y = hip.DeviceBuffer(m * 4)
    wall, ev, sus = timer.measure(lambda st: hip.gemm_f32_dev(m, 1, k, 1.0, False, d_a, d_x, d_y, st), long=True)
    out.append(entry(f"gemv_f32_{m}x1x{k}", "f32", 2 * m * k, 4 * (m * k + k + m), "hbm", wall, ev, sustained=sus))
    d_x16 = hip.DeviceBuffer.from_array(inputs.to_bf16(inputs.uniform(inputs.seed_for(1, 2), k, -1.0, 1.0)))
    wall, ev, sus = timer.measure(lambda st: hip.gemm_bf16_f32acc_dev(m, 1, k, d_a16, d_x16, d_y, st), long=True)
    out.append(entry(f"gemv_bf16_{m}x1x{k}", "bf16", 2 * m * k, 2 * (m * k + k) + 4 * m, "hbm", wall, ev, sustained=sus))
    # the same stored matrix read as k x m: A^T x, the gradient of the product above with respect to x
    wall, ev, sus = timer.measure(lambda st: hip.gemm_f32_dev(m, 1, k, 1.0, True, d_a, d_x, d_y, st), long=True)
    out.append(entry(f"gemv_f32_lhs_transposed_{m}x1x{k}", "f32", 2 * m * k, 4 * (m * k + k + m), "hbm", wall, ev, sustained=sus))
    m2, n2, k2 = 64, 64, 100000
    d_c = hip.DeviceBuffer(m2 * n2 * 4)
    d_b2 = hip.DeviceBuffer.from_array(inputs.uniform(inputs.seed_for(1, 4), k2 * n2, -1.0, 1.0))
    wall, ev, sus = timer.measure(lambda st: hip.gemm_f32_dev(m2, n2, k2, 1.0, False, d_a, d_b2, d_c, st), long=True)
    out.append(entry(f"gemm_f32_{m2}x{n2}x{k2}_k_sliced", "f32", 2 * m2 * n2 * k2, 4 * (m2 * k2 + k2 * n2 + m2 * n2), "hbm", wall, ev,
                     sustained=sus))
    rows, cols = 100, 100000
    d_in = hip.DeviceBuffer.from_array(inputs.normal(inputs.seed_for(5, 5), rows * cols))
    d_out = hip.DeviceBuffer(rows * cols * 4)
    wall, ev, sus = timer.measure(lambda st: hip.row_softmax_f32_dev(rows, cols, d_in, d_out, st), long=True)
    out.append(entry(f"row_softmax_f32_{rows}x{cols}", "f32", 0, 8 * rows * cols, "hbm", wall, ev, sustained=sus))
    # windowed attention: 16384 contexts of 16 positions, head size 64 (a wavefront per context)
    ctx, seq, dim = 16384, 16, 64
    n = ctx * seq * dim
    d_q, d_k, d_v = (hip.DeviceBuffer.from_array(inputs.normal(inputs.seed_for(3, 8 + i), n)) for i in range(3))
    d_o = hip.DeviceBuffer(n * 4)
    wall, ev, sus = timer.measure(lambda st: hip.attention_f32_dev(ctx, seq, dim, 0.125, False, d_q, d_k, d_v, None, None, d_o, st),
                                  long=True)
    out.append(entry(f"attention_f32_{ctx}_windows_of_{seq}x{dim}", "f32", 4 * ctx * seq * seq * dim, 16 * n, "hbm", wall, ev,
                     sustained=sus))
    return out


def wl_decoder_gemms(hip, inputs, timer):
    """The four projections of one decoder layer on their own (config 5's shapes: 16384 tokens, d_model 512, 2048-wide
    MLP; bf16 operands prepacked as the decoder holds them), so that profiles can attribute counters to each: QKV
    (bf16 out: the persistent kernel), out-proj and fc2 (f32 out + residual), fc1 (GELU, bf16 out)."""
    T, d, ff = 16384, 512, 2048
    out = []
    d_res = hip.DeviceBuffer.from_array(inputs.normal(inputs.seed_for(5, 7), T * d))
    for name, n, k, act, residual, out16 in (("qkv", 3 * d, d, 0, False, True), ("out_proj", d, d, 0, True, False),
                                             ("fc1_gelu", ff, d, 2, False, True), ("fc2", d, ff, 0, True, False)):
        d_a = hip.DeviceBuffer.from_array(inputs.to_bf16(inputs.normal(inputs.seed_for(5, 8), T * k)))
        d_b = hip.DeviceBuffer.from_array(inputs.to_bf16(inputs.normal(inputs.seed_for(5, 9), k * n, 0.0, 0.02)))
        d_packed = hip.DeviceBuffer(k * n * 2)
        hip.pack_rhs_bf16_dev(k, n, d_b, d_packed)
        d_bias = hip.DeviceBuffer.from_array(inputs.normal(inputs.seed_for(5, 10), n, 0.0, 0.02))
        d32 = None if out16 else hip.DeviceBuffer(T * n * 4)
        d16 = hip.DeviceBuffer(T * n * 2) if out16 else None
        step = lambda st: hip.gemm_bf16_prepacked_bias_act_dev(T, n, k, act, d_a, d_packed, d_bias, d_res if residual else None, d32, d16, st)
        wall, ev, sus = timer.measure(step)
        bytes_ = 2 * (T * k + k * n) + (2 if out16 else 4) * T * n + (4 * T * n if residual else 0)
        out.append(entry(f"decoder_gemm_{name}_bf16_{T}x{n}x{k}", "bf16", 2 * T * n * k, bytes_, "mfma", wall, ev, sustained=sus))
    return out


def wl_calibration(hip, inputs, timer):
    """Plain streaming kernel of known traffic (f32 -> bf16 rounding of 64 Mi values: 256 MiB read, 128 MiB
    written).  It anchors the FETCH_SIZE / WRITE_SIZE counters and shows the HBM rate a trivial kernel reaches."""
    count = 64 * 1024 * 1024
    d_src = hip.DeviceBuffer(count * 4)
    fill_tiled(d_src, inputs.normal(inputs.seed_for(5, 6), 16 * 1024 * 1024))
    d_dst = hip.DeviceBuffer(count * 2)

    def step(stream):
        hip.f32_to_bf16_dev(count, d_src, d_dst, stream)

    wall, ev, sus = timer.measure(step, long=True)
    return entry("calibration_f32_to_bf16_64mi", "f32", 0, count * 6, "hbm", wall, ev, sustained=sus)


def probe_ceilings(hip, inputs, timer):
    """What frames the bf16 GEMM figures on this box, measured in this process (stderr lines only, with --probes):
    (1) a loop of bf16 matrix instructions alone, on all-zero and on N(0, 0.02^2) register operands: the rate the matrix
        pipes sustain on those bits with no memory instruction in the way (power, hence clock, depends on the bits);
    (1b) a loop of direct-to-LDS loads alone: what a compute unit streams out of L2, the memory-side cache and HBM;
    (2) the vendor library (torch.mm -> hipBLASLt) on config 4's operands, B row-major (NN) and transposed (NT), under
        the same two protocols as the workloads.  torch is imported for this probe only; nothing else here uses it."""
    out = []
    sink = hip.DeviceBuffer(256 * 256 * 4)
    for label, values in (("zeros", np.zeros(32768, np.float32)),
                          ("normal_0.02", inputs.normal(inputs.seed_for(4, 3), 32768, 0.0, 0.02))):
        d_ops = hip.DeviceBuffer.from_array(inputs.to_bf16(values))
        iterations = 4000  # 256 workgroups x 4 wavefronts x 32 x 4000 matrix instructions: about 10 ms
        _, ev = timer.run(lambda st: hip.probe_mfma_bf16_dev(256, iterations, d_ops, sink, st), 2, 10)
        flops = 256 * 4 * iterations * 32 * 2 * 32 * 32 * 16
        out.append({"probe": f"mfma_bf16_32x32x16_only_{label}", "kernel_ms": round(ev, 4),
                    "tflops": round(flops / (ev * 1e-3) / 1e12, 1), "frac_of_bf16_peak": round(flops / (ev * 1e-3) / 1e12 / PEAK_TFLOPS["bf16"], 4)})
    for label, values in (("zeros", np.zeros(4096, np.float32)), ("normal_1", inputs.normal(inputs.seed_for(2, 3), 4096, 0.0, 1.0))):
        d_ops = hip.DeviceBuffer.from_array(values.astype(np.float32))
        iterations = 4000
        _, ev = timer.run(lambda st: hip.probe_mfma_f32_dev(256, iterations, d_ops, sink, st), 2, 10)
        flops = 256 * 4 * iterations * 32 * 2 * 32 * 32 * 2
        out.append({"probe": f"mfma_f32_32x32x2_only_{label}", "kernel_ms": round(ev, 4),
                    "tflops": round(flops / (ev * 1e-3) / 1e12, 1), "frac_of_f32_peak": round(flops / (ev * 1e-3) / 1e12 / PEAK_TFLOPS["f32"], 4)})
    # (1b) a loop of direct-to-LDS loads in the GEMM kernels' access shape, one workgroup per compute unit, over a region
    #      that fits every XCD's L2 (2 MiB), only the memory-side cache (64 MiB), or neither (1 GiB)
    for label, mib in (("l2_2mib", 2), ("memory_side_cache_64mib", 64), ("hbm_1gib", 1024)):
        region_bytes = mib << 20
        d_region = hip.DeviceBuffer(region_bytes)
        d_region.zero()  # every page touched; the values do not matter to a load
        iterations = 400  # 256 workgroups x 8 wavefronts x 400 x 8 KB = 6.7 GB per launch
        _, ev = timer.run(lambda st: hip.probe_stream_lds_dev(256, iterations, d_region, region_bytes, st), 2, 5)
        total = 256 * 8 * iterations * 8192
        out.append({"probe": f"direct_to_lds_stream_{label}", "kernel_ms": round(ev, 4), "tb_per_s": round(total / (ev * 1e-3) / 1e12, 2),
                    "gb_per_s_per_compute_unit": round(total / 256 / (ev * 1e-3) / 1e9, 1)})
        del d_region
    # this library's prepacked kernel with bf16 as the only output: what the vendor library's bf16-out figures compare with
    m = n = k = 4096
    d_a = hip.DeviceBuffer.from_array(inputs.to_bf16(inputs.normal(inputs.seed_for(4, 0), m * k, 0.0, 0.02)))
    d_b = hip.DeviceBuffer.from_array(inputs.to_bf16(inputs.normal(inputs.seed_for(4, 1), k * n, 0.0, 0.02)))
    d_packed, d_c16 = hip.DeviceBuffer(k * n * 2), hip.DeviceBuffer(m * n * 2)
    hip.pack_rhs_bf16_dev(k, n, d_b, d_packed)
    step = lambda st: hip.gemm_bf16_prepacked_bias_act_dev(m, n, k, 0, d_a, d_packed, None, None, None, d_c16, st)
    _, first = timer.run(step, timer.warmup, timer.steps)
    _, second = timer.run(step, SUSTAINED_WARMUP, SUSTAINED_STEPS)
    frac = lambda ms: round(2 * m * n * k / (ms * 1e-3) / 1e12 / PEAK_TFLOPS["bf16"], 4)
    out.append({"probe": "this_library_prepacked_bf16_4096_cubed_bf16_out", "kernel_ms_per_step": round(first, 5), "frac": frac(first),
                "sustained_kernel_ms_per_step": round(second, 5), "sustained_frac": frac(second)})
    # torch brings a HIP runtime of its own, which finds no device once this process has initialised the system's: the
    # library probe runs as a child process (the parent is idle meanwhile) and hands its lines back on stdout.
    import subprocess
    child = subprocess.run([sys.executable, "-c", VENDOR_PROBE, ROOT, str(timer.warmup), str(timer.steps),
                            str(SUSTAINED_WARMUP), str(SUSTAINED_STEPS), str(PEAK_TFLOPS["bf16"])],
                           stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    lines = [line for line in child.stdout.splitlines() if line.startswith("{")]
    if child.returncode != 0 or not lines:
        out.append({"probe": "vendor_library", "skipped": (child.stderr.strip().splitlines() or ["no output"])[-1][:200]})
    out.extend(json.loads(line) for line in lines)
    return out


# The vendor library on config 4's operands (torch.mm -> hipBLASLt), B row-major (NN) and transposed (NT), bf16 output,
# under the protocol asked for and the sustained one.  A probe for comparison only; run as `python -c`.
VENDOR_PROBE = r"""
import json, sys
root, warmup, steps, sus_warmup, sus_steps, peak = sys.argv[1], int(sys.argv[2]), int(sys.argv[3]), int(sys.argv[4]), int(sys.argv[5]), float(sys.argv[6])
sys.path.insert(0, root)
import torch
from spiraltorch_amd import inputs
n = 4096
a = torch.from_numpy(inputs.normal(inputs.seed_for(4, 0), n * n, 0.0, 0.02).reshape(n, n)).cuda().to(torch.bfloat16)
b = torch.from_numpy(inputs.normal(inputs.seed_for(4, 1), n * n, 0.0, 0.02).reshape(n, n)).cuda().to(torch.bfloat16)
bt = b.t().contiguous()
c = torch.empty(n, n, dtype=torch.bfloat16, device="cuda")
start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
def timed(fn, w, k):
    for _ in range(w):
        fn()
    torch.cuda.synchronize()
    start.record()
    for _ in range(k):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / k
cases = [("NN_bf16_out", lambda: torch.mm(a, b, out=c)), ("NT_bf16_out", lambda: torch.mm(a, bt.t(), out=c))]
try:  # f32 output, what config 4 asks for, where this torch offers it
    torch.mm(a, b, out_dtype=torch.float32)
    cases += [("NN_f32_out", lambda: torch.mm(a, b, out_dtype=torch.float32)), ("NT_f32_out", lambda: torch.mm(a, bt.t(), out_dtype=torch.float32))]
except Exception:
    pass
for label, fn in cases:
    first = timed(fn, warmup, steps)
    second = timed(fn, sus_warmup, sus_steps)
    frac = lambda ms: round(2 * n ** 3 / (ms * 1e-3) / 1e12 / peak, 4)
    print(json.dumps({"probe": "vendor_library_torch_mm_bf16_4096_cubed_" + label, "kernel_ms_per_step": round(first, 5),
                      "frac": frac(first), "sustained_kernel_ms_per_step": round(second, 5), "sustained_frac": frac(second)}), flush=True)
"""


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
                f"{passes} full passes of config 2, 1 thread, {sum(seconds):.1f} s in all, median pass {median:.2f} s; "
                f"host has {os.cpu_count()} logical CPUs")


def cpu_baselines(inputs, with_gemv=False):
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
            flops, sec, 1, f"2 of 128 contexts, 1 thread, {sec:.2f} s (full config: {sec * 64:.0f} s)")
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
    if with_gemv:  # matrix x vector: 2048 of the 16384 rows, all cores over rows
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
        f"1 of 6 layers on 1 of 16 sequences, 1 thread, {sec:.2f} s (full config: about {sec * 96:.0f} s)")
    return out


def final_line(args, headline, cpu, props, rows):
    """The one JSON line of stdout: the headline workload in the contract's keys, then a compact row per BASELINE
    workload."""
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
        "workloads": [compact(item) for item in rows],
    }
    if "sustained" in headline:
        line["sustained"] = headline["sustained"]
    return line


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=200)
    parser.add_argument("--warmup", type=int, default=50)
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-sustained", action="store_true", help="skip the second (50 + 200 steps) measurement")
    parser.add_argument("--only", default=None, help="run only the headline plus workloads whose name contains this")
    parser.add_argument("--probes", action="store_true",
                        help="also measure the bf16 ceilings of this box: a matrix-instruction-only loop and the vendor library "
                             "(stderr lines only)")
    parser.add_argument("--all", action="store_true",
                        help="also run the workloads that are no BASELINE configuration (stderr lines only)")
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
    timer = Timer(hip, args.warmup, args.steps, sustained=not args.no_sustained)

    headline, conv_inputs = wl_conv2d(hip, inputs, timer)
    log(json.dumps(headline))
    # BASELINE configurations (and the backward / biased / prepacked forms of the same kernels): rows of the final line.
    plan = [
        ("gemm_f32_512", lambda: wl_gemm_f32(hip, inputs, timer, 512, 512, 512, "gemm_f32_512x512x512")),
        ("gemm_bf16_4096", lambda: wl_gemm_bf16(hip, inputs, timer, 4096, 4096, 4096, "gemm_bf16_f32acc_4096x4096x4096", "mfma")),
        ("gemm_bf16_4096_prepacked", lambda: wl_gemm_bf16(hip, inputs, timer, 4096, 4096, 4096,
                                                          "gemm_bf16_f32acc_4096x4096x4096_prepacked_rhs", "mfma", True)),
        ("gemm_bf16_skinny", lambda: wl_gemm_bf16(hip, inputs, timer, 16, 4096, 4096, "gemm_bf16_f32acc_16x4096x4096", "hbm")),
        ("gemm_bf16_skinny_prepacked", lambda: wl_gemm_bf16(hip, inputs, timer, 16, 4096, 4096,
                                                            "gemm_bf16_f32acc_16x4096x4096_prepacked_rhs", "hbm", True)),
        ("attention_noncausal", lambda: wl_attention(hip, inputs, timer, False)),
        ("attention_causal", lambda: wl_attention(hip, inputs, timer, True)),
        ("decoder", lambda: wl_decoder(hip, inputs, timer)),
        ("attention_bf16", lambda: wl_attention_bf16(hip, inputs, timer)),
        ("gemm_f32_conv_equivalent", lambda: wl_gemm_f32(hip, inputs, timer, 100352, 128, 576,
                                                         "gemm_f32_100352x128x576_conv_equivalent")),
        ("conv2d_bf16", lambda: wl_conv2d_bf16(hip, inputs, timer)),
        ("conv2d_grad_input", lambda: wl_conv2d_backward(hip, inputs, timer, "grad_input")),
        ("conv2d_grad_weight", lambda: wl_conv2d_backward(hip, inputs, timer, "grad_weight")),
        ("attention_bias", lambda: [wl_attention_bias(hip, inputs, timer, 1, 2048), wl_attention_bias(hip, inputs, timer, 16, 1024)]),
    ]
    # Not BASELINE configurations: stderr lines only, and only when asked for.
    extra_plan = [
        ("gemm_f32_4096", lambda: wl_gemm_f32(hip, inputs, timer, 4096, 4096, 4096, "gemm_f32_4096x4096x4096", long=True)),
        ("decoder_gemms", lambda: wl_decoder_gemms(hip, inputs, timer)),
        ("rowops", lambda: wl_rowops(hip, inputs, timer)),
        ("lopsided", lambda: wl_lopsided(hip, inputs, timer)),
        ("calibration", lambda: wl_calibration(hip, inputs, timer)),
    ]

    def run(entries):
        out = []
        for name, fn in entries:
            if args.only and args.only not in name:
                continue
            result = fn()
            out.extend(result if isinstance(result, list) else [result])
        return out

    rows = run(plan)
    extras = run(extra_plan) if args.all else []
    if args.probes:
        for item in probe_ceilings(hip, inputs, timer):
            log(json.dumps(item))

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline_conv(conv_inputs)
        log(json.dumps(cpu))
        per_workload = cpu_baselines(inputs, with_gemv=bool(extras))
        for item in rows + extras:
            if item["workload"] in per_workload:
                item["cpu_baseline"] = per_workload[item["workload"]]
            elif item["workload"].startswith("conv2d_bias_relu_bf16"):
                item["cpu_baseline"] = dict(cpu, sample="the f32 pass of the same layer (the port computes bf16 operands in f32)")
            elif item["workload"].startswith("conv2d_grad"):
                item["cpu_baseline"] = dict(cpu, sample="forward pass of the same layer (the backward runs the same contraction sizes)")
    for item in rows + extras:
        log(json.dumps(item))
    print(json.dumps(final_line(args, headline, cpu, props, rows)), flush=True)


if __name__ == "__main__":
    main()
