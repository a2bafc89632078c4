"""bench.py pieces that can be checked without a GPU: argument handling, roofline arithmetic, traffic table."""
import importlib.util
import json
import pathlib
import subprocess
import sys

ROOT = pathlib.Path(__file__).resolve().parent.parent


def load_bench():
    spec = importlib.util.spec_from_file_location("bench_module", ROOT / "bench.py")
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def test_more_than_one_gpu_is_refused_with_a_message():
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert run.returncode != 0
    assert "one GPU" in run.stderr
    assert run.stdout.strip() == ""  # no JSON line that could be mistaken for a measurement


def test_roofline_arithmetic_uses_the_published_peaks():
    bench = load_bench()
    mfma = bench.roofline("mfma", "f32", 14_797_504_512, 77_365_760, 0.16)
    assert mfma["unit"] == "TFLOP/s" and mfma["peak"] == 157.3
    assert abs(mfma["achieved"] - 92.484) < 1e-2 and abs(mfma["frac"] - 92.484 / 157.3) < 1e-3
    assert bench.roofline("mfma", "bf16", 1, 1, 1.0)["peak"] == 2500.0
    hbm = bench.roofline("hbm", "f32", 0, 33_554_432, 0.01)
    assert hbm["unit"] == "GB/s" and hbm["peak"] == 8000.0 and abs(hbm["achieved"] - 3355.4) < 0.1


def test_entries_carry_measured_traffic_only_where_a_profile_has_it():
    bench = load_bench()
    name = "conv2d_bias_relu_f32_n32_c64to128_56x56_k3s1p1"
    item = bench.entry(name, "f32", 14_797_504_512, 77_365_760, "mfma", 0.16, 0.16)
    assert item["roofline"]["traffic"] == bench.MEASURED_TRAFFIC_BYTES[name]
    assert 1.0 < item["roofline"]["traffic"] / 77_365_760 < 1.2  # measured HBM bytes close to the algorithmic bytes
    assert bench.entry("decoder_bf16_v256_d512_h8_l6_ff2048_b16_s1024", "bf16", 1, 1, "mfma", 1.0, 1.0)["roofline"]["traffic"] is None
    json.dumps(item)  # serialisable


def test_the_final_line_stays_far_below_the_stdout_tail_the_driver_keeps():
    """Every BASELINE workload with its roofline, sustained figure and CPU baseline fits a line of well under 16 KB."""
    import argparse

    bench = load_bench()
    sustained = {"warmup": 50, "steps": 200, "kernel_ms_per_step": 0.123456}
    cpu = {"value": 12345.678, "unit": "GFLOP/s", "cores": 16, "kind": "port", "sample": "x" * 110}
    names = ["gemm_f32_512x512x512", "gemm_bf16_f32acc_4096x4096x4096", "gemm_bf16_f32acc_4096x4096x4096_prepacked_rhs",
             "gemm_bf16_f32acc_16x4096x4096", "gemm_bf16_f32acc_16x4096x4096_prepacked_rhs",
             "attention_f32_b8_h16_s2048_d64_noncausal", "attention_f32_b8_h16_s2048_d64_causal",
             "decoder_bf16_v256_d512_h8_l6_ff2048_b16_s1024", "attention_bf16_b16_h8_s1024_d64_causal",
             "gemm_f32_100352x128x576_conv_equivalent", "conv2d_grad_input_f32_n32_c64to128_56x56_k3s1p1",
             "conv2d_grad_weight_f32_n32_c64to128_56x56_k3s1p1", "attention_f32_attn_bias_c1_s2048_d64",
             "attention_f32_attn_bias_c16_s1024_d64", "conv2d_bias_relu_bf16_n32_c64to128_56x56_k3s1p1",
             "conv2d_bias_relu_bf16_n32_c64to128_56x56_k3s1p1_spare_row"]
    rows = []
    for name in names:
        item = bench.entry(name, "bf16", 725_950_136_320, 268_435_456, "mfma", 1.234567, 1.234567,
                           {"tokens_per_s": 12546492.2, "kernel_ms_per_step_rhs_cache_resident": 0.00501}, sustained=sustained)
        item["cpu_baseline"] = cpu
        rows.append(item)
    headline = bench.entry("conv2d_bias_relu_f32_n32_c64to128_56x56_k3s1p1", "f32", 14_797_504_512, 77_365_760, "mfma",
                           0.15, 0.15, sustained=sustained)
    args = argparse.Namespace(steps=20, warmup=5)
    props = {"arch": "gfx950:sramecc+:xnack-", "compute_units": 256, "clock_khz": 2400000}
    line = bench.final_line(args, headline, cpu, props, rows)
    text = json.dumps(line)
    assert len(text) < 12 * 1024, len(text)
    assert line["steps"] == 20 and line["warmup"] == 5  # echoes what was passed
    assert line["sustained"]["steps"] == 200 and "frac" in line["sustained"]
    for row in line["workloads"]:
        assert {"workload", "roofline", "sustained", "cpu_baseline"} <= set(row)
        assert set(row["roofline"]) == {"bound", "achieved", "peak", "unit", "frac", "traffic"}


def test_side_workloads_follow_the_protocol_asked_for_and_add_the_sustained_one():
    bench = load_bench()
    timer = bench.Timer.__new__(bench.Timer)
    timer.warmup, timer.steps, timer.sustained = 5, 20, True
    assert timer.protocols(long=False, headline=True) == ((5, 20), (50, 200))
    assert timer.protocols(long=False) == ((5, 20), (50, 200))
    assert timer.protocols(long=True) == ((5, 20), (10, 40))
    timer.warmup, timer.steps = 50, 200
    assert timer.protocols(long=False) == ((50, 200), (50, 200))
    assert timer.protocols(long=True) == ((10, 40), (10, 40))
