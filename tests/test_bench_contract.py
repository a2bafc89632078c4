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
