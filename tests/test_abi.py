"""CPU-side checks of the C-ABI boundary: the library loads, exports what include/st_hip.h declares,
the product never reaches into the oracle, and without a device every operator fails loudly."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "st_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(st_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_operator_surface():
    names = declared_symbols()
    for required in ("st_hip_init", "st_hip_gemm_f32", "st_hip_gemm_bias_act_f32", "st_hip_gemm_bf16_f32acc",
                     "st_hip_conv2d_bias_act_f32", "st_hip_attention_f32", "st_hip_gemm_f32_dev",
                     "st_hip_conv2d_bias_act_f32_dev", "st_hip_attention_f32_dev", "st_hip_decoder_forward_dev",
                     "st_hip_last_error_message"):
        assert required in names


def test_library_exports_every_declared_symbol():
    from spiraltorch_amd import _lib
    lib = ctypes.CDLL(_lib.LIBRARY_PATH)
    missing = [name for name in declared_symbols() if not hasattr(lib, name)]
    assert not missing, f"declared in st_hip.h but not exported: {missing}"


def test_python_binding_covers_every_declared_symbol():
    from spiraltorch_amd import _lib
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_rust_binding_matches_the_header():
    """The Rust crate's extern block (spiraltorch_amd/rust/st-backend-hip/src/ffi.rs) is generated from the header;
    it must be the generator's current output, name every declared symbol once, and every ffi:: call in the crate's
    hand-written sources must name a declared symbol with the declared number of arguments."""
    import subprocess
    import sys
    rust = os.path.join(ROOT, "spiraltorch_amd", "rust")
    subprocess.run([sys.executable, os.path.join(rust, "gen_ffi.py"), "--check"], check=True)
    ffi = open(os.path.join(rust, "st-backend-hip", "src", "ffi.rs")).read()
    bound = re.findall(r"pub fn (st_hip_\w+)\(([^)]*)\)", ffi)
    assert sorted(name for name, _ in bound) == declared_symbols()
    arity = {name: (0 if not args.strip() else args.count(":")) for name, args in bound}
    for source in ("lib.rs", "device.rs"):
        text = open(os.path.join(rust, "st-backend-hip", "src", source)).read()
        for match in re.finditer(r"ffi::(st_hip_\w+)\(", text):
            name = match.group(1)
            assert name in arity, f"{source} calls {name}, which the header does not declare"
            depth, i, commas, empty = 1, match.end(), 0, True
            while depth:
                ch = text[i]
                depth += ch in "([{"
                depth -= ch in ")]}"
                if depth == 1 and ch == ",":
                    commas += 1
                if depth >= 1 and not ch.isspace() and not (depth == 0):
                    empty = empty and ch == ")"
                i += 1
            passed = 0 if empty else commas + 1
            assert passed == arity[name], f"{source}: {name} called with {passed} arguments, declared with {arity[name]}"


def test_product_never_touches_the_oracle():
    offenders = []
    for base, _, files in os.walk(os.path.join(ROOT, "spiraltorch_amd")):
        for name in files:
            if name.endswith((".py", ".hip", ".h", ".cpp", "Makefile")):
                text = open(os.path.join(base, name), errors="replace").read()
                if re.search(r"\boracle\b|st_oracle", text):
                    offenders.append(os.path.join(base, name))
    assert not offenders, f"product sources mention the oracle: {offenders}"


def test_wire_codes_match_the_reference():
    # crates/st-backend-hip/src/lib.rs:29-34 (Relu = 1, Gelu = 2); the reference asserts the same codes
    # against its kernel source in tests/hip_build_support.rs:56-66.
    from spiraltorch_amd import hip
    assert int(hip.GemmActivation.Relu) == 1 and int(hip.GemmActivation.Gelu) == 2
    header = open(os.path.join(ROOT, "include", "st_hip.h")).read()
    assert re.search(r"ST_HIP_ACT_RELU\s*=\s*1", header) and re.search(r"ST_HIP_ACT_GELU\s*=\s*2", header)
    device = open(os.path.join(ROOT, "spiraltorch_amd", "csrc", "device_math.h")).read()
    assert "ST_HIP_ACT_RELU" in device and "ST_HIP_ACT_GELU" in device


def test_real_backend_is_compiled():
    from spiraltorch_amd import hip
    assert hip.real_backend_compiled() is True


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present; covered by the gpu tests")
def test_without_a_device_operators_fail_loudly():
    from spiraltorch_amd import Tensor, TensorError, hip
    assert hip.hip_available() is False
    with pytest.raises(hip.HipErr) as info:
        hip.init()
    assert info.value.kind == "NotEnabled"
    out = np.full(4, 13.0, np.float32)
    with pytest.raises(hip.HipErr):
        hip.gemm_f32(2, 2, 2, np.ones(4, np.float32), np.ones(4, np.float32), out)
    assert (out == 13.0).all()  # no CPU result was written
    with pytest.raises(TensorError) as err:
        Tensor(2, 2, [1, 2, 3, 4]).matmul(Tensor(2, 2, [1, 0, 0, 1]), backend="hip")
    assert err.value.kind == "BackendFailure"
    with pytest.raises(TensorError):
        Tensor(2, 2, [1, 2, 3, 4]).matmul(Tensor(2, 2, [1, 0, 0, 1]), backend="cpu")


def test_input_generator():
    from spiraltorch_amd import inputs
    # splitmix64 known answer for seed 0 (first three outputs of the published reference implementation)
    assert [hex(int(v)) for v in inputs.splitmix64(0, 3)] == ["0xe220a8397b1dcdaf", "0x6e789e6aa1b965f4",
                                                              "0x6c45d188009454f"]
    assert (inputs.splitmix64(5, 4, offset=3) == inputs.splitmix64(5, 7)[3:]).all()
    u = inputs.uniform(inputs.seed_for(1, 0), 1 << 16, -1.0, 1.0)
    assert u.dtype == np.float32 and u.min() >= -1.0 and u.max() < 1.0 and abs(u.mean()) < 0.02
    n = inputs.normal(inputs.seed_for(3, 1), 1 << 16)
    assert abs(n.mean()) < 0.02 and abs(n.std() - 1.0) < 0.02
    t = inputs.tokens(7, 4096, 256)
    assert t.min() >= 0 and t.max() <= 255 and len(np.unique(t)) > 200
