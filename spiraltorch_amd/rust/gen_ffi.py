"""Writes st-backend-hip/src/ffi.rs: the Rust `extern "C"` block for every function include/st_hip.h declares.

    python spiraltorch_amd/rust/gen_ffi.py            # rewrite ffi.rs
    python spiraltorch_amd/rust/gen_ffi.py --check    # exit 1 when ffi.rs is not what the header gives

The block replaces the hand-written one of the reference crate (crates/st-backend-hip/src/real.rs:45-157, the
hipMalloc / hipMemcpyAsync / rocblas_sgemm / epilogue-launcher imports): the crate binds libsthip.so and nothing
else.  tests/test_abi.py runs the check, so the binding cannot drift from the header."""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "..", "..", "include", "st_hip.h")
TARGET = os.path.join(HERE, "st-backend-hip", "src", "ffi.rs")

SCALARS = {"size_t": "usize", "int": "c_int", "float": "f32", "uint64_t": "u64", "uint16_t": "u16", "char": "c_char",
           "void": "c_void", "st_hip_device_props": "StHipDeviceProps", "st_hip_probe_result": "StHipProbeResult",
           "st_hip_decoder_config": "StHipDecoderConfig", "st_hip_attention_plan": "StHipAttentionPlan",
           "st_hip_gemm_tile_plan": "StHipGemmTilePlan"}
RUST_KEYWORDS = {"in": "input", "type": "kind", "ref": "reference"}

STRUCTS = '''/// `st_hip_device_props`.
#[repr(C)]
#[derive(Clone, Copy)]
pub struct StHipDeviceProps {
    pub compute_units: c_int,
    pub clock_khz: c_int,
    pub memory_clock_khz: c_int,
    pub memory_bus_bits: c_int,
    pub wavefront_size: c_int,
    pub lds_bytes_per_block: c_int,
    pub l2_bytes: c_int,
    pub total_memory_bytes: u64,
    pub arch: [c_char; 64],
}

/// `st_hip_probe_result`.
#[repr(C)]
#[derive(Clone, Copy)]
pub struct StHipProbeResult {
    pub available: c_int,
    pub initialized: c_int,
    pub device_count: c_int,
    pub error: [c_char; 256],
}

/// `st_hip_decoder_config`.
#[repr(C)]
#[derive(Clone, Copy, Debug, PartialEq)]
pub struct StHipDecoderConfig {
    pub vocab: usize,
    pub d_model: usize,
    pub heads: usize,
    pub layers: usize,
    pub d_ff: usize,
    pub batch: usize,
    pub seq: usize,
    pub ln_eps: f32,
}

/// `st_hip_attention_plan`.
#[repr(C)]
#[derive(Clone, Copy, Debug, Default, PartialEq)]
pub struct StHipAttentionPlan {
    pub kernel: c_int,
    pub key_splits: c_int,
    pub keys_per_split: c_int,
    pub consistent: c_int,
    pub workgroups: u64,
    pub items: u64,
    pub items_expected: u64,
    pub out_of_range: u64,
    pub duplicates: u64,
}

/// `st_hip_gemm_tile_plan`.
#[repr(C)]
#[derive(Clone, Copy, Debug, Default, PartialEq)]
pub struct StHipGemmTilePlan {
    pub tile_cols: c_int,
    pub tiles_m: c_int,
    pub tiles_n: c_int,
    pub k_splits: c_int,
    pub k_tiles_per_split: c_int,
    pub consistent: c_int,
    pub workgroups: u64,
    pub items: u64,
    pub out_of_range: u64,
    pub duplicates: u64,
}
'''


def declarations(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"typedef struct \{.*?\} \w+;", "", text, flags=re.S)
    for match in re.finditer(r"\b(int|size_t)\s+(st_hip_\w+)\s*\(([^)]*)\)\s*;", text):
        yield match.group(1), match.group(2), " ".join(match.group(3).split())


def rust_type(c_type):
    c_type = c_type.strip()
    const = c_type.startswith("const ")
    base = c_type[6:] if const else c_type
    stars = base.count("*")
    base = base.replace("*", "").strip()
    rust = SCALARS[base]
    for level in range(stars):
        rust = ("*const " if const and level == 0 else "*mut ") + rust
    return rust


def rust_argument(c_argument):
    if c_argument == "void":
        return None
    array = re.match(r"(.*\S)\s+(\w+)\[\d+\]$", c_argument)
    if array:
        c_type, name = array.group(1) + " *", array.group(2)
    else:
        match = re.match(r"(.*?)(\w+)$", c_argument)
        c_type, name = match.group(1), match.group(2)
    return f"{RUST_KEYWORDS.get(name, name)}: {rust_type(c_type)}"


def render():
    with open(HEADER) as handle:
        header = handle.read()
    out = ["// Generated from include/st_hip.h by spiraltorch_amd/rust/gen_ffi.py; do not edit by hand.",
           "// The C ABI of libsthip.so: plain pointers and sizes, 0 = ST_HIP_OK, else a status code whose text",
           "// st_hip_last_error_message returns for the calling thread.",
           "#![allow(clippy::too_many_arguments)]", "",
           "use std::os::raw::{c_char, c_int, c_void};", "", STRUCTS,
           '#[link(name = "sthip")]', 'extern "C" {']
    for ret, name, args in declarations(header):
        rendered = [a for a in (rust_argument(part.strip()) for part in args.split(",")) if a]
        out.append(f"    pub fn {name}({', '.join(rendered)}) -> {SCALARS[ret]};")
    out.append("}")
    return "\n".join(out) + "\n"


def main():
    text = render()
    if "--check" in sys.argv:
        with open(TARGET) as handle:
            if handle.read() != text:
                print("ffi.rs does not match include/st_hip.h; run spiraltorch_amd/rust/gen_ffi.py", file=sys.stderr)
                sys.exit(1)
        return
    with open(TARGET, "w") as handle:
        handle.write(text)


if __name__ == "__main__":
    main()
