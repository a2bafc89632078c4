//! `st-backend-hip` over `libsthip.so`: the operator surface `st-tensor`'s `hip_dense` adapter calls
//! (crates/st-tensor/src/backend/hip_dense.rs:14-261), with the same names, argument order `(m, n, k, …)`, checks
//! and error texts as the reference crate (crates/st-backend-hip/src/lib.rs:446-523, 607-799), plus the operators
//! that crate did not have: fused conv2d, scaled-dot-product attention and the bf16 GEMM.
//!
//! Validation lives behind the C ABI (the library checks lengths, overflow and scales before it touches `out`), so
//! the wrappers here only translate slices into pointer + length pairs and status codes into `HipErr`.
//!
//! This source is not compiled where the rest of this repository is built (no Rust toolchain there);
//! `src/ffi.rs` is generated from `include/st_hip.h` and checked against it by the repository's tests.

use std::borrow::Cow;
use std::ffi::CStr;
use std::os::raw::{c_char, c_int};
use std::sync::{Arc, Mutex, OnceLock};

use serde::{Deserialize, Serialize};
use thiserror::Error;

pub mod device;
pub mod ffi;

pub use device::{DeviceBuffer, Event, Stream};
pub use ffi::StHipDecoderConfig as DecoderConfig;

#[derive(Debug, Error)]
pub enum HipErr {
    #[error("HIP not enabled (build with feature 'hip-real')")]
    NotEnabled,
    #[error("Other: {0}")]
    Other(String),
}

/// Activation applied by the fused GEMM / conv2d epilogue (codes of `ST_HIP_ACT_*`).
#[repr(i32)]
#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub enum GemmActivation {
    Relu = 1,
    Gelu = 2,
}

pub const fn real_backend_compiled() -> bool {
    true
}

#[derive(Debug, Clone, Serialize, Deserialize, PartialEq, Eq)]
pub struct DeviceInfo {
    pub id: u32,
    pub name: Cow<'static, str>,
    pub multi_node: bool,
}

impl DeviceInfo {
    pub fn new<N: Into<Cow<'static, str>>>(id: u32, name: N, multi_node: bool) -> Self {
        Self { id, name: name.into(), multi_node }
    }
}

#[derive(Debug, Clone)]
pub struct HipProbe {
    pub available: bool,
    pub initialized: bool,
    pub devices: Vec<DeviceInfo>,
    pub error: Option<String>,
}

#[derive(Debug)]
pub struct HipRuntime {
    devices: Vec<DeviceInfo>,
}

impl HipRuntime {
    pub fn devices(&self) -> &[DeviceInfo] {
        &self.devices
    }

    pub fn device_count(&self) -> usize {
        self.devices.len()
    }
}

fn last_error() -> String {
    let mut buf = [0 as c_char; 512];
    unsafe { ffi::st_hip_last_error_message(buf.as_mut_ptr(), buf.len()) };
    unsafe { CStr::from_ptr(buf.as_ptr()) }.to_string_lossy().into_owned()
}

/// 0 is success; ST_HIP_ERR_NOT_ENABLED (1) maps to `NotEnabled`, every other code carries the library's message
/// (validator text, "{ctx}: {name} ({rc}) - {text}" for HIP failures, the non-finite label).
pub(crate) fn status(rc: c_int) -> Result<(), HipErr> {
    match rc {
        0 => Ok(()),
        1 => Err(HipErr::NotEnabled),
        _ => Err(HipErr::Other(last_error())),
    }
}

fn runtime_slot() -> &'static Mutex<Option<Arc<HipRuntime>>> {
    static RUNTIME: OnceLock<Mutex<Option<Arc<HipRuntime>>>> = OnceLock::new();
    RUNTIME.get_or_init(|| Mutex::new(None))
}

pub fn runtime() -> Option<Arc<HipRuntime>> {
    runtime_slot().lock().unwrap_or_else(|p| p.into_inner()).as_ref().map(Arc::clone)
}

/// Idempotent and thread-safe, like the library's own `st_hip_init`.
pub fn init() -> Result<Arc<HipRuntime>, HipErr> {
    if let Some(existing) = runtime() {
        return Ok(existing);
    }
    status(unsafe { ffi::st_hip_init() })?;
    let created = Arc::new(HipRuntime { devices: device_info() });
    let mut slot = runtime_slot().lock().unwrap_or_else(|p| p.into_inner());
    Ok(slot.get_or_insert(created).clone())
}

pub fn hip_available() -> bool {
    unsafe { ffi::st_hip_device_count() > 0 }
}

pub fn device_info() -> Vec<DeviceInfo> {
    let count = unsafe { ffi::st_hip_device_count() }.max(0);
    (0..count)
        .map(|index| {
            let mut name = [0 as c_char; 256];
            let rc = unsafe { ffi::st_hip_device_name(index, name.as_mut_ptr(), name.len()) };
            let text = if rc == 0 {
                unsafe { CStr::from_ptr(name.as_ptr()) }.to_string_lossy().into_owned()
            } else {
                format!("hip:{index}")
            };
            DeviceInfo::new(index as u32, text, false)
        })
        .collect()
}

pub fn probe() -> HipProbe {
    let mut raw = ffi::StHipProbeResult { available: 0, initialized: 0, device_count: 0, error: [0; 256] };
    unsafe { ffi::st_hip_probe(&mut raw) };
    let error = unsafe { CStr::from_ptr(raw.error.as_ptr()) }.to_string_lossy().into_owned();
    HipProbe {
        available: raw.available != 0,
        initialized: raw.initialized != 0,
        devices: if raw.available != 0 { device_info() } else { Vec::new() },
        error: if error.is_empty() { None } else { Some(error) },
    }
}

pub fn gemm_f32(m: usize, n: usize, k: usize, lhs: &[f32], rhs: &[f32], out: &mut [f32]) -> Result<(), HipErr> {
    gemm_scaled_f32(m, n, k, 1.0, lhs, rhs, out)
}

/// `out = (lhs @ rhs) * scale`, contiguous row-major; the scale is applied to the full sum.
pub fn gemm_scaled_f32(m: usize, n: usize, k: usize, scale: f32, lhs: &[f32], rhs: &[f32], out: &mut [f32]) -> Result<(), HipErr> {
    init()?;
    status(unsafe {
        ffi::st_hip_gemm_f32(m, n, k, scale, 0, lhs.as_ptr(), lhs.len(), rhs.as_ptr(), rhs.len(), out.as_mut_ptr(), out.len())
    })
}

/// `out = (lhs.T @ rhs) * scale`; `lhs` is `k x m`, `rhs` is `k x n`.
pub fn gemm_lhs_transpose_scaled_f32(m: usize, n: usize, k: usize, scale: f32, lhs: &[f32], rhs: &[f32], out: &mut [f32]) -> Result<(), HipErr> {
    init()?;
    status(unsafe {
        ffi::st_hip_gemm_f32(m, n, k, scale, 1, lhs.as_ptr(), lhs.len(), rhs.as_ptr(), rhs.len(), out.as_mut_ptr(), out.len())
    })
}

/// GEMM, then `(acc + bias) + residual`, then the activation, fused into the GEMM's store.
#[allow(clippy::too_many_arguments)]
pub fn gemm_bias_activation_f32(
    m: usize, n: usize, k: usize, activation: GemmActivation, lhs: &[f32], rhs: &[f32], bias: &[f32],
    residual: Option<&[f32]>, out: &mut [f32],
) -> Result<(), HipErr> {
    init()?;
    let (res_ptr, res_len) = residual.map_or((std::ptr::null(), 0), |r| (r.as_ptr(), r.len()));
    status(unsafe {
        ffi::st_hip_gemm_bias_act_f32(m, n, k, activation as c_int, lhs.as_ptr(), lhs.len(), rhs.as_ptr(), rhs.len(),
                                      bias.as_ptr(), bias.len(), res_ptr, res_len, out.as_mut_ptr(), out.len())
    })
}

/// The same on a right-hand side prepacked as its `(n, k)` transpose (`PackedB`, pure.rs:1285-1323).
#[allow(clippy::too_many_arguments)]
pub fn gemm_prepacked_bias_activation_f32(
    m: usize, n: usize, k: usize, activation: Option<GemmActivation>, lhs: &[f32], packed_rhs: &[f32],
    bias: Option<&[f32]>, residual: Option<&[f32]>, out: &mut [f32],
) -> Result<(), HipErr> {
    init()?;
    let (bias_ptr, bias_len) = bias.map_or((std::ptr::null(), 0), |b| (b.as_ptr(), b.len()));
    let (res_ptr, res_len) = residual.map_or((std::ptr::null(), 0), |r| (r.as_ptr(), r.len()));
    status(unsafe {
        ffi::st_hip_gemm_prepacked_bias_act_f32(m, n, k, activation.map_or(0, |a| a as c_int), lhs.as_ptr(), lhs.len(),
                                                packed_rhs.as_ptr(), packed_rhs.len(), bias_ptr, bias_len, res_ptr, res_len,
                                                out.as_mut_ptr(), out.len())
    })
}

/// # Safety
/// `lhs`, `rhs` and `out` must point to `m*k`, `k*n` and `m*n` valid, non-aliasing `f32` values.
pub unsafe fn gemm_f32_raw(m: usize, n: usize, k: usize, lhs: *const f32, rhs: *const f32, out: *mut f32) -> Result<(), HipErr> {
    init()?;
    status(ffi::st_hip_gemm_f32_raw(m, n, k, lhs, rhs, out))
}

/// bf16 operands (raw bit patterns), f32 accumulation and output.
pub fn gemm_bf16_f32acc(m: usize, n: usize, k: usize, lhs: &[u16], rhs: &[u16], out: &mut [f32]) -> Result<(), HipErr> {
    init()?;
    status(unsafe {
        ffi::st_hip_gemm_bf16_f32acc(m, n, k, lhs.as_ptr(), lhs.len(), rhs.as_ptr(), rhs.len(), out.as_mut_ptr(), out.len())
    })
}

/// Geometry of a 2-D convolution in the order `Conv2d` keeps it (crates/st-nn/src/layers/conv.rs:685-748).
#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub struct Conv2dGeometry {
    pub batch: usize,
    pub c_in: usize,
    pub h: usize,
    pub w: usize,
    pub c_out: usize,
    pub kernel: (usize, usize),
    pub stride: (usize, usize),
    pub padding: (usize, usize),
    pub dilation: (usize, usize),
}

/// NCHW input, OIHW weight, per-channel bias, optional activation, NCHW output: `Conv2d::forward` fused.
pub fn conv2d_bias_activation_f32(
    g: &Conv2dGeometry, activation: Option<GemmActivation>, input: &[f32], weight: &[f32], bias: &[f32], out: &mut [f32],
) -> Result<(), HipErr> {
    init()?;
    status(unsafe {
        ffi::st_hip_conv2d_bias_act_f32(g.batch, g.c_in, g.h, g.w, g.c_out, g.kernel.0, g.kernel.1, g.stride.0, g.stride.1,
                                        g.padding.0, g.padding.1, g.dilation.0, g.dilation.1,
                                        activation.map_or(0, |a| a as c_int), input.as_ptr(), input.len(), weight.as_ptr(),
                                        weight.len(), bias.as_ptr(), bias.len(), out.as_mut_ptr(), out.len())
    })
}

/// `scaled_dot_attention` (crates/st-tensor/src/pure.rs:4061-4354): q, k, v and out are `(contexts * sequence,
/// head_dim)`; `z_bias` is `(contexts, sequence)`, `attn_bias` `(contexts * sequence, sequence)`.
#[allow(clippy::too_many_arguments)]
pub fn scaled_dot_attention_f32(
    contexts: usize, sequence: usize, head_dim: usize, scale: f32, causal: bool, q: &[f32], k: &[f32], v: &[f32],
    z_bias: Option<&[f32]>, attn_bias: Option<&[f32]>, out: &mut [f32],
) -> Result<(), HipErr> {
    init()?;
    let (z_ptr, z_len) = z_bias.map_or((std::ptr::null(), 0), |b| (b.as_ptr(), b.len()));
    let (a_ptr, a_len) = attn_bias.map_or((std::ptr::null(), 0), |b| (b.as_ptr(), b.len()));
    status(unsafe {
        ffi::st_hip_attention_f32(contexts, sequence, head_dim, scale, causal as c_int, q.as_ptr(), q.len(), k.as_ptr(),
                                  k.len(), v.as_ptr(), v.len(), z_ptr, z_len, a_ptr, a_len, out.as_mut_ptr(), out.len())
    })
}

/// Device-resident GEMM + epilogue on a caller's stream: operands stay in HBM between operators.
#[allow(clippy::too_many_arguments)]
pub fn gemm_bias_activation_f32_dev(
    m: usize, n: usize, k: usize, activation: Option<GemmActivation>, lhs: &DeviceBuffer<f32>, rhs: &DeviceBuffer<f32>,
    bias: Option<&DeviceBuffer<f32>>, residual: Option<&DeviceBuffer<f32>>, out: &mut DeviceBuffer<f32>, stream: &Stream,
) -> Result<(), HipErr> {
    let expect = |what: &str, have: usize, want: Option<usize>| match want {
        Some(w) if w == have => Ok(()),
        _ => Err(HipErr::Other(format!("{what} buffer length {have} does not match the GEMM shape"))),
    };
    expect("lhs", lhs.len(), m.checked_mul(k))?;
    expect("rhs", rhs.len(), k.checked_mul(n))?;
    expect("out", out.len(), m.checked_mul(n))?;
    if let Some(b) = bias {
        expect("bias", b.len(), Some(n))?;
    }
    if let Some(r) = residual {
        expect("residual", r.len(), m.checked_mul(n))?;
    }
    status(unsafe {
        ffi::st_hip_gemm_bias_act_f32_dev(m, n, k, activation.map_or(0, |a| a as c_int), lhs.as_ptr(), rhs.as_ptr(),
                                          bias.map_or(std::ptr::null(), |b| b.as_ptr()),
                                          residual.map_or(std::ptr::null(), |r| r.as_ptr()), out.as_mut_ptr(), stream.as_raw())
    })
}
