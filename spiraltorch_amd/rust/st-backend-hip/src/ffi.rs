// Generated from include/st_hip.h by spiraltorch_amd/rust/gen_ffi.py; do not edit by hand.
// The C ABI of libsthip.so: plain pointers and sizes, 0 = ST_HIP_OK, else a status code whose text
// st_hip_last_error_message returns for the calling thread.
#![allow(clippy::too_many_arguments)]

use std::os::raw::{c_char, c_int, c_void};

/// `st_hip_device_props`.
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

#[link(name = "sthip")]
extern "C" {
    pub fn st_hip_init() -> c_int;
    pub fn st_hip_real_backend_compiled() -> c_int;
    pub fn st_hip_device_count() -> c_int;
    pub fn st_hip_device_name(index: c_int, buf: *mut c_char, len: usize) -> c_int;
    pub fn st_hip_device_properties(index: c_int, out: *mut StHipDeviceProps) -> c_int;
    pub fn st_hip_probe(out: *mut StHipProbeResult) -> c_int;
    pub fn st_hip_last_error_message(buf: *mut c_char, len: usize) -> usize;
    pub fn st_hip_malloc(device_ptr: *mut *mut c_void, bytes: usize) -> c_int;
    pub fn st_hip_free(device_ptr: *mut c_void) -> c_int;
    pub fn st_hip_memcpy_h2d(device_dst: *mut c_void, host_src: *const c_void, bytes: usize, stream: *mut c_void) -> c_int;
    pub fn st_hip_memcpy_d2h(host_dst: *mut c_void, device_src: *const c_void, bytes: usize, stream: *mut c_void) -> c_int;
    pub fn st_hip_memset_zero(device_dst: *mut c_void, bytes: usize, stream: *mut c_void) -> c_int;
    pub fn st_hip_transfer_counters(counters: *mut u64, reset: c_int) -> c_int;
    pub fn st_hip_stream_create(stream: *mut *mut c_void) -> c_int;
    pub fn st_hip_stream_synchronize(stream: *mut c_void) -> c_int;
    pub fn st_hip_stream_destroy(stream: *mut c_void) -> c_int;
    pub fn st_hip_device_synchronize() -> c_int;
    pub fn st_hip_release_scratch(stream: *mut c_void) -> c_int;
    pub fn st_hip_scratch_buffer_count() -> usize;
    pub fn st_hip_event_create(event: *mut *mut c_void) -> c_int;
    pub fn st_hip_event_record(event: *mut c_void, stream: *mut c_void) -> c_int;
    pub fn st_hip_event_synchronize(event: *mut c_void) -> c_int;
    pub fn st_hip_event_elapsed_ms(start: *mut c_void, stop: *mut c_void, milliseconds: *mut f32) -> c_int;
    pub fn st_hip_event_destroy(event: *mut c_void) -> c_int;
    pub fn st_hip_gemm_f32(m: usize, n: usize, k: usize, scale: f32, lhs_transposed: c_int, lhs: *const f32, lhs_len: usize, rhs: *const f32, rhs_len: usize, out: *mut f32, out_len: usize) -> c_int;
    pub fn st_hip_gemm_f32_raw(m: usize, n: usize, k: usize, lhs: *const f32, rhs: *const f32, out: *mut f32) -> c_int;
    pub fn st_hip_gemm_bias_act_f32(m: usize, n: usize, k: usize, activation: c_int, lhs: *const f32, lhs_len: usize, rhs: *const f32, rhs_len: usize, bias: *const f32, bias_len: usize, residual: *const f32, residual_len: usize, out: *mut f32, out_len: usize) -> c_int;
    pub fn st_hip_gemm_prepacked_bias_act_f32(m: usize, n: usize, k: usize, activation: c_int, lhs: *const f32, lhs_len: usize, packed_rhs: *const f32, packed_len: usize, bias: *const f32, bias_len: usize, residual: *const f32, residual_len: usize, out: *mut f32, out_len: usize) -> c_int;
    pub fn st_hip_gemm_bf16_f32acc(m: usize, n: usize, k: usize, lhs: *const u16, lhs_len: usize, rhs: *const u16, rhs_len: usize, out: *mut f32, out_len: usize) -> c_int;
    pub fn st_hip_conv2d_output_hw(h: usize, w: usize, kh: usize, kw: usize, stride_h: usize, stride_w: usize, pad_h: usize, pad_w: usize, dil_h: usize, dil_w: usize, oh: *mut usize, ow: *mut usize) -> c_int;
    pub fn st_hip_conv2d_bias_act_f32(batch: usize, c_in: usize, h: usize, w: usize, c_out: usize, kh: usize, kw: usize, stride_h: usize, stride_w: usize, pad_h: usize, pad_w: usize, dil_h: usize, dil_w: usize, activation: c_int, input: *const f32, input_len: usize, weight: *const f32, weight_len: usize, bias: *const f32, bias_len: usize, out: *mut f32, out_len: usize) -> c_int;
    pub fn st_hip_conv2d_force_family(family: c_int) -> c_int;
    pub fn st_hip_conv2d_planned_kernel(batch: usize, c_in: usize, h: usize, w: usize, c_out: usize, kh: usize, kw: usize, stride_h: usize, stride_w: usize, pad_h: usize, pad_w: usize, dil_h: usize, dil_w: usize, direction: c_int, kernel: *mut c_int) -> c_int;
    pub fn st_hip_conv2d_backward_f32(batch: usize, c_in: usize, h: usize, w: usize, c_out: usize, kh: usize, kw: usize, stride_h: usize, stride_w: usize, pad_h: usize, pad_w: usize, dil_h: usize, dil_w: usize, input: *const f32, input_len: usize, weight: *const f32, weight_len: usize, grad_output: *const f32, grad_output_len: usize, grad_input: *mut f32, grad_input_len: usize, grad_weight: *mut f32, grad_weight_len: usize, grad_bias: *mut f32, grad_bias_len: usize) -> c_int;
    pub fn st_hip_attention_f32(contexts: usize, sequence: usize, head_dim: usize, scale: f32, causal: c_int, q: *const f32, q_len: usize, k: *const f32, k_len: usize, v: *const f32, v_len: usize, z_bias: *const f32, z_bias_len: usize, attn_bias: *const f32, attn_bias_len: usize, out: *mut f32, out_len: usize) -> c_int;
    pub fn st_hip_attention_f32_launch_plan(contexts: usize, sequence: usize, head_dim: usize, causal: c_int, biased: c_int, plan: *mut StHipAttentionPlan) -> c_int;
    pub fn st_hip_gemm_bf16_tile_plan(m: usize, n: usize, k: usize, plan: *mut StHipGemmTilePlan) -> c_int;
    pub fn st_hip_gemm_row_block(k: usize, element_bytes: usize) -> usize;
    pub fn st_hip_gemm_f32_dev(m: usize, n: usize, k: usize, scale: f32, lhs_transposed: c_int, lhs: *const f32, rhs: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_gemm_bias_act_f32_dev(m: usize, n: usize, k: usize, activation: c_int, lhs: *const f32, rhs: *const f32, bias: *const f32, residual: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_gemm_prepacked_bias_act_f32_dev(m: usize, n: usize, k: usize, activation: c_int, lhs: *const f32, packed_rhs: *const f32, bias: *const f32, residual: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_pack_rhs_f32_dev(k: usize, n: usize, rhs: *const f32, packed: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_gemm_bf16_f32acc_dev(m: usize, n: usize, k: usize, lhs: *const u16, rhs: *const u16, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_gemm_bf16_bias_act_dev(m: usize, n: usize, k: usize, activation: c_int, lhs: *const u16, rhs: *const u16, bias: *const f32, residual: *const f32, out_f32: *mut f32, out_bf16: *mut u16, stream: *mut c_void) -> c_int;
    pub fn st_hip_gemm_bf16_prepacked_bias_act_dev(m: usize, n: usize, k: usize, activation: c_int, lhs: *const u16, packed_rhs: *const u16, bias: *const f32, residual: *const f32, out_f32: *mut f32, out_bf16: *mut u16, stream: *mut c_void) -> c_int;
    pub fn st_hip_gemm_bf16_prepacked_residual_layer_norm_dev(m: usize, n: usize, k: usize, lhs: *const u16, packed_rhs: *const u16, bias: *const f32, residual: *const f32, gamma: *const f32, beta: *const f32, epsilon: f32, out_f32: *mut f32, out_ln_bf16: *mut u16, stream: *mut c_void) -> c_int;
    pub fn st_hip_pack_rhs_bf16_dev(k: usize, n: usize, rhs: *const u16, packed: *mut u16, stream: *mut c_void) -> c_int;
    pub fn st_hip_conv2d_bias_act_f32_dev(batch: usize, c_in: usize, h: usize, w: usize, c_out: usize, kh: usize, kw: usize, stride_h: usize, stride_w: usize, pad_h: usize, pad_w: usize, dil_h: usize, dil_w: usize, activation: c_int, input: *const f32, weight: *const f32, bias: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_conv2d_bias_act_bf16_dev(batch: usize, c_in: usize, h: usize, w: usize, c_out: usize, kh: usize, kw: usize, stride_h: usize, stride_w: usize, pad_h: usize, pad_w: usize, dil_h: usize, dil_w: usize, activation: c_int, input: *const u16, weight: *const u16, bias: *const f32, out_f32: *mut f32, out_bf16: *mut u16, stream: *mut c_void) -> c_int;
    pub fn st_hip_conv2d_grad_input_f32_dev(batch: usize, c_in: usize, h: usize, w: usize, c_out: usize, kh: usize, kw: usize, stride_h: usize, stride_w: usize, pad_h: usize, pad_w: usize, dil_h: usize, dil_w: usize, grad_output: *const f32, weight: *const f32, grad_input: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_conv2d_grad_input_f32_noalloc_dev(batch: usize, c_in: usize, h: usize, w: usize, c_out: usize, kh: usize, kw: usize, stride_h: usize, stride_w: usize, pad_h: usize, pad_w: usize, dil_h: usize, dil_w: usize, grad_output: *const f32, weight: *const f32, grad_input: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_conv2d_grad_weight_f32_dev(batch: usize, c_in: usize, h: usize, w: usize, c_out: usize, kh: usize, kw: usize, stride_h: usize, stride_w: usize, pad_h: usize, pad_w: usize, dil_h: usize, dil_w: usize, input: *const f32, grad_output: *const f32, scale: f32, grad_weight: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_conv2d_grad_bias_f32_dev(batch: usize, c_in: usize, h: usize, w: usize, c_out: usize, kh: usize, kw: usize, stride_h: usize, stride_w: usize, pad_h: usize, pad_w: usize, dil_h: usize, dil_w: usize, grad_output: *const f32, scale: f32, grad_bias: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_attention_f32_dev(contexts: usize, sequence: usize, head_dim: usize, scale: f32, causal: c_int, q: *const f32, k: *const f32, v: *const f32, z_bias: *const f32, attn_bias: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_attention_bf16_dev(batch: usize, heads: usize, sequence: usize, head_dim: usize, scale: f32, causal: c_int, q: *const u16, k: *const u16, v: *const u16, ld_in: usize, out: *mut u16, ld_out: usize, stream: *mut c_void) -> c_int;
    pub fn st_hip_row_softmax_f32_dev(rows: usize, cols: usize, input: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_gelu_f32_dev(count: usize, input: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_count_nonfinite_f32_dev(count: usize, data: *const f32, nonfinite: *mut u64, first_index: *mut u64, first_value: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_gelu_backward_f32_dev(count: usize, z: *const f32, grad: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_scale_f32_dev(count: usize, input: *const f32, scale: f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_add_row_f32_dev(rows: usize, cols: usize, data: *mut f32, bias: *const f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_sum_axis0_f32_dev(rows: usize, cols: usize, input: *const f32, scale: f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_layer_norm_f32_dev(rows: usize, cols: usize, x: *const f32, residual: *const f32, gamma: *const f32, beta: *const f32, epsilon: f32, out_f32: *mut f32, out_bf16: *mut u16, stream: *mut c_void) -> c_int;
    pub fn st_hip_embedding_f32_dev(tokens: usize, vocab: usize, dim: usize, token_ids: *const f32, table: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_f32_to_bf16_dev(count: usize, input: *const f32, out: *mut u16, stream: *mut c_void) -> c_int;
    pub fn st_hip_split_heads_f32_dev(batch: usize, seq: usize, heads: usize, head_dim: usize, qkv: *const f32, q: *mut f32, k: *mut f32, v: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_merge_heads_f32_dev(batch: usize, seq: usize, heads: usize, head_dim: usize, contexts_in: *const f32, out_f32: *mut f32, out_bf16: *mut u16, stream: *mut c_void) -> c_int;
    pub fn st_hip_probe_mfma_bf16_dev(workgroups: usize, iterations: usize, operands: *const u16, sink: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_probe_mfma_f32_dev(workgroups: usize, iterations: usize, operands: *const f32, sink: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_probe_stream_lds_dev(workgroups: usize, iterations: usize, region: *const c_void, region_bytes: usize, stream: *mut c_void) -> c_int;
    pub fn st_hip_decoder_weight_count(config: *const StHipDecoderConfig) -> usize;
    pub fn st_hip_decoder_create(config: *const StHipDecoderConfig, host_weights: *const f32, weight_len: usize, decoder: *mut *mut c_void) -> c_int;
    pub fn st_hip_decoder_forward_dev(decoder: *mut c_void, tokens: *const f32, logits: *mut f32, stream: *mut c_void) -> c_int;
    pub fn st_hip_decoder_destroy(decoder: *mut c_void) -> c_int;
}
