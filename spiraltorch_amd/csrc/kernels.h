// Internal launcher interface between the C-ABI entry points and the gfx950 kernels.
// Every launcher validates nothing: callers have already checked shapes, pointers and alignment
// assumptions that the kernels rely on are re-derived inside the launcher from the arguments.
#pragma once

#include "common.h"

namespace sthip {

struct GemmEpilogue {
    float scale = 1.0f;              // applied to the full sum, before bias (pure.rs:2256-2262)
    const float *bias = nullptr;     // per column (per row for the convolution)
    const float *residual = nullptr; // same shape as the output
    int activation = ST_HIP_ACT_NONE;
};

// C(m×n) = epilogue(A·B); A is m×k (k×m when lhs_transposed), B is k×n, all f32 row-major.
// `scratch_free`: the stream's scratch buffer is not holding anything of the caller's, so a launch of few tiles with a
// long k may put its k-sliced partial sums there; callers that keep an operand or a result in it pass false.
hipError_t launch_gemm_f32(size_t m, size_t n, size_t k, bool lhs_transposed, const float *lhs,
                           const float *rhs, float *out, const GemmEpilogue &epilogue,
                           hipStream_t stream, bool scratch_free = true);

// Matrix times a few columns (n <= 3 for f32, n <= 7 for bf16; 16-byte aligned operands, k a multiple of the 16-byte
// vector): a stream over A, one wavefront or workgroup per row.  The tiled launchers route here when `*_applies`.
bool gemv_f32_applies(size_t m, size_t n, size_t k, const float *lhs, const float *rhs);
hipError_t launch_gemv_f32(size_t m, size_t n, size_t k, const float *lhs, const float *rhs, float *out,
                           const GemmEpilogue &epilogue, hipStream_t stream);
// A stored k×m (lhs_transposed): uses the stream's scratch memory.
bool gemv_t_f32_applies(size_t m, size_t n, size_t k);
hipError_t launch_gemv_t_f32(size_t m, size_t n, size_t k, const float *lhs, const float *rhs, float *out,
                             const GemmEpilogue &epilogue, hipStream_t stream);
bool gemv_bf16_applies(size_t m, size_t n, size_t k, const uint16_t *lhs, const uint16_t *rhs);
hipError_t launch_gemv_bf16(size_t m, size_t n, size_t k, const uint16_t *lhs, const uint16_t *rhs, bool rhs_packed,
                            float *out_f32, uint16_t *out_bf16, const GemmEpilogue &epilogue, hipStream_t stream);

// `batch` plain products that share B in one launch: product i reads lhs + i·lhs_stride and writes out + i·out_stride
// (values, not bytes).  Never touches the stream's scratch buffer.
hipError_t launch_gemm_f32_batched(size_t batch, size_t m, size_t n, size_t k, bool lhs_transposed, const float *lhs,
                                   size_t lhs_stride, const float *rhs, float *out, size_t out_stride, hipStream_t stream);

// Same with B prepacked as n×k (column-major packing, crates/st-tensor/src/pure.rs:1285-1323).
hipError_t launch_gemm_f32_packed(size_t m, size_t n, size_t k, const float *lhs, const float *packed_rhs,
                                  float *out, const GemmEpilogue &epilogue, hipStream_t stream);
// out(cols×rows) = in(rows×cols) transposed.
hipError_t launch_transpose_f32(size_t rows, size_t cols, const float *in, float *out, hipStream_t stream);

// bf16 operands, f32 accumulation; writes out_f32 and/or out_bf16 (either may be null).  `rhs_packed`: rhs is the
// n×k transpose of B (PackedB's layout, crates/st-tensor/src/pure.rs:1285-1323) instead of k×n.
hipError_t launch_gemm_bf16(size_t m, size_t n, size_t k, const uint16_t *lhs, const uint16_t *rhs,
                            float *out_f32, uint16_t *out_bf16, const GemmEpilogue &epilogue,
                            hipStream_t stream, bool rhs_packed = false);
// The launch arithmetic of the 256-row bf16 kernels for a shape, every workgroup decoded on the host: see
// st_hip_gemm_tile_plan.
struct GemmTilePlanReport {
    int tile_cols, tiles_m, tiles_n, k_splits, k_tiles_per_split, consistent;
    uint64_t workgroups, items, out_of_range, duplicates;
};
GemmTilePlanReport gemm_bf16_tile_plan_report(size_t m, size_t n, size_t k);

// out_f32 = (lhs·rhs + bias) + residual and out_ln = layer_norm(out_f32) rounded to bf16, rhs packed n×k: Linear + residual +
// LayerNorm of a transformer block (crates/st-vision/src/models/vit.rs:256-265) in one launch where the shape allows.
hipError_t launch_gemm_bf16_residual_layer_norm(size_t m, size_t n, size_t k, const uint16_t *lhs, const uint16_t *packed_rhs,
                                                const float *bias, const float *residual, const float *gamma, const float *beta,
                                                float epsilon, float *out_f32, uint16_t *out_ln, hipStream_t stream);
// out(cols×rows) = in(rows×cols) transposed, 16-bit elements.
hipError_t launch_transpose_u16(size_t rows, size_t cols, const uint16_t *in, uint16_t *out, hipStream_t stream);

struct ConvShape {
    int batch, c_in, h, w, c_out, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, oh, ow;
};
// Entries of the general implicit-GEMM kernel's LDS offset table: longer reductions (c_in*kh*kw) go through it in
// segments of this many terms.
constexpr int kConvTableEntries = 8192;
// `scratch`: where a launch of few tiles with a long reduction may keep its k-sliced partial sums —
// kConvScratchStream: in the stream's scratch buffer from byte `scratch_offset` on (the caller holds what lies before
// it and has sized the buffer with conv2d_scratch_bytes, so that it does not move); kConvScratchNone: nowhere, such
// launches run unsliced.
constexpr int kConvScratchStream = 0, kConvScratchNone = 1;
hipError_t launch_conv2d_f32(const ConvShape &shape, int activation, const float *input,
                             const float *weight, const float *bias, float *out, hipStream_t stream,
                             int scratch = kConvScratchStream, size_t scratch_offset = 0);
// Bytes of the stream's scratch buffer launch_conv2d_f32 uses for `shape` (0 for most shapes).
size_t conv2d_scratch_bytes(const ConvShape &shape, bool weight_aligned, bool out_aligned);

// Which kernel launch_conv2d_f32 would run for `shape` (one of ST_HIP_CONV_KERNEL_*; 0 when the family forced with
// set_conv_forced_family cannot serve it), and the same for launch_conv2d_grad_input_f32 on the forward `shape`.
int planned_conv_kernel(const ConvShape &shape, bool weight_aligned, bool out_aligned);
int planned_conv_grad_input_kernel(const ConvShape &shape);
void set_conv_forced_family(int family);

// The same convolution on bf16 images and weights (NCHW / OIHW bit patterns), f32 accumulation, f32 bias, f32 and/or bf16
// output (either may be null).  Uses the stream's scratch buffer for the re-laid operands.
bool conv2d_bf16_supported(const ConvShape &shape);
hipError_t launch_conv2d_bf16(const ConvShape &shape, int activation, const uint16_t *input, const uint16_t *weight,
                              const float *bias, float *out_f32, uint16_t *out_bf16, hipStream_t stream);

// Adjoint gather of the implicit GEMM (`shape` is the virtual forward problem: grad_output as the image, input
// positions as output pixels, original stride/padding/dilation; weight laid out [c_in][c_out·kh·kw]).
hipError_t launch_conv2d_adjoint_f32(const ConvShape &shape, const float *grad_output,
                                     const float *weight_ic_major, float *grad_input, hipStream_t stream);
// Conv2d backward (crates/st-nn/src/layers/conv.rs:780-813, 860-916); `shape` is the forward shape.
// The re-laid weights (c_out·c_in·kh·kw values) go to `weight_scratch` when given, else to the stream's workspace.
hipError_t launch_conv2d_grad_input_f32(const ConvShape &shape, const float *grad_output, const float *weight,
                                        float *grad_input, hipStream_t stream, float *weight_scratch = nullptr);
// Static device array behind st_hip_conv2d_grad_input_f32_noalloc_dev: its size, and its address on the current GPU.
constexpr size_t kNoAllocScratchBytes = ST_HIP_NOALLOC_SCRATCH_BYTES;
hipError_t noalloc_scratch(void **out);
hipError_t launch_conv2d_grad_weight_f32(const ConvShape &shape, const float *input, const float *grad_output,
                                         float scale, float *grad_weight, hipStream_t stream);
hipError_t launch_conv2d_grad_bias_f32(const ConvShape &shape, const float *grad_output, float scale,
                                       float *grad_bias, hipStream_t stream);

// Largest head_dim the attention kernel is instantiated for.
constexpr int kAttentionMaxHeadDim = 256;
hipError_t launch_attention_f32(size_t contexts, size_t sequence, size_t head_dim, float scale,
                                bool causal, const float *q, const float *k, const float *v,
                                const float *z_bias, const float *attn_bias, float *out,
                                hipStream_t stream);

// The launch arithmetic of launch_attention_f32 for a shape (16-byte aligned operands assumed), with every workgroup
// of the fast kernel's grid decoded on the host the way the kernel decodes it: see st_hip_attention_plan.
struct AttentionPlanReport {
    int kernel, key_splits, keys_per_split, consistent;
    uint64_t workgroups, items, items_expected, out_of_range, duplicates;
};
AttentionPlanReport attention_f32_plan_report(size_t contexts, size_t sequence, size_t head_dim, bool causal, bool biased);

// bf16 attention over heads stored as column slices of (batch·sequence, ld) matrices; head_dim 64 or 128.
bool attention_bf16_supported(size_t sequence, size_t head_dim, size_t ld_in, size_t ld_out, const void *q,
                              const void *k, const void *v, const void *out);
hipError_t launch_attention_bf16(size_t batch, size_t heads, size_t sequence, size_t head_dim, float scale,
                                 bool causal, const uint16_t *q, const uint16_t *k, const uint16_t *v,
                                 size_t ld_in, uint16_t *out, size_t ld_out, hipStream_t stream);

hipError_t launch_layer_norm_f32(size_t rows, size_t cols, const float *x, const float *residual,
                                 const float *gamma, const float *beta, float epsilon, float *out_f32,
                                 uint16_t *out_bf16, hipStream_t stream);
hipError_t launch_embedding_layer_norm_f32(size_t tokens, size_t vocab, size_t dim, const float *token_ids, const float *table,
                                           float *embedded, const float *gamma, const float *beta, float epsilon,
                                           uint16_t *out_bf16, hipStream_t stream);
hipError_t launch_embedding_f32(size_t tokens, size_t vocab, size_t dim, const float *token_ids,
                                const float *table, float *out, hipStream_t stream);
hipError_t launch_f32_to_bf16(size_t count, const float *in, uint16_t *out, hipStream_t stream);
hipError_t launch_split_heads_f32(size_t batch, size_t seq, size_t heads, size_t head_dim,
                                  const float *qkv, float *q, float *k, float *v, bool round_to_bf16,
                                  hipStream_t stream);
hipError_t launch_merge_heads_f32(size_t batch, size_t seq, size_t heads, size_t head_dim,
                                  const float *contexts_in, float *out_f32, uint16_t *out_bf16,
                                  hipStream_t stream);

// Element-wise and row-wise tensor utilities (all f32, row-major).
hipError_t launch_row_softmax_f32(size_t rows, size_t cols, const float *in, float *out, hipStream_t stream);
hipError_t launch_gelu_f32(size_t count, const float *in, float *out, hipStream_t stream);
// status[0] += number of non-finite values of data, status[1] = min(status[1], index of one).
hipError_t launch_nonfinite_probe_f32(size_t count, const float *data, unsigned long long *status, hipStream_t stream);
hipError_t launch_gelu_backward_f32(size_t count, const float *z, const float *grad, float *out, hipStream_t stream);
hipError_t launch_scale_f32(size_t count, const float *in, float scale, float *out, hipStream_t stream);
hipError_t launch_add_row_f32(size_t rows, size_t cols, float *data, const float *bias, hipStream_t stream);
hipError_t launch_sum_axis0_f32(size_t rows, size_t cols, const float *in, float scale, float *out, hipStream_t stream);

// Measurement aid: `workgroups` × 4 wavefronts each issue 32·iterations bf16 32x32x16 matrix instructions on register
// operands read once from `operands` (32768 bf16 values); sink receives workgroups·256 floats.
hipError_t launch_probe_mfma_bf16(size_t workgroups, size_t iterations, const uint16_t *operands, float *sink, hipStream_t stream);
hipError_t launch_probe_mfma_f32(size_t workgroups, size_t iterations, const float *operands, float *sink, hipStream_t stream);
hipError_t launch_probe_stream_lds(size_t workgroups, size_t iterations, const void *region, size_t region_bytes, hipStream_t stream);

// One grow-only device buffer per (stream, host thread) for kernels that need scratch memory (split-k partial sums,
// column-sum partials).  A thread's work on a stream is ordered, so two of its launches never use the buffer at the
// same time, and threads that share a stream (the NULL stream) do not share scratch.  A buffer whose thread has exited
// is handed to the next thread that asks on that stream; buffers are freed when their stream is destroyed or released.
hipError_t stream_workspace(hipStream_t stream, size_t bytes, void **out);
// A second buffer of the same kind (slot 1) for re-laid copies of a call's operands, which must stay where they are
// while the kernels that read them take scratch from slot 0.
hipError_t stream_workspace_slot(hipStream_t stream, int slot, size_t bytes, void **out);
void release_stream_workspace(hipStream_t stream);
size_t stream_workspace_entry_count();
// Host<->device copies made by the library, for tests that check where tensors live.
void count_transfer(bool to_device, size_t bytes);

}  // namespace sthip
