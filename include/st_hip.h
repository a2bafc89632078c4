/*
 * st_hip.h — C ABI of libsthip.so, the gfx950 (MI355X) dense-compute backend for SpiralTorch's
 * `st-backend-hip` crate.
 *
 * Every entry point returns an `int` status: 0 on success, otherwise one of ST_HIP_ERR_*; the text of
 * the last failure on the calling thread is read with st_hip_last_error_message().  All matrices are
 * contiguous row-major.  "Host-slice" entry points take host pointers plus the slice lengths the Rust
 * caller holds, validate them BEFORE touching `out`, and are synchronous.  "_dev" entry points take
 * device pointers and an explicit stream (NULL = the default stream), enqueue work and return.
 *
 * Reference interfaces these replace (paths below the SpiralTorch checkout):
 *   crates/st-backend-hip/src/lib.rs:607-799   gemm_f32 / gemm_scaled_f32 /
 *                                              gemm_lhs_transpose_scaled_f32 /
 *                                              gemm_bias_activation_f32 / gemm_f32_raw
 *   crates/st-backend-hip/src/real.rs:45-157   the extern "C" block the Rust crate binds
 *   crates/st-backend-hip/src/hip_kernels/hip_gemm_epilogue.cu:46-54   st_gemm_epilogue_f32
 */
#ifndef ST_HIP_H
#define ST_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes ------------------------------------------------------------------------- */
enum {
    ST_HIP_OK = 0,
    ST_HIP_ERR_NOT_ENABLED = 1, /* HipErr::NotEnabled — no usable HIP device (lib.rs:14-20)        */
    ST_HIP_ERR_INVALID = 2,     /* HipErr::Other from a validator; `out` was not touched            */
    ST_HIP_ERR_RUNTIME = 3,     /* HIP call failed: "{ctx}: {name} ({rc}) - {text}" (real.rs:166)   */
    ST_HIP_ERR_NONFINITE = 4,   /* TensorError::NonFiniteValue{label} (pure.rs:5521-5533)           */
    ST_HIP_ERR_UNSUPPORTED = 5  /* shape outside what the kernels implement                         */
};

/* GemmActivation wire codes — crates/st-backend-hip/src/lib.rs:29-34 (Relu = 1, Gelu = 2);
 * 0 (bias only) extends them for the convolution, whose reference applies ReLU as a separate layer. */
enum { ST_HIP_ACT_NONE = 0, ST_HIP_ACT_RELU = 1, ST_HIP_ACT_GELU = 2 };

/* ---- runtime ------------------------------------------------------------------------------ */

/* st_backend_hip::init() — lib.rs:168-186.  Idempotent, thread-safe. */
int st_hip_init(void);
/* st_backend_hip::real_backend_compiled() — lib.rs:47-49.  Always 1 for this library. */
int st_hip_real_backend_compiled(void);
/* HipRuntime::device_count() — lib.rs:188-207 (probe) / real.rs enumerate_devices. */
int st_hip_device_count(void);
int st_hip_device_name(int index, char *buf, size_t len);

typedef struct {
    int compute_units;
    int clock_khz;
    int memory_clock_khz;
    int memory_bus_bits;
    int wavefront_size;
    int lds_bytes_per_block;
    int l2_bytes;
    uint64_t total_memory_bytes;
    char arch[64];
} st_hip_device_props;
int st_hip_device_properties(int index, st_hip_device_props *out);

/* st_backend_hip::probe() — lib.rs:188-207 (HipProbe: available, initialized, devices, error): tries init() and
 * reports instead of failing.  `error` receives the init failure text (empty when initialised); returns 0 always. */
typedef struct {
    int available;    /* a HIP runtime and at least one device answered */
    int initialized;  /* init() succeeded: device 0 is a gfx950 this library can run on */
    int device_count;
    char error[256];
} st_hip_probe_result;
int st_hip_probe(st_hip_probe_result *out);

/* Copies the calling thread's last error text (NUL-terminated, truncated to len) and returns its full
 * length.  Precedent: spiraltorch_last_error_* in bindings/spiraltorch-sys/src/lib.rs:149-185. */
size_t st_hip_last_error_message(char *buf, size_t len);

/* DeviceBuffer / HipStream RAII pairs of real.rs:649-667 and :190-220, flattened to C. */
int st_hip_malloc(void **device_ptr, size_t bytes);
int st_hip_free(void *device_ptr);
int st_hip_memcpy_h2d(void *device_dst, const void *host_src, size_t bytes, void *stream);
int st_hip_memcpy_d2h(void *host_dst, const void *device_src, size_t bytes, void *stream);
int st_hip_memset_zero(void *device_dst, size_t bytes, void *stream);
/* Host<->device copies made through this library since start (or since the last call with reset != 0):
 * {host-to-device copies, bytes, device-to-host copies, bytes}.  For callers and tests that check that tensors
 * stay resident between operators (the per-call traffic of crates/st-backend-hip/src/real.rs:718-756 is what a
 * resident tensor removes); the 16-byte status words of st_hip_count_nonfinite_f32_dev are not counted. */
int st_hip_transfer_counters(uint64_t counters[4], int reset);
int st_hip_stream_create(void **stream);
int st_hip_stream_synchronize(void *stream);
int st_hip_stream_destroy(void *stream);
int st_hip_device_synchronize(void);
/* Scratch memory (split-k partial sums, re-laid weights, padded operand copies) is kept per (stream, host thread) and
 * grows on demand; a buffer whose host thread has exited is re-used by the next thread that launches on that stream,
 * and st_hip_stream_destroy frees its stream's buffers.  st_hip_release_scratch waits for `stream` (NULL = the default
 * stream, which is never destroyed) and frees every scratch buffer kept for it; no other thread may be launching on
 * that stream meanwhile.  st_hip_scratch_buffer_count reports how many buffers are held in all.  No reference
 * counterpart: the reference allocates and frees per call (crates/st-backend-hip/src/real.rs:718-756). */
int st_hip_release_scratch(void *stream);
size_t st_hip_scratch_buffer_count(void);
/* Timing events recorded on the stream the kernels run on. */
int st_hip_event_create(void **event);
int st_hip_event_record(void *event, void *stream);
int st_hip_event_synchronize(void *event);
int st_hip_event_elapsed_ms(void *start, void *stop, float *milliseconds);
int st_hip_event_destroy(void *event);

/* ---- host-slice (drop-in) forms ----------------------------------------------------------- */

/* gemm_f32 / gemm_scaled_f32 / gemm_lhs_transpose_scaled_f32 — lib.rs:607-700.
 * out(m×n) = (lhs·rhs)·scale; lhs is m×k, or k×m when lhs_transposed != 0; rhs is k×n.
 * Errors (out untouched): "lhs buffer length {} does not match m*k={}", "rhs buffer length ...",
 * "output buffer length ...", "gemm scale must be finite, received {}", null pointers. */
int st_hip_gemm_f32(size_t m, size_t n, size_t k, float scale, int lhs_transposed,
                    const float *lhs, size_t lhs_len, const float *rhs, size_t rhs_len,
                    float *out, size_t out_len);

/* gemm_f32_raw — lib.rs:760-799: the raw-pointer form (host pointers, lengths implied by m, n, k).  Null pointers
 * are rejected ("gemm received a null pointer; provide contiguous row-major buffers", lib.rs:779-783), dimension
 * products are checked for overflow ("gemm dimensions overflow while constructing lhs slice" ...). */
int st_hip_gemm_f32_raw(size_t m, size_t n, size_t k, const float *lhs, const float *rhs, float *out);

/* gemm_bias_activation_f32 — lib.rs:700-720; epilogue semantics of lib.rs:572-605:
 * out = act((lhs·rhs + bias[col]) + residual).  residual may be NULL (residual_len ignored).
 * k == 0 still runs the epilogue on zeros (real.rs:869-871). */
int st_hip_gemm_bias_act_f32(size_t m, size_t n, size_t k, int activation, const float *lhs,
                             size_t lhs_len, const float *rhs, size_t rhs_len, const float *bias,
                             size_t bias_len, const float *residual, size_t residual_len,
                             float *out, size_t out_len);

/* out = act((lhs · B + bias) + residual) with B prepacked column-major, i.e. `packed_rhs` is the
 * n×k row-major transpose that PackedB::from_row_major builds (crates/st-tensor/src/pure.rs:1285-1323).
 * Replaces Tensor::matmul_prepacked[_bias]_with_backend (pure.rs:2559-2757), the path
 * crates/st-nn/src/layers/linear.rs:96-104 takes.  bias (length n) and residual (m*n) may be NULL with
 * length 0; activation may be ST_HIP_ACT_NONE. */
int st_hip_gemm_prepacked_bias_act_f32(size_t m, size_t n, size_t k, int activation,
                                       const float *lhs, size_t lhs_len, const float *packed_rhs,
                                       size_t packed_len, const float *bias, size_t bias_len,
                                       const float *residual, size_t residual_len, float *out,
                                       size_t out_len);

/* bf16 operands (raw bit patterns), f32 accumulate and output.  No reference counterpart (the
 * reference lists bf16 as roadmap in docs/backend_matrix.md); same slice contract as gemm_f32. */
int st_hip_gemm_bf16_f32acc(size_t m, size_t n, size_t k, const uint16_t *lhs, size_t lhs_len,
                            const uint16_t *rhs, size_t rhs_len, float *out, size_t out_len);

/* Conv2d::forward (+ bias, + optional activation) — crates/st-nn/src/layers/conv.rs:952-969,
 * 2559-2599: NCHW input (batch, c_in·h·w), OIHW weight (c_out, c_in·kh·kw), bias (c_out) or NULL,
 * NCHW output (batch, c_out·oh·ow) with oh/ow from conv.rs:685-700. */
int st_hip_conv2d_output_hw(size_t h, size_t w, size_t kh, size_t kw, size_t stride_h,
                            size_t stride_w, size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
                            size_t *oh, size_t *ow);
int st_hip_conv2d_bias_act_f32(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out,
                               size_t kh, size_t kw, size_t stride_h, size_t stride_w, size_t pad_h,
                               size_t pad_w, size_t dil_h, size_t dil_w, int activation,
                               const float *input, size_t input_len, const float *weight,
                               size_t weight_len, const float *bias, size_t bias_len, float *out,
                               size_t out_len);

/* Which kernel the dispatcher runs for a convolution.  The choice is made from the shape alone (plus 16-byte
 * alignment of the weight and output pointers, assumed here); st_hip_conv2d_planned_kernel reports it for the forward
 * pass (direction 0) or for grad_input of that forward shape (direction 1) as one of ST_HIP_CONV_KERNEL_*.
 * st_hip_conv2d_force_family is a process-wide diagnostic switch (the parity tests use it to run every family on
 * small shapes): with a family forced, a convolution whose shape that family cannot serve fails with
 * ST_HIP_ERR_UNSUPPORTED instead of silently running another kernel, and the query reports 0 for it.  No reference
 * counterpart (the reference has one CPU path, conv.rs:2559-2599). */
enum { ST_HIP_CONV_FAMILY_AUTO = 0, ST_HIP_CONV_FAMILY_TILE = 1, ST_HIP_CONV_FAMILY_RING = 2, ST_HIP_CONV_FAMILY_STRIP = 3 };
enum {
    ST_HIP_CONV_KERNEL_TILE = 1,         /* register-staged general kernel                                  */
    ST_HIP_CONV_KERNEL_RING = 2,         /* direct-to-LDS ring kernel                                       */
    ST_HIP_CONV_KERNEL_STRIP12 = 3,      /* strip kernel, weight rows padded to 12 words, 32-bit stores     */
    ST_HIP_CONV_KERNEL_STRIP12_WIDE = 4, /* the same with 128-bit stores through LDS                        */
    ST_HIP_CONV_KERNEL_STRIP9 = 5,       /* strip kernel, packed weight rows (more than 104 input channels) */
    ST_HIP_CONV_KERNEL_ADJOINT = 6,      /* grad_input only: adjoint gather (stride != 1 or padding > reach) */
    ST_HIP_CONV_KERNEL_COL2IM = 7,       /* grad_input only: per-image GEMM grad_outputᵀ·W, then a col2im gather  */
    ST_HIP_CONV_KERNEL_TILE_KSLICED = 8, /* few tiles, long reduction: general kernel cut along c_in·kh·kw + a sum */
    ST_HIP_CONV_KERNEL_DIRECT = 9        /* at most four output channels over many pixels: a thread per output pixel */
};
int st_hip_conv2d_force_family(int family);
int st_hip_conv2d_planned_kernel(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out, size_t kh,
                                 size_t kw, size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w,
                                 size_t dil_h, size_t dil_w, int direction, int *kernel);

/* Conv2d::backward, crates/st-nn/src/layers/conv.rs:780-813 with col2im :860-916: from the forward input
 * (N, C_in, H, W), the OIHW weight and grad_output (N, C_out, OH, OW) computes
 *   grad_input  (N, C_in, H, W)       = col2im(G · W)
 *   grad_weight (C_out, C_in·KH·KW)   = (Gᵀ · patches) / batch
 *   grad_bias   (C_out)               = column sums of G / batch
 * where G is grad_output viewed per pixel.  An empty batch is a no-op (:787-789). */
int st_hip_conv2d_backward_f32(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out, size_t kh,
                               size_t kw, size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w,
                               size_t dil_h, size_t dil_w, const float *input, size_t input_len,
                               const float *weight, size_t weight_len, const float *grad_output,
                               size_t grad_output_len, float *grad_input, size_t grad_input_len,
                               float *grad_weight, size_t grad_weight_len, float *grad_bias,
                               size_t grad_bias_len);

/* Tensor::scaled_dot_attention_with_backend — crates/st-tensor/src/pure.rs:4083-4354 with the CPU
 * kernel of :11845-11919.  q,k,v,out are (contexts·sequence, head_dim); z_bias (contexts, sequence)
 * or NULL; attn_bias (contexts·sequence, sequence) or NULL.  `causal` != 0 limits query i to keys
 * 0..=i (crates/st-core/src/backend/cuda_attention.cu:160-164).  Inputs and scale are checked finite
 * first (pure.rs:4148-4157), the output afterwards (:4206-4210); failures give
 * ST_HIP_ERR_NONFINITE with the reference's label in the message.  Empty volume returns zeros. */
int st_hip_attention_f32(size_t contexts, size_t sequence, size_t head_dim, float scale, int causal,
                         const float *q, size_t q_len, const float *k, size_t k_len, const float *v,
                         size_t v_len, const float *z_bias, size_t z_bias_len,
                         const float *attn_bias, size_t attn_bias_len, float *out, size_t out_len);

/* ---- launch arithmetic, computed on the host (no device is touched; usable without a GPU) ---- */

/* The kernels whose workgroups decode their index into (context, query tile, key chunk) are launched only after the
 * launcher has checked, with the decode function the kernel itself uses, that the grid is the product the decode
 * assumes and that its first and last workgroups land inside the operands (otherwise the call fails with
 * ST_HIP_ERR_RUNTIME and nothing is launched).  st_hip_attention_f32_launch_plan reports that plan for a shape and
 * additionally walks the whole grid: `items` distinct work items decoded, `items_expected` what the shape calls for,
 * `out_of_range` workgroups that would read outside the operands and `duplicates` items decoded twice (both must be
 * 0), `consistent` the launcher's own check.  No reference counterpart (the reference's CPU loop,
 * crates/st-tensor/src/pure.rs:11845-11919, has no launch geometry). */
enum { ST_HIP_ATTN_KERNEL_GENERAL = 1, ST_HIP_ATTN_KERNEL_FAST = 2, ST_HIP_ATTN_KERNEL_FAST_BIASED = 3, ST_HIP_ATTN_KERNEL_TINY = 4 };
typedef struct {
    int kernel;         /* ST_HIP_ATTN_KERNEL_* */
    int key_splits;     /* most key chunks a query tile is cut into (1: keys not split over workgroups) */
    int keys_per_split; /* keys per chunk */
    int consistent;     /* the check made before every launch passed */
    uint64_t workgroups, items, items_expected, out_of_range, duplicates;
} st_hip_attention_plan;
int st_hip_attention_f32_launch_plan(size_t contexts, size_t sequence, size_t head_dim, int causal, int biased,
                                     st_hip_attention_plan *plan);
/* The same for the 256-row bf16 GEMM kernels, whose workgroups decode their index into (k-split, tile): the tiling and
 * k-split launch_gemm would use for an m×n×k product (k a multiple of 64), the launcher's own check (`consistent`) and a
 * walk over the whole grid (`items` must equal `workgroups`, `out_of_range` and `duplicates` must be 0). */
typedef struct {
    int tile_cols;          /* 256 or 128 columns per tile (256 rows) */
    int tiles_m, tiles_n;
    int k_splits;           /* workgroups along k per tile (1: not split) */
    int k_tiles_per_split;  /* 64-wide k-tiles each of them walks */
    int consistent;
    uint64_t workgroups, items, out_of_range, duplicates;
} st_hip_gemm_tile_plan;
int st_hip_gemm_bf16_tile_plan(size_t m, size_t n, size_t k, st_hip_gemm_tile_plan *plan);
/* Rows of A per launch when a GEMM whose A is 2 GiB or larger is cut into row blocks for the kernels that address
 * operands through 32-bit byte offsets: a multiple of 256 with rows*k*element_bytes < 2^31, or 0 when 256 rows do not
 * fit (such products run on the kernels with 64-bit addressing). */
size_t st_hip_gemm_row_block(size_t k, size_t element_bytes);

/* ---- device-resident forms (caller owns device buffers; asynchronous on `stream`) ---------- */

int st_hip_gemm_f32_dev(size_t m, size_t n, size_t k, float scale, int lhs_transposed,
                        const float *lhs, const float *rhs, float *out, void *stream);
/* Replaces sgemm + st_gemm_epilogue_f32 (hip_gemm_epilogue.cu:46-71) with one fused launch. */
int st_hip_gemm_bias_act_f32_dev(size_t m, size_t n, size_t k, int activation, const float *lhs,
                                 const float *rhs, const float *bias, const float *residual,
                                 float *out, void *stream);
/* Device-resident form of st_hip_gemm_prepacked_bias_act_f32, and the packing itself done on the device:
 * packed(n×k) = rhs(k×n) transposed (PackedB::from_row_major, pure.rs:1299-1316). */
int st_hip_gemm_prepacked_bias_act_f32_dev(size_t m, size_t n, size_t k, int activation,
                                           const float *lhs, const float *packed_rhs,
                                           const float *bias, const float *residual, float *out,
                                           void *stream);
int st_hip_pack_rhs_f32_dev(size_t k, size_t n, const float *rhs, float *packed, void *stream);
int st_hip_gemm_bf16_f32acc_dev(size_t m, size_t n, size_t k, const uint16_t *lhs,
                                const uint16_t *rhs, float *out, void *stream);
/* bf16 GEMM with the fused epilogue act((lhs·rhs + bias) + residual); bias/residual may be NULL;
 * the result is written as f32 to out_f32 and/or rounded (nearest-even) to bf16 into out_bf16. */
int st_hip_gemm_bf16_bias_act_dev(size_t m, size_t n, size_t k, int activation,
                                  const uint16_t *lhs, const uint16_t *rhs, const float *bias,
                                  const float *residual, float *out_f32, uint16_t *out_bf16,
                                  void *stream);
/* The same with B prepacked as its n×k transpose — PackedB's column-major layout (crates/st-tensor/src/pure.rs:
 * 1285-1323; what Linear::forward passes, crates/st-nn/src/layers/linear.rs:96-104), in bf16 storage — and the packing
 * itself on the device.  With both operands k-contiguous neither needs transposing on its way to the matrix cores. */
int st_hip_gemm_bf16_prepacked_bias_act_dev(size_t m, size_t n, size_t k, int activation,
                                            const uint16_t *lhs, const uint16_t *packed_rhs,
                                            const float *bias, const float *residual, float *out_f32,
                                            uint16_t *out_bf16, void *stream);
/* Linear + residual + LayerNorm of a pre-norm transformer block in one call (block order of
 * crates/st-vision/src/models/vit.rs:256-265; Linear::forward, crates/st-nn/src/layers/linear.rs:87-107; layer_norm,
 * crates/st-tensor/src/pure.rs:4008-4058): out_f32 = (lhs·rhs + bias) + residual, the rows the next residual add needs,
 * and out_ln_bf16 = layer_norm(out_f32; gamma, beta, epsilon) rounded nearest-even to bf16, the operand of the next
 * projection.  bf16 lhs (m×k), rhs prepacked as its (n, k) transpose, f32 accumulation; bias (n) and residual (m×n)
 * may be NULL, gamma and beta (n) may not.  n = 512 with m > 64, k a multiple of 64 up to 1024, 16-byte aligned
 * buffers and no split of k in the plain GEMM's launch plan (few rows with a long k are split there) is a single
 * kernel whose workgroups own whole rows; any other shape runs the GEMM and the layer-norm kernel one after the other.  The single kernel adds the k products and a row's statistics in the order the tiled GEMM and
 * the layer-norm kernel use, so for its shapes it returns, bit for bit, what those two return. */
int st_hip_gemm_bf16_prepacked_residual_layer_norm_dev(size_t m, size_t n, size_t k, const uint16_t *lhs,
                                                      const uint16_t *packed_rhs, const float *bias,
                                                      const float *residual, const float *gamma, const float *beta,
                                                      float epsilon, float *out_f32, uint16_t *out_ln_bf16,
                                                      void *stream);
int st_hip_pack_rhs_bf16_dev(size_t k, size_t n, const uint16_t *rhs, uint16_t *packed, void *stream);
int st_hip_conv2d_bias_act_f32_dev(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out,
                                   size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                                   size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
                                   int activation, const float *input, const float *weight,
                                   const float *bias, float *out, void *stream);
/* Conv2d::forward (+ bias, + optional activation) on bf16 operands — the arithmetic of
 * crates/st-nn/src/layers/conv.rs:685-748, 2559-2599 with the image (NCHW) and the weight (OIHW) stored as bf16 bit
 * patterns, products accumulated in f32, f32 bias (or NULL), and the NCHW result written as f32 to out_f32 and/or rounded
 * nearest-even to bf16 into out_bf16 (either may be NULL, not both).  The reference has no bf16 path; this is the conv
 * counterpart of st_hip_gemm_bf16_bias_act_dev.  Any geometry the f32 entry point takes; the padded channels-last copy
 * of the input that the kernel works on (batch·(h+2·pad_h)·(w+2·pad_w)·ceil64(c_in)·2 bytes, in the stream's scratch)
 * must stay below 2 GiB, out_f32 must be 16-byte and out_bf16 8-byte aligned: otherwise ST_HIP_ERR_UNSUPPORTED. */
int st_hip_conv2d_bias_act_bf16_dev(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out,
                                    size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                                    size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
                                    int activation, const uint16_t *input, const uint16_t *weight,
                                    const float *bias, float *out_f32, uint16_t *out_bf16, void *stream);
/* The three gradients of Conv2d::backward one by one (conv.rs:791-809); grad_weight and grad_bias are
 * multiplied by `scale` (the reference passes 1/batch). */
int st_hip_conv2d_grad_input_f32_dev(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out,
                                     size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                                     size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
                                     const float *grad_output, const float *weight,
                                     float *grad_input, void *stream);
/* No counterpart in the reference.  st_hip_conv2d_grad_input_f32_dev for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): same arguments, but the
 * flipped weights the kernels read go to a static device array of ST_HIP_NOALLOC_SCRATCH_BYTES instead of the stream's
 * grow-on-demand workspace, and the call performs no hipMalloc / hipFree on any path.  The two routes of the allocating
 * entry point that need further scratch memory are not taken here: a long reduction over few tiles is not cut into
 * k-slices (st_hip_conv2d_planned_kernel reports ST_HIP_CONV_KERNEL_TILE_KSLICED for such shapes: same products, added
 * in another order, so results agree within the f32 parity bar, not bit for bit, and the call is slower), and strided
 * layers whose adjoint gather is wasteful do not go through the per-image GEMM + col2im route (reported as
 * ST_HIP_CONV_KERNEL_COL2IM: the gather kernel runs instead, correct but up to three orders of magnitude slower on
 * patch-embedding-like shapes — such callers should give the allocating entry point one warm-up call outside the
 * capture instead).  For every other shape the kernels, and the result bits, are those of the allocating entry point.
 * c_out*c_in*kh*kw*4 bytes must fit the array, otherwise ST_HIP_ERR_UNSUPPORTED (nothing is launched).  Every call on a
 * GPU shares that GPU's array: calls that overlap on one GPU (different streams or threads) race; calls on one stream
 * are ordered and safe.  st_hip_init must have succeeded first. */
#define ST_HIP_NOALLOC_SCRATCH_BYTES (16u << 20)
int st_hip_conv2d_grad_input_f32_noalloc_dev(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out,
                                             size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                                             size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
                                             const float *grad_output, const float *weight,
                                             float *grad_input, void *stream);
int st_hip_conv2d_grad_weight_f32_dev(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out,
                                      size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                                      size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
                                      const float *input, const float *grad_output, float scale,
                                      float *grad_weight, void *stream);
int st_hip_conv2d_grad_bias_f32_dev(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out,
                                    size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                                    size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
                                    const float *grad_output, float scale, float *grad_bias,
                                    void *stream);
int st_hip_attention_f32_dev(size_t contexts, size_t sequence, size_t head_dim, float scale,
                             int causal, const float *q, const float *k, const float *v,
                             const float *z_bias, const float *attn_bias, float *out, void *stream);
/* Attention on bf16 operands (both matrix products take bf16 inputs and accumulate in f32; the softmax
 * stays in f32; the result is rounded nearest-even to bf16), same recurrence as
 * crates/st-tensor/src/pure.rs:11845-11919 with `causal` limiting keys to 0..=query.  Heads are read in place
 * from row-major (batch*sequence, ld_in) matrices: context (b, h) owns columns h*head_dim .. +head_dim-1 of rows
 * b*sequence .. b*sequence+sequence-1 of q, k and v (the head slicing of
 * crates/st-vision/src/models/vit.rs:151-180), and writes the same columns of `out` (row stride ld_out).
 * A fused [Q | K | V] projection is passed as q = qkv, k = qkv + heads*head_dim, v = qkv + 2*heads*head_dim,
 * ld_in = 3*heads*head_dim; a (contexts*sequence, head_dim) layout as batch = contexts, heads = 1.
 * head_dim must be 64 or 128, ld_in a multiple of 8, ld_out a multiple of 4, q/k/v 16-byte aligned, out
 * 8-byte aligned; anything else returns ST_HIP_ERR_UNSUPPORTED. */
int st_hip_attention_bf16_dev(size_t batch, size_t heads, size_t sequence, size_t head_dim, float scale,
                              int causal, const uint16_t *q, const uint16_t *k, const uint16_t *v,
                              size_t ld_in, uint16_t *out, size_t ld_out, void *stream);

/* Tensor utilities the reference's HIP policy still leaves on the CPU (device pointers, async on `stream`).
 * row_softmax:   Tensor::row_softmax CPU path, crates/st-tensor/src/pure.rs:3277-3335 with
 *                cpu_row_softmax_hardmax :11930-11980 (NaN entries skipped, one-hot fallback when the
 *                denominator is not above f32 epsilon).
 * gelu_backward: out = gelu_prime(z) * grad, pure.rs:6454-6552, gelu_prime :12033-12040.
 * scale:         out = in * scale (out may alias in), pure.rs:5625-5700, scale_inplace :11993-11997;
 *                a non-finite scale is rejected like validate_scale_factor :5535-5543.
 * add_row:       data[r][c] += bias[c] in place, pure.rs:6196-6290.
 * sum_axis0:     out[c] = (sum over rows of in[r][c]) * scale, pure.rs:6999-7210 (scale 1 is sum_axis0). */
int st_hip_row_softmax_f32_dev(size_t rows, size_t cols, const float *in, float *out, void *stream);
/* gelu: out = gelu(in), Gelu::forward, crates/st-nn/src/layers/gelu.rs:78-94 (tanh form of pure.rs:12026-12031). */
int st_hip_gelu_f32_dev(size_t count, const float *in, float *out, void *stream);
/* The finite check the reference makes on every operator result (validate_finite_tensor_util_slice,
 * crates/st-tensor/src/pure.rs:5521-5533; call sites :2169, :4537, :4206-4210), for a tensor that lives on the
 * device: counts the non-finite values of `data` and reports the first one's index and value.  Synchronous on
 * `stream`; moves 16 bytes each way, whatever `count` is. */
int st_hip_count_nonfinite_f32_dev(size_t count, const float *data, uint64_t *nonfinite,
                                   uint64_t *first_index, float *first_value, void *stream);
int st_hip_gelu_backward_f32_dev(size_t count, const float *z, const float *grad, float *out,
                                 void *stream);
int st_hip_scale_f32_dev(size_t count, const float *in, float scale, float *out, void *stream);
int st_hip_add_row_f32_dev(size_t rows, size_t cols, float *data, const float *bias, void *stream);
int st_hip_sum_axis0_f32_dev(size_t rows, size_t cols, const float *in, float scale, float *out,
                             void *stream);

/* Row-wise building blocks of the decoder stack.
 * layer_norm: crates/st-tensor/src/pure.rs:4008-4058; writes f32 and/or bf16 (either may be NULL).
 * embedding:  crates/st-nn/src/layers/embedding.rs:42-100,325-330 (round, clamp, gather).
 * split_heads / merge_heads: (B·S, width) column slices <-> (B·H·S, D) contexts, the re-layout
 * crates/st-vision/src/models/vit.rs:151-180 performs by indexing. */
int st_hip_layer_norm_f32_dev(size_t rows, size_t cols, const float *x, const float *residual,
                              const float *gamma, const float *beta, float epsilon, float *out_f32,
                              uint16_t *out_bf16, void *stream);
int st_hip_embedding_f32_dev(size_t tokens, size_t vocab, size_t dim, const float *token_ids,
                             const float *table, float *out, void *stream);
int st_hip_f32_to_bf16_dev(size_t count, const float *in, uint16_t *out, void *stream);
int st_hip_split_heads_f32_dev(size_t batch, size_t seq, size_t heads, size_t head_dim,
                               const float *qkv, float *q, float *k, float *v, void *stream);
int st_hip_merge_heads_f32_dev(size_t batch, size_t seq, size_t heads, size_t head_dim,
                               const float *contexts_in, float *out_f32, uint16_t *out_bf16,
                               void *stream);

/* ---- measurement aid ---------------------------------------------------------------------------- */
/* A loop of nothing but bf16 matrix instructions (v_mfma_f32_32x32x16_bf16) on register operands: `workgroups` × 4
 * wavefronts each issue 32·iterations of them (2·32·32·16 flop each) on fragments read once from `operands` (device,
 * 32768 bf16 values, 16-byte aligned); `sink` (device, workgroups·256 floats) receives the sums so that nothing is
 * optimised away.  What the matrix pipes deliver on given operand bits with no memory instruction in the way — the
 * ceiling bench.py --probes reports beside the bf16 GEMM.  No reference counterpart. */
int st_hip_probe_mfma_bf16_dev(size_t workgroups, size_t iterations, const uint16_t *operands, float *sink, void *stream);
/* The same with the f32 matrix instruction (v_mfma_f32_32x32x2_f32, 2·32·32·2 flop each) of the f32 GEMM, convolution and
 * attention kernels; `operands` holds 4096 f32 values.  No reference counterpart. */
int st_hip_probe_mfma_f32_dev(size_t workgroups, size_t iterations, const float *operands, float *sink, void *stream);
/* A loop of nothing but direct-to-LDS loads: `workgroups` × 8 wavefronts each fetch 8·iterations KB of `region` (device,
 * region_bytes from 64 KiB to below 2 GiB) in the access shape of a bf16 operand k-tile (eight 128-byte rows, 1 KB apart, per
 * instruction; 8 to 16 KB in flight per wavefront), walking all of the region: the rate one compute unit streams at out of
 * L2, the memory-side cache or HBM, depending on region_bytes.  Nothing is written.  No reference counterpart. */
int st_hip_probe_stream_lds_dev(size_t workgroups, size_t iterations, const void *region, size_t region_bytes, void *stream);

/* ---- byte-level decoder stack (built from the ops above) ------------------------------------ */
typedef struct {
    size_t vocab, d_model, heads, layers, d_ff, batch, seq;
    float ln_eps;
} st_hip_decoder_config;
/* Number of f32 values in the flat weight blob: embed (vocab,d); per layer ln1_g, ln1_b,
 * w_qkv (d,3d), b_qkv, w_o (d,d), b_o, ln2_g, ln2_b, w_fc1 (d,ff), b_fc1, w_fc2 (ff,d), b_fc2;
 * then lnf_g, lnf_b, w_head (d,vocab), b_head.  Linear weights are (in, out) as in
 * crates/st-nn/src/layers/linear.rs:49-64. */
size_t st_hip_decoder_weight_count(const st_hip_decoder_config *config);
/* Uploads the weights (GEMM operands rounded once to bf16) and allocates all activations. */
int st_hip_decoder_create(const st_hip_decoder_config *config, const float *host_weights,
                          size_t weight_len, void **decoder);
/* tokens: device (batch·seq) f32 ids; logits: device (batch·seq, vocab) f32.  Asynchronous. */
int st_hip_decoder_forward_dev(void *decoder, const float *tokens, float *logits, void *stream);
int st_hip_decoder_destroy(void *decoder);

#ifdef __cplusplus
}
#endif
#endif /* ST_HIP_H */
