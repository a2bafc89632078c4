/*
 * st_oracle.h — CPU restatement of SpiralTorch's dense CPU path (TEST INFRASTRUCTURE ONLY).
 *
 * This library is the checker for the HIP backend: it restates, loop for loop, what the reference's
 * Rust CPU kernels compute (sequential-k f32 sums with separately rounded multiply and add, the
 * normalised online-softmax attention recurrence, im2col convolution, layer-norm).  It must never be
 * linked into, imported by, or called from the product path; only tests, the smoke check and the
 * CPU-baseline leg of the benchmark may use it.
 *
 * Every function returns 0 on success.  Attention and layer-norm return a positive label code when the
 * reference would raise NonFiniteValue (see ST_ORACLE_NONFINITE_*).
 */
#ifndef ST_ORACLE_H
#define ST_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    ST_ORACLE_ACT_NONE = 0,
    ST_ORACLE_ACT_RELU = 1, /* crates/st-backend-hip/src/lib.rs:29-34 */
    ST_ORACLE_ACT_GELU = 2
};

enum {
    ST_ORACLE_OK = 0,
    ST_ORACLE_BAD_ARGUMENT = -1,
    ST_ORACLE_NONFINITE_DOT = 1,         /* "scaled_dot_attention_dot"         */
    ST_ORACLE_NONFINITE_LOGIT = 2,       /* "scaled_dot_attention_logit"       */
    ST_ORACLE_NONFINITE_DENOM = 3,       /* "scaled_dot_attention_denom"       */
    ST_ORACLE_NONFINITE_WEIGHT = 4,      /* "scaled_dot_attention_weight"      */
    ST_ORACLE_NONFINITE_ACCUMULATOR = 5, /* "scaled_dot_attention_accumulator" */
    ST_ORACLE_NONFINITE_LAYER_NORM = 6
};

/* out(m×n) = (lhs·rhs)·scale, row-major.  lhs is m×k, or k×m when lhs_transposed != 0.
 * threads <= 1 runs serially; > 1 splits rows over that many OpenMP threads (values are unchanged:
 * every output element is still one left-to-right sum). */
int st_oracle_gemm_f32(size_t m, size_t n, size_t k, float scale, int lhs_transposed,
                       const float *lhs, const float *rhs, float *out, int threads);

/* The naive path on a prepacked rhs (n×k): sequential sums for the columns taken four at a time, the four-way
 * unrolled dot product for the cols % 4 columns left over (crates/st-tensor/src/pure.rs:11664-11758). */
int st_oracle_gemm_f32_packed_naive(size_t m, size_t n, size_t k, const float *lhs, const float *packed_rhs,
                                    float *out);

/* out = act((lhs·rhs + bias[col]) + residual), residual may be NULL; activation NONE/RELU/GELU. */
int st_oracle_gemm_bias_act_f32(size_t m, size_t n, size_t k, int activation, const float *lhs,
                                const float *rhs, const float *bias, const float *residual,
                                float *out, int threads);

/* bf16 operands (raw bit patterns) widened exactly to f32, then the same sequential-k f32 sum. */
int st_oracle_gemm_bf16_f32acc(size_t m, size_t n, size_t k, const uint16_t *lhs,
                               const uint16_t *rhs, float *out, int threads);

/* Output extent of the convolution; returns ST_ORACLE_BAD_ARGUMENT when the padded input is smaller
 * than the dilated kernel. */
int st_oracle_conv2d_output_hw(size_t h, size_t w, size_t kh, size_t kw, size_t stride_h,
                               size_t stride_w, size_t pad_h, size_t pad_w, size_t dil_h,
                               size_t dil_w, size_t *oh, size_t *ow);

/* NCHW input, OIHW weight, NCHW output; bias may be NULL (zeros). */
int st_oracle_conv2d_bias_act_f32(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out,
                                  size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                                  size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
                                  int activation, const float *input, const float *weight,
                                  const float *bias, float *out, int threads);

/* Conv2d backward (crates/st-nn/src/layers/conv.rs:750-813, 860-916): grad_input (N, C_in, H, W),
 * grad_weight (C_out, C_in·KH·KW) and grad_bias (C_out), the latter two multiplied by weight_scale
 * (the reference passes 1/batch).  Outputs may be NULL; `input` is only needed for grad_weight. */
int st_oracle_conv2d_backward_f32(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out,
                                  size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                                  size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
                                  const float *input, const float *weight, const float *grad_output,
                                  float weight_scale, float *grad_input, float *grad_weight,
                                  float *grad_bias);

/* q,k,v,out: (contexts·sequence, head_dim); z_bias (contexts, sequence) or NULL; attn_bias
 * (contexts·sequence, sequence) or NULL; causal != 0 restricts query i to keys 0..=i. */
int st_oracle_attention_f32(size_t contexts, size_t sequence, size_t head_dim, float scale,
                            int causal, const float *q, const float *k, const float *v,
                            const float *z_bias, const float *attn_bias, float *out, int threads);

/* Two-pass softmax(QKᵀ·scale + biases)·V evaluated in double precision (closed form used to pin the
 * recurrence above; not a restatement of reference code). */
int st_oracle_attention_f64(size_t contexts, size_t sequence, size_t head_dim, double scale,
                            int causal, const float *q, const float *k, const float *v,
                            const float *z_bias, const float *attn_bias, double *out);

int st_oracle_layer_norm_f32(size_t rows, size_t cols, const float *x, const float *residual,
                             const float *gamma, const float *beta, float epsilon, float *out);

/* Tensor utilities: row_softmax (pure.rs:11930-11986), gelu_backward (:12033-12040, :6549-6552),
 * scale (:11993-11997), add_row (:6284-6288), sum_axis0[_scaled] (:7201-7210). */
int st_oracle_row_softmax_f32(size_t rows, size_t cols, const float *in, float *out);
int st_oracle_gelu_backward_f32(size_t count, const float *z, const float *grad, float *out);
int st_oracle_scale_f32(size_t count, const float *in, float scale, float *out);
int st_oracle_add_row_f32(size_t rows, size_t cols, float *data, const float *bias);
int st_oracle_sum_axis0_f32(size_t rows, size_t cols, const float *in, float scale, float *out);

/* Token ids as f32 -> rows of table(vocab, dim); round, clamp to [0, vocab-1], non-finite -> 0. */
int st_oracle_embedding_f32(size_t tokens, size_t vocab, size_t dim, const float *token_ids,
                            const float *table, float *out);

float st_oracle_gelu(float x);

/* Round-to-nearest-even f32 -> bf16 bit pattern (NaN kept quiet). */
void st_oracle_f32_to_bf16(size_t n, const float *in, uint16_t *out);
void st_oracle_bf16_to_f32(size_t n, const uint16_t *in, float *out);

/* Byte-level pre-LN decoder forward.  Weights layout (all f32, row-major; GEMM operands are rounded
 * to bf16 at the points documented in st_oracle.c):
 *   embed (vocab, d)
 *   per layer: ln1_g (d), ln1_b (d), w_qkv (d, 3d), b_qkv (3d), w_o (d, d), b_o (d),
 *              ln2_g (d), ln2_b (d), w_fc1 (d, ff), b_fc1 (ff), w_fc2 (ff, d), b_fc2 (d)
 *   lnf_g (d), lnf_b (d), w_head (d, vocab), b_head (vocab)
 * tokens: (batch·seq) f32 ids.  logits: (batch·seq, vocab).  layers_to_run <= layers truncates the
 * stack (used to time a bounded sample). */
typedef struct {
    size_t vocab, d_model, heads, layers, d_ff, batch, seq;
    float ln_eps;
} st_oracle_decoder_config;

size_t st_oracle_decoder_weight_count(const st_oracle_decoder_config *cfg);
int st_oracle_decoder_forward(const st_oracle_decoder_config *cfg, const float *weights,
                              const float *tokens, size_t layers_to_run, float *logits,
                              int threads);

#ifdef __cplusplus
}
#endif
#endif /* ST_ORACLE_H */
