/*
 * st_oracle.c — CPU restatement of SpiralTorch's dense CPU path.  TEST INFRASTRUCTURE ONLY: the
 * HIP product path must never call into this file (see st_oracle.h).
 *
 * Build with FP contraction off (no FMA) and without fast-math: the reference is Rust, which rounds
 * every multiply and every add separately, and parity is owed to that arithmetic.
 *
 * All citations are paths below the reference checkout.
 *
 * Pinning status (checked in tests/test_oracle_*.py):
 *   gemm / scaled / lhs-transposed / bias+act   — reference known-answer vectors + float64 closed form
 *   packed naive gemm (dot_unrolled tail)       — bit-equal to the sequential gemm on the 4-column blocks, an
 *                                                 order-revealing vector (2^24 and ones) and float64 on the tail
 *   conv2d                                      — reference layout vector + float64 direct convolution
 *   attention                                   — reference vectors vs float64 two-pass softmax, invariants
 *   layer-norm, gelu, embedding, bf16 rounding  — textbook closed forms
 *   decoder forward                             — composition of the above; no reference counterpart
 *                                                 exists (the reference has no bf16 path), so the stack's
 *                                                 rounding points are this build's own definition.
 */
#include "st_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static int clamp_threads(int threads) { return threads < 1 ? 1 : threads; }

static int mul_overflows(size_t a, size_t b) { return b != 0 && a > (size_t)-1 / b; }

/* ------------------------------------------------------------------------------------------------
 * GEMM.  crates/st-tensor/src/backend/cpu_dense.rs:330-363 (microkernel_8x12_scalar) and :135-159
 * (scalar_block_with_packed): for every output element `acc = 0; for p in 0..k { acc += a*b }` and
 * `C += acc` onto a zero-filled C (cpu_dense.rs:626) — i.e. one strictly left-to-right f32 sum.
 * Scale is applied after the full sum (crates/st-tensor/src/pure.rs:2256-2262, scale_inplace
 * :11993-11997).  lhs-transposed form: pure.rs:11640-11662 (`acc * scale`).
 * The loop nest below is (row, p, col) so the compiler can vectorise over columns; each element's
 * sequence of operations is unchanged.
 * ---------------------------------------------------------------------------------------------- */
static void gemm_rows(size_t row_begin, size_t row_end, size_t m, size_t n, size_t k,
                      int lhs_transposed, const float *lhs, const float *rhs, float *out)
{
    for (size_t row = row_begin; row < row_end; ++row) {
        float *acc = out + row * n;
        for (size_t col = 0; col < n; ++col) acc[col] = 0.0f;
        for (size_t p = 0; p < k; ++p) {
            const float a = lhs_transposed ? lhs[p * m + row] : lhs[row * k + p];
            const float *b = rhs + p * n;
            for (size_t col = 0; col < n; ++col) {
                const float prod = a * b[col];
                acc[col] = acc[col] + prod;
            }
        }
    }
}

int st_oracle_gemm_f32(size_t m, size_t n, size_t k, float scale, int lhs_transposed,
                       const float *lhs, const float *rhs, float *out, int threads)
{
    if (mul_overflows(m, k) || mul_overflows(k, n) || mul_overflows(m, n)) return ST_ORACLE_BAD_ARGUMENT;
    if (!isfinite(scale)) return ST_ORACLE_BAD_ARGUMENT;
    if (m == 0 || n == 0) return ST_ORACLE_OK;
    threads = clamp_threads(threads);
#pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
    for (long long row = 0; row < (long long)m; ++row) {
        gemm_rows((size_t)row, (size_t)row + 1, m, n, k, lhs_transposed, lhs, rhs, out);
        if (scale != 1.0f) {
            float *dst = out + (size_t)row * n;
            for (size_t col = 0; col < n; ++col) dst[col] = dst[col] * scale;
        }
    }
    return ST_ORACLE_OK;
}

/* ------------------------------------------------------------------------------------------------
 * The naive CPU path on a prepacked rhs (PackedB, n×k with k contiguous): crates/st-tensor/src/pure.rs:11688-11758
 * (matmul_naive_packed_row).  Columns are taken four at a time (PACKED_MATMUL_COL_BLOCK, :11567), each with one
 * accumulator that adds its k products strictly in order — the same sequence as st_oracle_gemm_f32 —; the
 * cols % 4 columns left over go through dot_unrolled (:11664-11686): four partial sums over k ≡ 0,1,2,3 (mod 4),
 * added as ((acc0 + acc1) + acc2) + acc3, then the k % 4 tail products in order.
 * ---------------------------------------------------------------------------------------------- */
static float dot_unrolled(const float *lhs, const float *rhs, size_t len)
{
    float acc0 = 0.0f, acc1 = 0.0f, acc2 = 0.0f, acc3 = 0.0f;
    const size_t chunks = len / 4;
    for (size_t i = 0; i < chunks; ++i) {
        const size_t base = i * 4;
        const float p0 = lhs[base] * rhs[base];
        const float p1 = lhs[base + 1] * rhs[base + 1];
        const float p2 = lhs[base + 2] * rhs[base + 2];
        const float p3 = lhs[base + 3] * rhs[base + 3];
        acc0 = acc0 + p0;
        acc1 = acc1 + p1;
        acc2 = acc2 + p2;
        acc3 = acc3 + p3;
    }
    float sum = acc0 + acc1;
    sum = sum + acc2;
    sum = sum + acc3;
    for (size_t i = chunks * 4; i < len; ++i) {
        const float prod = lhs[i] * rhs[i];
        sum = sum + prod;
    }
    return sum;
}

int st_oracle_gemm_f32_packed_naive(size_t m, size_t n, size_t k, const float *lhs, const float *packed_rhs,
                                    float *out)
{
    if (mul_overflows(m, k) || mul_overflows(k, n) || mul_overflows(m, n)) return ST_ORACLE_BAD_ARGUMENT;
    for (size_t row = 0; row < m; ++row) {
        const float *lhs_row = lhs + row * k;
        float *dst = out + row * n;
        size_t col = 0;
        for (; col + 4 <= n; col += 4) {
            for (size_t j = 0; j < 4; ++j) {
                const float *column = packed_rhs + (col + j) * k;
                float acc = 0.0f;
                for (size_t p = 0; p < k; ++p) {
                    const float prod = lhs_row[p] * column[p];
                    acc = acc + prod;
                }
                dst[col + j] = acc;
            }
        }
        for (; col < n; ++col) dst[col] = dot_unrolled(lhs_row, packed_rhs + col * k, k);
    }
    return ST_ORACLE_OK;
}

/* crates/st-tensor/src/pure.rs:12026-12031 (gelu) — `x*x*x` evaluated left to right. */
float st_oracle_gelu(float x)
{
    const float coeff = 0.044715f;
    const float sqrt_2_over_pi = 0.7978846f;
    const float x_cubed = (x * x) * x;
    const float inner = sqrt_2_over_pi * (x + coeff * x_cubed);
    return (0.5f * x) * (1.0f + tanhf(inner));
}

/* crates/st-backend-hip/src/lib.rs:572-605 (apply_gemm_epilogue_stub) and
 * crates/st-tensor/src/pure.rs:12012-12096: value = (acc + bias) + residual; ReLU keeps value only
 * when `value > 0` (so -0.0 and NaN become +0.0). */
static float apply_activation(float value, int activation)
{
    switch (activation) {
    case ST_ORACLE_ACT_RELU:
        return value > 0.0f ? value : 0.0f;
    case ST_ORACLE_ACT_GELU:
        return st_oracle_gelu(value);
    default:
        return value;
    }
}

int st_oracle_gemm_bias_act_f32(size_t m, size_t n, size_t k, int activation, const float *lhs,
                                const float *rhs, const float *bias, const float *residual,
                                float *out, int threads)
{
    if (activation < ST_ORACLE_ACT_NONE || activation > ST_ORACLE_ACT_GELU) return ST_ORACLE_BAD_ARGUMENT;
    int rc = st_oracle_gemm_f32(m, n, k, 1.0f, 0, lhs, rhs, out, threads);
    if (rc != ST_ORACLE_OK) return rc;
    for (size_t row = 0; row < m; ++row) {
        for (size_t col = 0; col < n; ++col) {
            const size_t idx = row * n + col;
            float value = out[idx];
            if (bias) value = value + bias[col];
            if (residual) value = value + residual[idx];
            out[idx] = apply_activation(value, activation);
        }
    }
    return ST_ORACLE_OK;
}

static float bf16_bits_to_f32(uint16_t bits)
{
    uint32_t u = (uint32_t)bits << 16;
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

static uint16_t f32_to_bf16_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    const uint32_t rounding = 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)((u + rounding) >> 16);
}

void st_oracle_f32_to_bf16(size_t n, const float *in, uint16_t *out)
{
    for (size_t i = 0; i < n; ++i) out[i] = f32_to_bf16_bits(in[i]);
}

void st_oracle_bf16_to_f32(size_t n, const uint16_t *in, float *out)
{
    for (size_t i = 0; i < n; ++i) out[i] = bf16_bits_to_f32(in[i]);
}

/* A product of two bf16 values is exact in f32, so this is the f32 GEMM above on widened operands. */
int st_oracle_gemm_bf16_f32acc(size_t m, size_t n, size_t k, const uint16_t *lhs,
                               const uint16_t *rhs, float *out, int threads)
{
    if (mul_overflows(m, k) || mul_overflows(k, n) || mul_overflows(m, n)) return ST_ORACLE_BAD_ARGUMENT;
    if (m == 0 || n == 0) return ST_ORACLE_OK;
    float *rhs_f = (float *)malloc((k * n + 1) * sizeof(float));
    if (!rhs_f) return ST_ORACLE_BAD_ARGUMENT;
    st_oracle_bf16_to_f32(k * n, rhs, rhs_f);
    threads = clamp_threads(threads);
#pragma omp parallel num_threads(threads) if (threads > 1)
    {
        float *lhs_row = (float *)malloc((k + 1) * sizeof(float));
#pragma omp for schedule(static)
        for (long long row = 0; row < (long long)m; ++row) {
            st_oracle_bf16_to_f32(k, lhs + (size_t)row * k, lhs_row);
            gemm_rows(0, 1, 1, n, k, 0, lhs_row, rhs_f, out + (size_t)row * n);
        }
        free(lhs_row);
    }
    free(rhs_f);
    return ST_ORACLE_OK;
}

/* ------------------------------------------------------------------------------------------------
 * Conv2d.  crates/st-nn/src/layers/conv.rs:685-700 (output_hw, dilated_extent :106-114),
 * :702-748 (im2col: patch column s = (ic*KH + ky)*KW + kx, zero outside the image),
 * :155-197 + :2559-2599 (einsum "ps,os->po": acc = 0; acc += patch[s]*w[o][s] for s ascending;
 * then + bias[o]), :918-948 (store into NCHW: out[b, o*OH*OW + sp]).
 * ---------------------------------------------------------------------------------------------- */
int st_oracle_conv2d_output_hw(size_t h, size_t w, size_t kh, size_t kw, size_t stride_h,
                               size_t stride_w, size_t pad_h, size_t pad_w, size_t dil_h,
                               size_t dil_w, size_t *oh, size_t *ow)
{
    if (kh == 0 || kw == 0 || stride_h == 0 || stride_w == 0 || dil_h == 0 || dil_w == 0 || h == 0 ||
        w == 0)
        return ST_ORACLE_BAD_ARGUMENT;
    const size_t eff_kh = (kh - 1) * dil_h + 1;
    const size_t eff_kw = (kw - 1) * dil_w + 1;
    if (h + 2 * pad_h < eff_kh || w + 2 * pad_w < eff_kw) return ST_ORACLE_BAD_ARGUMENT;
    *oh = (h + 2 * pad_h - eff_kh) / stride_h + 1;
    *ow = (w + 2 * pad_w - eff_kw) / stride_w + 1;
    return ST_ORACLE_OK;
}

int st_oracle_conv2d_bias_act_f32(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out,
                                  size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                                  size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
                                  int activation, const float *input, const float *weight,
                                  const float *bias, float *out, int threads)
{
    size_t oh, ow;
    if (c_in == 0 || c_out == 0) return ST_ORACLE_BAD_ARGUMENT;
    int rc = st_oracle_conv2d_output_hw(h, w, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w,
                                        &oh, &ow);
    if (rc != ST_ORACLE_OK) return rc;
    const size_t span = c_in * kh * kw;
    const size_t spatial = oh * ow;
    /* weight transposed once to (span, c_out) so the inner loop runs over output channels; the
     * per-element order (s ascending) is unchanged. */
    float *wt = (float *)malloc(span * c_out * sizeof(float));
    if (!wt) return ST_ORACLE_BAD_ARGUMENT;
    for (size_t o = 0; o < c_out; ++o)
        for (size_t s = 0; s < span; ++s) wt[s * c_out + o] = weight[o * span + s];
    threads = clamp_threads(threads);
    const long long total_pixels = (long long)(batch * spatial);
#pragma omp parallel num_threads(threads) if (threads > 1)
    {
        float *patch = (float *)malloc(span * sizeof(float));
        float *acc = (float *)malloc(c_out * sizeof(float));
#pragma omp for schedule(static)
        for (long long pix = 0; pix < total_pixels; ++pix) {
            const size_t b = (size_t)pix / spatial;
            const size_t sp = (size_t)pix % spatial;
            const size_t oy = sp / ow, ox = sp % ow;
            const float *image = input + b * c_in * h * w;
            size_t s = 0;
            for (size_t ic = 0; ic < c_in; ++ic)
                for (size_t ky = 0; ky < kh; ++ky)
                    for (size_t kx = 0; kx < kw; ++kx, ++s) {
                        const long long iy = (long long)(oy * stride_h + ky * dil_h) - (long long)pad_h;
                        const long long ix = (long long)(ox * stride_w + kx * dil_w) - (long long)pad_w;
                        patch[s] = (iy < 0 || ix < 0 || iy >= (long long)h || ix >= (long long)w)
                                       ? 0.0f
                                       : image[ic * h * w + (size_t)iy * w + (size_t)ix];
                    }
            for (size_t o = 0; o < c_out; ++o) acc[o] = 0.0f;
            for (s = 0; s < span; ++s) {
                const float p = patch[s];
                const float *wrow = wt + s * c_out;
                for (size_t o = 0; o < c_out; ++o) {
                    const float prod = p * wrow[o];
                    acc[o] = acc[o] + prod;
                }
            }
            for (size_t o = 0; o < c_out; ++o) {
                float value = acc[o];
                if (bias) value = value + bias[o];
                out[(b * c_out + o) * spatial + sp] = apply_activation(value, activation);
            }
        }
        free(patch);
        free(acc);
    }
    free(wt);
    return ST_ORACLE_OK;
}

/* Conv2d backward, crates/st-nn/src/layers/conv.rs:750-813 and :860-916:
 *   G (batch·OH·OW, C_out) is grad_output re-laid per pixel (:750-778);
 *   grad_weight = (Gᵀ · patches) · weight_scale  — matmul_lhs_transpose_scaled (:791-795), k = pixel index ascending;
 *   grad_bias   = (column sums of G) · weight_scale (:796-799);
 *   grad_input  = col2im(G · W): grad_patches[p][s] = Σ_o G[p][o]·W[o][s] (o ascending), scattered with += in the
 *   loop order of col2im (:880-912).  The reference passes weight_scale = 1/batch.  Any output may be NULL. */
int st_oracle_conv2d_backward_f32(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out,
                                  size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                                  size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
                                  const float *input, const float *weight, const float *grad_output,
                                  float weight_scale, float *grad_input, float *grad_weight, float *grad_bias)
{
    size_t oh, ow;
    if (c_in == 0 || c_out == 0) return ST_ORACLE_BAD_ARGUMENT;
    int rc = st_oracle_conv2d_output_hw(h, w, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, &oh, &ow);
    if (rc != ST_ORACLE_OK) return rc;
    const size_t span = c_in * kh * kw, spatial = oh * ow;
    if (grad_input) memset(grad_input, 0, batch * c_in * h * w * sizeof(float));
    if (grad_weight) memset(grad_weight, 0, c_out * span * sizeof(float));
    if (grad_bias) memset(grad_bias, 0, c_out * sizeof(float));
    float *patch = (float *)malloc((span ? span : 1) * sizeof(float));
    float *grad_patch = (float *)malloc((span ? span : 1) * sizeof(float));
    if (!patch || !grad_patch) { free(patch); free(grad_patch); return ST_ORACLE_BAD_ARGUMENT; }
    for (size_t b = 0; b < batch; ++b)
        for (size_t oy = 0; oy < oh; ++oy)
            for (size_t ox = 0; ox < ow; ++ox) {
                const size_t sp = oy * ow + ox;
                const float *g = grad_output + b * c_out * spatial + sp;  /* G[p][o] = g[o*spatial] */
                if (grad_weight && input) {
                    size_t s = 0;
                    const float *image = input + b * c_in * h * w;
                    for (size_t ic = 0; ic < c_in; ++ic)
                        for (size_t ky = 0; ky < kh; ++ky)
                            for (size_t kx = 0; kx < kw; ++kx, ++s) {
                                const long long iy = (long long)(oy * stride_h + ky * dil_h) - (long long)pad_h;
                                const long long ix = (long long)(ox * stride_w + kx * dil_w) - (long long)pad_w;
                                patch[s] = (iy < 0 || ix < 0 || iy >= (long long)h || ix >= (long long)w)
                                               ? 0.0f
                                               : image[ic * h * w + (size_t)iy * w + (size_t)ix];
                            }
                    for (size_t o = 0; o < c_out; ++o) {
                        const float go = g[o * spatial];
                        float *row = grad_weight + o * span;
                        for (s = 0; s < span; ++s) {
                            const float prod = go * patch[s];
                            row[s] = row[s] + prod;
                        }
                    }
                }
                if (grad_bias)
                    for (size_t o = 0; o < c_out; ++o) grad_bias[o] = grad_bias[o] + g[o * spatial];
                if (grad_input) {
                    for (size_t s = 0; s < span; ++s) grad_patch[s] = 0.0f;
                    for (size_t o = 0; o < c_out; ++o) {
                        const float go = g[o * spatial];
                        const float *wrow = weight + o * span;
                        for (size_t s = 0; s < span; ++s) {
                            const float prod = go * wrow[s];
                            grad_patch[s] = grad_patch[s] + prod;
                        }
                    }
                    float *gin = grad_input + b * c_in * h * w;
                    size_t s = 0;
                    for (size_t ic = 0; ic < c_in; ++ic)
                        for (size_t ky = 0; ky < kh; ++ky)
                            for (size_t kx = 0; kx < kw; ++kx, ++s) {
                                const long long iy = (long long)(oy * stride_h + ky * dil_h) - (long long)pad_h;
                                const long long ix = (long long)(ox * stride_w + kx * dil_w) - (long long)pad_w;
                                if (iy < 0 || ix < 0 || iy >= (long long)h || ix >= (long long)w) continue;
                                float *dst = gin + ic * h * w + (size_t)iy * w + (size_t)ix;
                                *dst = *dst + grad_patch[s];
                            }
                }
            }
    if (grad_weight)
        for (size_t i = 0; i < c_out * span; ++i) grad_weight[i] = grad_weight[i] * weight_scale;
    if (grad_bias)
        for (size_t o = 0; o < c_out; ++o) grad_bias[o] = grad_bias[o] * weight_scale;
    free(patch);
    free(grad_patch);
    return ST_ORACLE_OK;
}

/* ------------------------------------------------------------------------------------------------
 * Attention.  crates/st-tensor/src/pure.rs:11845-11919 (fused_attention_cpu): normalised online
 * softmax, one key at a time, a finite check after every scalar step.  `causal` restricts the key
 * loop to 0..=query, the definition used by the reference's CUDA kernel
 * (crates/st-core/src/backend/cuda_attention.cu:160-164).
 * ---------------------------------------------------------------------------------------------- */
static int attention_context(size_t context, size_t sequence, size_t head_dim, float scale, int causal,
                             const float *q, const float *k, const float *v, const float *z_bias,
                             const float *attn_bias, float *out, float *accum)
{
    const size_t context_offset = context * sequence;
    for (size_t query_idx = 0; query_idx < sequence; ++query_idx) {
        for (size_t d = 0; d < head_dim; ++d) accum[d] = 0.0f;
        float running_max = -INFINITY;
        float running_sum = 0.0f;
        const size_t query_row = context_offset + query_idx;
        const size_t query_offset = query_row * head_dim;
        const size_t key_end = causal ? query_idx + 1 : sequence;
        for (size_t key_idx = 0; key_idx < key_end; ++key_idx) {
            const size_t key_offset = (context_offset + key_idx) * head_dim;
            float dot = 0.0f;
            for (size_t d = 0; d < head_dim; ++d) {
                const float prod = q[query_offset + d] * k[key_offset + d];
                dot = dot + prod;
                if (!isfinite(dot)) return ST_ORACLE_NONFINITE_DOT;
            }
            float logit = dot * scale;
            if (!isfinite(logit)) return ST_ORACLE_NONFINITE_LOGIT;
            if (z_bias) {
                logit = logit + z_bias[context_offset + key_idx];
                if (!isfinite(logit)) return ST_ORACLE_NONFINITE_LOGIT;
            }
            if (attn_bias) {
                logit = logit + attn_bias[query_row * sequence + key_idx];
                if (!isfinite(logit)) return ST_ORACLE_NONFINITE_LOGIT;
            }
            const float new_max = running_max > logit ? running_max : logit; /* f32::max, finite logit */
            const float scaled_sum = running_sum > 0.0f ? running_sum * expf(running_max - new_max) : 0.0f;
            const float exp_curr = expf(logit - new_max);
            const float denom = scaled_sum + exp_curr;
            if (!isfinite(denom)) return ST_ORACLE_NONFINITE_DENOM;
            const float alpha = denom > 0.0f ? scaled_sum / denom : 0.0f;
            const float weight = denom > 0.0f ? exp_curr / denom : 0.0f;
            if (!isfinite(alpha) || !isfinite(weight)) return ST_ORACLE_NONFINITE_WEIGHT;
            running_max = new_max;
            running_sum = denom;
            for (size_t d = 0; d < head_dim; ++d) {
                const float kept = accum[d] * alpha;
                const float added = weight * v[key_offset + d];
                accum[d] = kept + added;
                if (!isfinite(accum[d])) return ST_ORACLE_NONFINITE_ACCUMULATOR;
            }
        }
        memcpy(out + query_offset, accum, head_dim * sizeof(float));
    }
    return ST_ORACLE_OK;
}

int st_oracle_attention_f32(size_t contexts, size_t sequence, size_t head_dim, float scale,
                            int causal, const float *q, const float *k, const float *v,
                            const float *z_bias, const float *attn_bias, float *out, int threads)
{
    if (mul_overflows(contexts, sequence) || mul_overflows(contexts * sequence, head_dim))
        return ST_ORACLE_BAD_ARGUMENT;
    if (!isfinite(scale)) return ST_ORACLE_BAD_ARGUMENT;
    if (contexts * sequence == 0 || head_dim == 0) return ST_ORACLE_OK;
    threads = clamp_threads(threads);
    int status = ST_ORACLE_OK;
#pragma omp parallel num_threads(threads) if (threads > 1)
    {
        float *accum = (float *)malloc(head_dim * sizeof(float));
#pragma omp for schedule(dynamic, 1)
        for (long long context = 0; context < (long long)contexts; ++context) {
            int rc = attention_context((size_t)context, sequence, head_dim, scale, causal, q, k, v,
                                       z_bias, attn_bias, out, accum);
            if (rc != ST_ORACLE_OK) {
#pragma omp critical
                if (status == ST_ORACLE_OK) status = rc;
            }
        }
        free(accum);
    }
    return status;
}

int st_oracle_attention_f64(size_t contexts, size_t sequence, size_t head_dim, double scale,
                            int causal, const float *q, const float *k, const float *v,
                            const float *z_bias, const float *attn_bias, double *out)
{
    if (contexts * sequence == 0 || head_dim == 0) return ST_ORACLE_OK;
    double *logits = (double *)malloc(sequence * sizeof(double));
    if (!logits) return ST_ORACLE_BAD_ARGUMENT;
    for (size_t c = 0; c < contexts; ++c) {
        for (size_t i = 0; i < sequence; ++i) {
            const size_t qrow = c * sequence + i;
            const size_t key_end = causal ? i + 1 : sequence;
            double max_logit = -INFINITY;
            for (size_t j = 0; j < key_end; ++j) {
                const size_t krow = c * sequence + j;
                double dot = 0.0;
                for (size_t d = 0; d < head_dim; ++d)
                    dot += (double)q[qrow * head_dim + d] * (double)k[krow * head_dim + d];
                double logit = dot * scale;
                if (z_bias) logit += (double)z_bias[c * sequence + j];
                if (attn_bias) logit += (double)attn_bias[qrow * sequence + j];
                logits[j] = logit;
                if (logit > max_logit) max_logit = logit;
            }
            double denom = 0.0;
            for (size_t j = 0; j < key_end; ++j) {
                logits[j] = exp(logits[j] - max_logit);
                denom += logits[j];
            }
            for (size_t d = 0; d < head_dim; ++d) {
                double acc = 0.0;
                for (size_t j = 0; j < key_end; ++j)
                    acc += logits[j] * (double)v[(c * sequence + j) * head_dim + d];
                out[qrow * head_dim + d] = acc / denom;
            }
        }
    }
    free(logits);
    return ST_ORACLE_OK;
}

/* crates/st-tensor/src/pure.rs:11930-11986 (cpu_row_softmax_hardmax, softmax half). */
int st_oracle_row_softmax_f32(size_t rows, size_t cols, const float *in, float *out)
{
    for (size_t row = 0; row < rows; ++row) {
        const float *x = in + row * cols;
        float *y = out + row * cols;
        float max_value = -INFINITY;
        size_t max_index = 0;
        int found = 0;
        for (size_t i = 0; i < cols; ++i) {
            const float value = x[i];
            if (isnan(value)) continue;
            if (!found || value > max_value) {
                max_value = value;
                max_index = i;
                found = 1;
            }
        }
        const float base = (found && isfinite(max_value)) ? max_value : 0.0f;
        float denom = 0.0f;
        for (size_t i = 0; i < cols; ++i) {
            const float weight = (!found || isnan(x[i])) ? 0.0f : expf(x[i] - base);
            y[i] = weight;
            denom = denom + weight;
        }
        if (found) {
            if (isfinite(denom) && denom > FLT_EPSILON) {
                const float inv = 1.0f / denom;
                for (size_t i = 0; i < cols; ++i) y[i] = y[i] * inv;
            } else {
                for (size_t i = 0; i < cols; ++i) y[i] = 0.0f;
                y[max_index] = 1.0f;
            }
        }
    }
    return ST_ORACLE_OK;
}

/* crates/st-tensor/src/pure.rs:12033-12040 (gelu_prime) times the incoming gradient (:6549-6552). */
int st_oracle_gelu_backward_f32(size_t count, const float *z, const float *grad, float *out)
{
    const float sqrt_2_over_pi = 0.7978846f, kappa = 0.044715f;
    for (size_t i = 0; i < count; ++i) {
        const float x = z[i];
        const float x2 = x * x;
        const float inner = sqrt_2_over_pi * (x + (kappa * x) * x2);
        const float t = tanhf(inner);
        const float left = 0.5f * (1.0f + t);
        const float right = (((0.5f * x) * (1.0f - t * t)) * sqrt_2_over_pi) * (1.0f + (3.0f * kappa) * x2);
        out[i] = (left + right) * grad[i];
    }
    return ST_ORACLE_OK;
}

/* crates/st-tensor/src/pure.rs:11993-11997 (scale_inplace). */
int st_oracle_scale_f32(size_t count, const float *in, float scale, float *out)
{
    for (size_t i = 0; i < count; ++i) out[i] = in[i] * scale;
    return ST_ORACLE_OK;
}

/* crates/st-tensor/src/pure.rs:6284-6288 (add_row_inplace: value += bias per column). */
int st_oracle_add_row_f32(size_t rows, size_t cols, float *data, const float *bias)
{
    for (size_t r = 0; r < rows; ++r)
        for (size_t c = 0; c < cols; ++c) data[r * cols + c] = data[r * cols + c] + bias[c];
    return ST_ORACLE_OK;
}

/* crates/st-tensor/src/pure.rs:7201-7210 (sum_axis0_scaled: rows added in order, then one multiply). */
int st_oracle_sum_axis0_f32(size_t rows, size_t cols, const float *in, float scale, float *out)
{
    for (size_t c = 0; c < cols; ++c) out[c] = 0.0f;
    for (size_t r = 0; r < rows; ++r)
        for (size_t c = 0; c < cols; ++c) out[c] = out[c] + in[r * cols + c];
    for (size_t c = 0; c < cols; ++c) out[c] = out[c] * scale;
    return ST_ORACLE_OK;
}

/* crates/st-tensor/src/pure.rs:4008-4058 (layer_norm_cpu). */
int st_oracle_layer_norm_f32(size_t rows, size_t cols, const float *x, const float *residual,
                             const float *gamma, const float *beta, float epsilon, float *out)
{
    const float cols_f = (float)cols;
    for (size_t r = 0; r < rows; ++r) {
        const size_t offset = r * cols;
        float sum = 0.0f, sumsq = 0.0f;
        for (size_t c = 0; c < cols; ++c) {
            float v = x[offset + c];
            if (residual) v = v + residual[offset + c];
            if (!isfinite(v)) return ST_ORACLE_NONFINITE_LAYER_NORM;
            sum = sum + v;
            const float sq = v * v;
            sumsq = sumsq + sq;
            if (!isfinite(sum) || !isfinite(sumsq)) return ST_ORACLE_NONFINITE_LAYER_NORM;
        }
        const float mean = sum / cols_f;
        const float mean_sq = mean * mean;
        const float raw_var = sumsq / cols_f - mean_sq;
        if (!isfinite(mean) || !isfinite(raw_var)) return ST_ORACLE_NONFINITE_LAYER_NORM;
        const float var = raw_var > 0.0f ? raw_var : 0.0f;
        const float denom = sqrtf(var + epsilon);
        if (!isfinite(denom)) return ST_ORACLE_NONFINITE_LAYER_NORM;
        for (size_t c = 0; c < cols; ++c) {
            float v = x[offset + c];
            if (residual) v = v + residual[offset + c];
            const float normed = (v - mean) / denom;
            const float scaled = normed * gamma[c];
            out[offset + c] = scaled + beta[c];
            if (!isfinite(out[offset + c])) return ST_ORACLE_NONFINITE_LAYER_NORM;
        }
    }
    return ST_ORACLE_OK;
}

/* crates/st-nn/src/layers/embedding.rs:42-100 (token_to_index) and :325-330 (row gather). */
int st_oracle_embedding_f32(size_t tokens, size_t vocab, size_t dim, const float *token_ids,
                            const float *table, float *out)
{
    if (vocab == 0) return ST_ORACLE_BAD_ARGUMENT;
    for (size_t t = 0; t < tokens; ++t) {
        const float value = token_ids[t];
        size_t idx = 0;
        if (isfinite(value)) {
            const float rounded = roundf(value);
            if (rounded > 0.0f) {
                idx = rounded >= (float)vocab ? vocab - 1 : (size_t)rounded;
                if (idx > vocab - 1) idx = vocab - 1;
            }
        }
        memcpy(out + t * dim, table + idx * dim, dim * sizeof(float));
    }
    return ST_ORACLE_OK;
}

/* ------------------------------------------------------------------------------------------------
 * Decoder forward (no reference counterpart; composed from the restated ops in the block order of
 * crates/st-vision/src/models/vit.rs:256-265: h = x + Attn(LN1(x)); y = h + FC2(GELU(FC1(LN2(h))))).
 * Linear layers follow crates/st-nn/src/layers/linear.rs:49-64,96-104: W is (in, out), y = x·W + b.
 * Rounding points of the bf16 build: every GEMM rounds BOTH operands to bf16 (RNE) and accumulates
 * in f32; bias, residual, GELU and layer-norm run in f32.  The attention's q, k and v are GEMM operands
 * as well and are rounded to bf16 after the projection's bias add; its softmax recurrence runs in f32
 * (a device kernel that also rounds the softmax weights to bf16 before the value product differs from
 * this by rounding noise only).
 * ---------------------------------------------------------------------------------------------- */
size_t st_oracle_decoder_weight_count(const st_oracle_decoder_config *c)
{
    const size_t d = c->d_model, ff = c->d_ff;
    const size_t per_layer = 2 * d + d * 3 * d + 3 * d + d * d + d + 2 * d + d * ff + ff + ff * d + d;
    return c->vocab * d + c->layers * per_layer + 2 * d + d * c->vocab + c->vocab;
}

static void round_to_bf16_inplace(size_t n, const float *in, uint16_t *out) { st_oracle_f32_to_bf16(n, in, out); }

/* out(rows×n) = act(bf16(x)·bf16(w) + b (+ residual)) */
static int linear_bf16(size_t rows, size_t in_dim, size_t out_dim, const float *x, const float *w,
                       const float *b, const float *residual, int activation, float *out, int threads)
{
    uint16_t *xb = (uint16_t *)malloc(rows * in_dim * sizeof(uint16_t));
    uint16_t *wb = (uint16_t *)malloc(in_dim * out_dim * sizeof(uint16_t));
    if (!xb || !wb) { free(xb); free(wb); return ST_ORACLE_BAD_ARGUMENT; }
    round_to_bf16_inplace(rows * in_dim, x, xb);
    round_to_bf16_inplace(in_dim * out_dim, w, wb);
    int rc = st_oracle_gemm_bf16_f32acc(rows, out_dim, in_dim, xb, wb, out, threads);
    free(xb);
    free(wb);
    if (rc != ST_ORACLE_OK) return rc;
    for (size_t r = 0; r < rows; ++r)
        for (size_t c = 0; c < out_dim; ++c) {
            const size_t idx = r * out_dim + c;
            float value = out[idx] + b[c];
            if (residual) value = value + residual[idx];
            out[idx] = apply_activation(value, activation);
        }
    return ST_ORACLE_OK;
}

int st_oracle_decoder_forward(const st_oracle_decoder_config *cfg, const float *weights,
                              const float *tokens, size_t layers_to_run, float *logits, int threads)
{
    const size_t d = cfg->d_model, ff = cfg->d_ff, heads = cfg->heads, vocab = cfg->vocab;
    const size_t batch = cfg->batch, seq = cfg->seq, T = batch * seq;
    if (heads == 0 || d % heads != 0) return ST_ORACLE_BAD_ARGUMENT;
    const size_t hd = d / heads;
    if (layers_to_run > cfg->layers) layers_to_run = cfg->layers;
    const float scale = 1.0f / sqrtf((float)hd);

    float *x = (float *)malloc(T * d * sizeof(float));
    float *h = (float *)malloc(T * d * sizeof(float));
    float *qkv = (float *)malloc(T * 3 * d * sizeof(float));
    float *qh = (float *)malloc(T * d * sizeof(float));
    float *kh = (float *)malloc(T * d * sizeof(float));
    float *vh = (float *)malloc(T * d * sizeof(float));
    float *ah = (float *)malloc(T * d * sizeof(float));
    float *attn = (float *)malloc(T * d * sizeof(float));
    float *u = (float *)malloc(T * ff * sizeof(float));
    float *x2 = (float *)malloc(T * d * sizeof(float));
    int rc = ST_ORACLE_BAD_ARGUMENT;
    if (!x || !h || !qkv || !qh || !kh || !vh || !ah || !attn || !u || !x2) goto done;

    const float *p = weights;
    const float *embed = p; p += vocab * d;
    rc = st_oracle_embedding_f32(T, vocab, d, tokens, embed, x);
    if (rc) goto done;

    for (size_t layer = 0; layer < cfg->layers; ++layer) {
        const float *ln1_g = p; p += d;
        const float *ln1_b = p; p += d;
        const float *w_qkv = p; p += d * 3 * d;
        const float *b_qkv = p; p += 3 * d;
        const float *w_o = p; p += d * d;
        const float *b_o = p; p += d;
        const float *ln2_g = p; p += d;
        const float *ln2_b = p; p += d;
        const float *w_fc1 = p; p += d * ff;
        const float *b_fc1 = p; p += ff;
        const float *w_fc2 = p; p += ff * d;
        const float *b_fc2 = p; p += d;
        if (layer >= layers_to_run) continue;

        rc = st_oracle_layer_norm_f32(T, d, x, NULL, ln1_g, ln1_b, cfg->ln_eps, h);
        if (rc) goto done;
        rc = linear_bf16(T, d, 3 * d, h, w_qkv, b_qkv, NULL, ST_ORACLE_ACT_NONE, qkv, threads);
        if (rc) goto done;
        /* The attention's two matrix products are GEMMs too: their q, k, v inputs are rounded to bf16
         * like every other GEMM operand (the softmax and the weighted sum stay in f32 here). */
        for (size_t i = 0; i < T * 3 * d; ++i) qkv[i] = bf16_bits_to_f32(f32_to_bf16_bits(qkv[i]));
        /* (B·S, 3·H·D) -> three (B·H·S, D) tensors; column blocks are [Q | K | V], heads are
         * contiguous head_dim-wide slices (vit.rs:151-180). */
        for (size_t b = 0; b < batch; ++b)
            for (size_t hh = 0; hh < heads; ++hh)
                for (size_t s = 0; s < seq; ++s) {
                    const float *src = qkv + (b * seq + s) * 3 * d + hh * hd;
                    const size_t dst = ((b * heads + hh) * seq + s) * hd;
                    memcpy(qh + dst, src, hd * sizeof(float));
                    memcpy(kh + dst, src + d, hd * sizeof(float));
                    memcpy(vh + dst, src + 2 * d, hd * sizeof(float));
                }
        rc = st_oracle_attention_f32(batch * heads, seq, hd, scale, 1, qh, kh, vh, NULL, NULL, ah, threads);
        if (rc) goto done;
        for (size_t b = 0; b < batch; ++b)
            for (size_t hh = 0; hh < heads; ++hh)
                for (size_t s = 0; s < seq; ++s)
                    memcpy(attn + (b * seq + s) * d + hh * hd, ah + ((b * heads + hh) * seq + s) * hd,
                           hd * sizeof(float));
        rc = linear_bf16(T, d, d, attn, w_o, b_o, x, ST_ORACLE_ACT_NONE, x2, threads);
        if (rc) goto done;
        rc = st_oracle_layer_norm_f32(T, d, x2, NULL, ln2_g, ln2_b, cfg->ln_eps, h);
        if (rc) goto done;
        rc = linear_bf16(T, d, ff, h, w_fc1, b_fc1, NULL, ST_ORACLE_ACT_GELU, u, threads);
        if (rc) goto done;
        rc = linear_bf16(T, ff, d, u, w_fc2, b_fc2, x2, ST_ORACLE_ACT_NONE, x, threads);
        if (rc) goto done;
    }
    {
        const float *lnf_g = p; p += d;
        const float *lnf_b = p; p += d;
        const float *w_head = p; p += d * vocab;
        const float *b_head = p; p += vocab;
        rc = st_oracle_layer_norm_f32(T, d, x, NULL, lnf_g, lnf_b, cfg->ln_eps, h);
        if (rc) goto done;
        rc = linear_bf16(T, d, vocab, h, w_head, b_head, NULL, ST_ORACLE_ACT_NONE, logits, threads);
    }
done:
    free(x); free(h); free(qkv); free(qh); free(kh); free(vh); free(ah); free(attn); free(u); free(x2);
    return rc;
}
