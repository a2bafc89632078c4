// Row-wise, HBM-bound helpers of the decoder stack: layer-norm, embedding gather, f32->bf16 rounding
// and the (tokens, heads*dim) <-> (contexts*seq, dim) re-layouts around attention.
#include "device_math.h"
#include "kernels.h"

namespace sthip {

namespace {

// A token id stored as f32 -> a row of the table: rounded to the nearest integer, clamped to [0, vocab - 1], anything
// that is not finite to row 0 (token_to_index, crates/st-nn/src/layers/embedding.rs:325-330).
__device__ __forceinline__ int token_to_index(float value, int vocab)
{
    int index = 0;
    if (isfinite(value)) {
        const float rounded = roundf(value);
        if (rounded > 0.0f) index = rounded >= static_cast<float>(vocab) ? vocab - 1 : static_cast<int>(rounded);
        if (index > vocab - 1) index = vocab - 1;
    }
    return index;
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset);
    return v;
}

// One wavefront per row.  layer_norm_cpu, crates/st-tensor/src/pure.rs:4008-4058:
// mean = Σv/cols; var = max(Σv²/cols − mean², 0); out = ((v − mean)/sqrt(var + eps))·γ + β.
__global__ __launch_bounds__(256) void layer_norm_kernel(int rows, int cols, const float *x, const float *residual,
                                                         const float *gamma, const float *beta, float epsilon,
                                                         float *out_f32, uint16_t *out_bf16)
{
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const size_t offset = static_cast<size_t>(row) * cols;
    float sum = 0.0f, sumsq = 0.0f;
    for (int c = lane; c < cols; c += 64) {
        float v = x[offset + c];
        if (residual) v += residual[offset + c];
        sum += v;
        sumsq += v * v;
    }
    sum = wave_sum(sum);
    sumsq = wave_sum(sumsq);
    const float cols_f = static_cast<float>(cols);
    const float mean = sum / cols_f;
    const float var = layer_norm_variance(sumsq, mean, cols_f);
    const float denom = layer_norm_denominator(var, epsilon);
    for (int c = lane; c < cols; c += 64) {
        float v = x[offset + c];
        if (residual) v += residual[offset + c];
        const float value = layer_norm_scale_shift((v - mean) / denom, gamma[c], beta[c]);
        if (out_f32) out_f32[offset + c] = value;
        if (out_bf16) out_bf16[offset + c] = f32_to_bf16_rne(value);
    }
}

// Same, for rows of at most 2048 values with 16-byte aligned rows: the row is read once, 128 bits per lane, and
// stays in registers between the statistics and the normalisation.
// GATHER: row r of the input is row token_to_index(token_ids[r]) of the table `x` (an embedding lookup,
// crates/st-nn/src/layers/embedding.rs:42-100), which is also written to `gathered` as it passes: the lookup and the
// layer norm that follows it in a pre-norm stack as one launch, the same arithmetic on the same values in the same order.
struct RowGather {
    const float *token_ids;
    float *gathered;
    int vocab;
};

template <int CHUNKS, int ROWS, bool GATHER = false>
__global__ __launch_bounds__(256) void layer_norm_vec_kernel(int rows, int cols, const float *x, const float *residual,
                                                             const float *gamma, const float *beta, float epsilon,
                                                             float *out_f32, uint16_t *out_bf16, RowGather gather)
{
    // A wavefront takes ROWS consecutive rows and has all their loads in flight before the first reduction: with one
    // short row per wavefront the launch is bound by the latency of that one load, not by bandwidth.
    const int lane = threadIdx.x & 63;
    const int row0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * ROWS;
    if (row0 >= rows) return;
    float4 v[ROWS][CHUNKS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const size_t offset = static_cast<size_t>(row0 + r) * cols;
        size_t source = offset;
        if constexpr (GATHER) {
            if (row0 + r < rows) source = static_cast<size_t>(token_to_index(gather.token_ids[row0 + r], gather.vocab)) * cols;
        }
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i) {
            const int c = (lane + 64 * i) * 4;
            v[r][i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (c < cols && row0 + r < rows) {
                v[r][i] = *reinterpret_cast<const float4 *>(x + source + c);
                if constexpr (GATHER) *reinterpret_cast<float4 *>(gather.gathered + offset + c) = v[r][i];
                if (residual) {
                    const float4 q = *reinterpret_cast<const float4 *>(residual + offset + c);
                    v[r][i].x += q.x; v[r][i].y += q.y; v[r][i].z += q.z; v[r][i].w += q.w;
                }
            }
        }
    }
    float4 g[CHUNKS], b[CHUNKS];
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
        const int c = (lane + 64 * i) * 4;
        g[i] = b[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c < cols) {
            g[i] = *reinterpret_cast<const float4 *>(gamma + c);
            b[i] = *reinterpret_cast<const float4 *>(beta + c);
        }
    }
    const float cols_f = static_cast<float>(cols);
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        if (row0 + r >= rows) break;
        const size_t offset = static_cast<size_t>(row0 + r) * cols;
        float sum = 0.0f, sumsq = 0.0f;
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i) {
            sum += sum4(v[r][i]);
            sumsq += sumsq4(v[r][i]);
        }
        sum = wave_sum(sum);
        sumsq = wave_sum(sumsq);
        const float mean = sum / cols_f;
        const float var = layer_norm_variance(sumsq, mean, cols_f);
        const float denom = layer_norm_denominator(var, epsilon);
        // (v - mean) / denom for every element, with one real division per row: the product with the correctly rounded
        // reciprocal, corrected once by its exact remainder (two fused multiply-adds), is the correctly rounded quotient
        // again, i.e. bit for bit what the division gives; only the last bit matters here, because it decides some of
        // the bf16 roundings downstream and the decoder is compared with a CPU stack that divides.
        const float inv = 1.0f / denom;
        auto quotient = [&](float a) {
            const float q = a * inv;
            return fmaf(fmaf(-q, denom, a), inv, q);
        };
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i) {
            const int c = (lane + 64 * i) * 4;
            if (c >= cols) continue;
            float4 o;
            o.x = layer_norm_scale_shift(quotient(v[r][i].x - mean), g[i].x, b[i].x);
            o.y = layer_norm_scale_shift(quotient(v[r][i].y - mean), g[i].y, b[i].y);
            o.z = layer_norm_scale_shift(quotient(v[r][i].z - mean), g[i].z, b[i].z);
            o.w = layer_norm_scale_shift(quotient(v[r][i].w - mean), g[i].w, b[i].w);
            if (out_f32) *reinterpret_cast<float4 *>(out_f32 + offset + c) = o;
            if (out_bf16) {
                uint2 packed;
                packed.x = pack_bf16x2_rne(o.x, o.y);
                packed.y = pack_bf16x2_rne(o.z, o.w);
                *reinterpret_cast<uint2 *>(out_bf16 + offset + c) = packed;
            }
        }
    }
}

// Sum / maximum / minimum over a workgroup of THREADS threads: the butterfly inside each wavefront, then the wavefronts'
// values added (compared) in wavefront order by every thread, so all threads hold the same result and it depends on
// nothing but the shape.  `scratch` holds THREADS/64 values and may be reused after the call returns.
template <int THREADS, class T, class Op>
__device__ __forceinline__ T block_reduce(T v, T *scratch, Op op)
{
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v = op(v, __shfl_xor(v, offset));
    __syncthreads();  // earlier readers of scratch are done
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    T total = scratch[0];
#pragma unroll
    for (int w = 1; w < THREADS / 64; ++w) total = op(total, scratch[w]);
    return total;
}

// Rows of up to 65536 values held in the registers of one 1024-thread workgroup (CH 16-byte pieces per thread, all
// requested before the first reduction): the row is read once and written once, whatever its alignment — a row of
// 50257 values starts at any 4-byte boundary, which global memory takes for 16-byte accesses; the types say so.
typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef unsigned int u32x2_a2 __attribute__((ext_vector_type(2), aligned(2)));

template <int CH>
__global__ __launch_bounds__(1024) void layer_norm_block_kernel(int cols, const float *x, const float *residual,
                                                                const float *gamma, const float *beta, float epsilon,
                                                                float *out_f32, uint16_t *out_bf16)
{
    __shared__ float scratch[16];
    const int tid = threadIdx.x;
    const size_t offset = static_cast<size_t>(blockIdx.x) * cols;
    float v[CH][4];
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int c = (tid + 1024 * i) * 4;
        if (c + 4 <= cols) {
            const f32x4_a4 t = *reinterpret_cast<const f32x4_a4 *>(x + offset + c);
            v[i][0] = t[0]; v[i][1] = t[1]; v[i][2] = t[2]; v[i][3] = t[3];
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[i][e] = c + e < cols ? x[offset + c + e] : 0.0f;
        }
    }
    if (residual) {
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            const int c = (tid + 1024 * i) * 4;
            if (c + 4 <= cols) {
                const f32x4_a4 t = *reinterpret_cast<const f32x4_a4 *>(residual + offset + c);
                v[i][0] += t[0]; v[i][1] += t[1]; v[i][2] += t[2]; v[i][3] += t[3];
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (c + e < cols) v[i][e] += residual[offset + c + e];
            }
        }
    }
    float sum = 0.0f, sumsq = 0.0f;
#pragma unroll
    for (int i = 0; i < CH; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {  // values past the end are zero
            sum += v[i][e];
            sumsq = fmaf(v[i][e], v[i][e], sumsq);
        }
    auto add = [](float a, float b) { return a + b; };
    sum = block_reduce<1024>(sum, scratch, add);
    sumsq = block_reduce<1024>(sumsq, scratch, add);
    const float cols_f = static_cast<float>(cols);
    const float mean = sum / cols_f;
    const float var = layer_norm_variance(sumsq, mean, cols_f);
    const float denom = layer_norm_denominator(var, epsilon);
    const float inv = 1.0f / denom;
    auto quotient = [&](float a) {  // a / denom, correctly rounded (see layer_norm_vec_kernel)
        const float q = a * inv;
        return fmaf(fmaf(-q, denom, a), inv, q);
    };
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int c = (tid + 1024 * i) * 4;
        if (c >= cols) continue;
        float o[4];
        if (c + 4 <= cols) {
            const f32x4_a4 g = *reinterpret_cast<const f32x4_a4 *>(gamma + c), b = *reinterpret_cast<const f32x4_a4 *>(beta + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = layer_norm_scale_shift(quotient(v[i][e] - mean), g[e], b[e]);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = c + e < cols ? layer_norm_scale_shift(quotient(v[i][e] - mean), gamma[c + e], beta[c + e]) : 0.0f;
        }
        if (c + 4 <= cols) {
            if (out_f32) *reinterpret_cast<f32x4_a4 *>(out_f32 + offset + c) = f32x4_a4{o[0], o[1], o[2], o[3]};
            if (out_bf16)
                *reinterpret_cast<u32x2_a2 *>(out_bf16 + offset + c) = u32x2_a2{pack_bf16x2_rne(o[0], o[1]), pack_bf16x2_rne(o[2], o[3])};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (c + e >= cols) continue;
                if (out_f32) out_f32[offset + c + e] = o[e];
                if (out_bf16) out_bf16[offset + c + e] = f32_to_bf16_rne(o[e]);
            }
        }
    }
}

// Long rows (more than 2048 values, or rows that are not 16-byte aligned): one workgroup per row, two sweeps over the
// row (statistics, then the normalisation; the second sweep is served by the caches for rows of up to a few MB).
template <int THREADS, bool VEC>
__global__ __launch_bounds__(THREADS) void layer_norm_long_kernel(int cols, const float *x, const float *residual,
                                                                  const float *gamma, const float *beta, float epsilon,
                                                                  float *out_f32, uint16_t *out_bf16)
{
    __shared__ float scratch[THREADS / 64];
    const int tid = threadIdx.x;
    const size_t offset = static_cast<size_t>(blockIdx.x) * cols;
    constexpr int W = VEC ? 4 : 1;
    auto load = [&](int c, float (&v)[W]) {
        if constexpr (VEC) {
            const float4 t = *reinterpret_cast<const float4 *>(x + offset + c);
            v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
            if (residual) {
                const float4 q = *reinterpret_cast<const float4 *>(residual + offset + c);
                v[0] += q.x; v[1] += q.y; v[2] += q.z; v[3] += q.w;
            }
        } else {
            v[0] = x[offset + c];
            if (residual) v[0] += residual[offset + c];
        }
    };
    float sum = 0.0f, sumsq = 0.0f;
#pragma unroll 4
    for (int c = tid * W; c < cols; c += THREADS * W) {
        float v[W];
        load(c, v);
#pragma unroll
        for (int e = 0; e < W; ++e) {
            sum += v[e];
            sumsq = fmaf(v[e], v[e], sumsq);
        }
    }
    auto add = [](float a, float b) { return a + b; };
    sum = block_reduce<THREADS>(sum, scratch, add);
    sumsq = block_reduce<THREADS>(sumsq, scratch, add);
    const float cols_f = static_cast<float>(cols);
    const float mean = sum / cols_f;
    const float var = layer_norm_variance(sumsq, mean, cols_f);
    const float denom = layer_norm_denominator(var, epsilon);
    const float inv = 1.0f / denom;
    auto quotient = [&](float a) {  // a / denom, correctly rounded (see layer_norm_vec_kernel)
        const float q = a * inv;
        return fmaf(fmaf(-q, denom, a), inv, q);
    };
#pragma unroll 4
    for (int c = tid * W; c < cols; c += THREADS * W) {
        float v[W], o[W];
        load(c, v);
#pragma unroll
        for (int e = 0; e < W; ++e) o[e] = layer_norm_scale_shift(quotient(v[e] - mean), gamma[c + e], beta[c + e]);
        if constexpr (VEC) {
            if (out_f32) *reinterpret_cast<float4 *>(out_f32 + offset + c) = make_float4(o[0], o[1], o[2], o[3]);
            if (out_bf16) {
                uint2 packed;
                packed.x = pack_bf16x2_rne(o[0], o[1]);
                packed.y = pack_bf16x2_rne(o[2], o[3]);
                *reinterpret_cast<uint2 *>(out_bf16 + offset + c) = packed;
            }
        } else {
            if (out_f32) out_f32[offset + c] = o[0];
            if (out_bf16) out_bf16[offset + c] = f32_to_bf16_rne(o[0]);
        }
    }
}


// token_to_index + row gather, crates/st-nn/src/layers/embedding.rs:42-100,325-330.
__global__ __launch_bounds__(256) void embedding_kernel(int tokens, int vocab, int dim, const float *token_ids,
                                                        const float *table, float *out)
{
    const int token = blockIdx.x;
    if (token >= tokens) return;
    const float value = token_ids[token];
    const int index = token_to_index(value, vocab);
    const float *src = table + static_cast<size_t>(index) * dim;
    float *dst = out + static_cast<size_t>(token) * dim;
    for (int c = threadIdx.x; c < dim; c += 256) dst[c] = src[c];
}

// Same gather, 128 bits per thread (dim a multiple of 4, 16-byte aligned table and output): thread i of the launch
// copies chunk i % (dim/4) of token i / (dim/4).
__global__ __launch_bounds__(256) void embedding_vec_kernel(size_t chunks, int vocab, int dim4, const float *token_ids,
                                                            const float4 *table, float4 *out)
{
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= chunks) return;
    const size_t token = i / static_cast<size_t>(dim4);
    const int c = static_cast<int>(i - token * dim4);
    const float value = token_ids[token];
    const int index = token_to_index(value, vocab);
    out[i] = table[static_cast<size_t>(index) * dim4 + c];
}

__global__ __launch_bounds__(256) void f32_to_bf16_kernel(size_t count, const float *in, uint16_t *out)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count; i += stride)
        out[i] = f32_to_bf16_rne(in[i]);
}

// qkv (B·S, 3·H·D) with column blocks [Q | K | V] -> q, k, v each (B·H·S, D).
template <bool ROUND_BF16>
__global__ __launch_bounds__(256) void split_heads_kernel(int batch, int seq, int heads, int dim, const float *qkv,
                                                          float *q, float *k, float *v)
{
    auto keep = [](float x) {
        return ROUND_BF16 ? __uint_as_float(static_cast<uint32_t>(f32_to_bf16_rne(x)) << 16) : x;
    };
    const size_t total = static_cast<size_t>(batch) * seq * heads * dim;
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    const int width = heads * dim;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += stride) {
        const int d = static_cast<int>(i % dim);
        size_t rest = i / dim;
        const int s = static_cast<int>(rest % seq);
        rest /= seq;
        const int h = static_cast<int>(rest % heads);
        const int b = static_cast<int>(rest / heads);
        const size_t src = (static_cast<size_t>(b) * seq + s) * 3 * width + static_cast<size_t>(h) * dim + d;
        q[i] = keep(qkv[src]);
        k[i] = keep(qkv[src + width]);
        v[i] = keep(qkv[src + 2 * width]);
    }
}

// (B·H·S, D) -> (B·S, H·D)
__global__ __launch_bounds__(256) void merge_heads_kernel(int batch, int seq, int heads, int dim, const float *in,
                                                          float *out_f32, uint16_t *out_bf16)
{
    const size_t total = static_cast<size_t>(batch) * seq * heads * dim;
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += stride) {
        // i indexes the OUTPUT (b, s, h, d) so stores are contiguous
        const int d = static_cast<int>(i % dim);
        size_t rest = i / dim;
        const int h = static_cast<int>(rest % heads);
        rest /= heads;
        const int s = static_cast<int>(rest % seq);
        const int b = static_cast<int>(rest / seq);
        const float value = in[((static_cast<size_t>(b) * heads + h) * seq + s) * dim + d];
        if (out_f32) out_f32[i] = value;
        if (out_bf16) out_bf16[i] = f32_to_bf16_rne(value);
    }
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset));
    return v;
}

// One wavefront per row.  cpu_row_softmax_hardmax, crates/st-tensor/src/pure.rs:11930-11980: the maximum is
// taken over the non-NaN entries (first occurrence wins), base = max if finite else 0, weights exp(v - base)
// (0 for NaN), divided by their sum when that is finite and above f32 epsilon; otherwise the row becomes the
// one-hot of the maximum.  A row of only NaNs gives zeros.
__global__ __launch_bounds__(256) void row_softmax_kernel(int rows, int cols, const float *in, float *out)
{
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *x = in + static_cast<size_t>(row) * cols;
    float *y = out + static_cast<size_t>(row) * cols;
    float best = -INFINITY;
    int best_index = 0x7fffffff;
    for (int c = lane; c < cols; c += 64) {
        const float v = x[c];
        if (v != v) continue;
        if (best_index == 0x7fffffff || v > best) {
            best = v;
            best_index = c;
        }
    }
    // first occurrence of the largest value across the wavefront
    const float row_max = wave_max(best_index == 0x7fffffff ? -INFINITY : best);
    int candidate = (best_index != 0x7fffffff && best == row_max) ? best_index : 0x7fffffff;
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) candidate = min(candidate, __shfl_xor(candidate, offset));
    const bool found = candidate != 0x7fffffff;
    const float base = (found && isfinite(row_max)) ? row_max : 0.0f;
    float denom = 0.0f;
    for (int c = lane; c < cols; c += 64) {
        const float v = x[c];
        denom += (!found || v != v) ? 0.0f : expf(v - base);
    }
    denom = wave_sum(denom);
    const bool normal = isfinite(denom) && denom > 1.1920929e-7f;
    const float inv = normal ? 1.0f / denom : 0.0f;
    for (int c = lane; c < cols; c += 64) {
        const float v = x[c];
        const float weight = (!found || v != v) ? 0.0f : expf(v - base);
        float value = weight * inv;
        if (found && !normal) value = c == candidate ? 1.0f : 0.0f;
        y[c] = value;
    }
}

// Same for rows of at most 2048 values with 16-byte aligned rows: one 128-bit read per lane and chunk, the row stays
// in registers for all three phases.
template <int CHUNKS>
__global__ __launch_bounds__(256) void row_softmax_vec_kernel(int rows, int cols, const float *in, float *out)
{
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *x = in + static_cast<size_t>(row) * cols;
    float *y = out + static_cast<size_t>(row) * cols;
    float v[CHUNKS][4];
    float best = -INFINITY;
    int best_index = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
        const int c = (lane + 64 * i) * 4;
        if (c < cols) {
            const float4 t = *reinterpret_cast<const float4 *>(x + c);
            v[i][0] = t.x; v[i][1] = t.y; v[i][2] = t.z; v[i][3] = t.w;
        } else {
            v[i][0] = v[i][1] = v[i][2] = v[i][3] = __builtin_nanf("");  // skipped like NaN entries, never stored
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float value = v[i][e];
            if (value != value) continue;
            if (best_index == 0x7fffffff || value > best) {  // columns visited in ascending order per lane
                best = value;
                best_index = c + e;
            }
        }
    }
    const float row_max = wave_max(best_index == 0x7fffffff ? -INFINITY : best);
    int candidate = (best_index != 0x7fffffff && best == row_max) ? best_index : 0x7fffffff;
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) candidate = min(candidate, __shfl_xor(candidate, offset));
    const bool found = candidate != 0x7fffffff;
    const float base = (found && isfinite(row_max)) ? row_max : 0.0f;
    float denom = 0.0f;
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float value = v[i][e];
            const float weight = (!found || value != value) ? 0.0f : __expf(value - base);  // exp2 of a scaled argument
            v[i][e] = weight;
            denom += weight;
        }
    denom = wave_sum(denom);
    const bool normal = isfinite(denom) && denom > 1.1920929e-7f;
    const float inv = normal ? 1.0f / denom : 0.0f;
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
        const int c = (lane + 64 * i) * 4;
        if (c >= cols) continue;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            o[e] = v[i][e] * inv;
            if (found && !normal) o[e] = (c + e == candidate) ? 1.0f : 0.0f;
        }
        *reinterpret_cast<float4 *>(y + c) = make_float4(o[0], o[1], o[2], o[3]);
    }
}

// Long rows: one workgroup per row, three sweeps (maximum and its first position; the sum of the weights; the output).
template <int THREADS, bool VEC>
__global__ __launch_bounds__(THREADS) void row_softmax_long_kernel(int cols, const float *in, float *out)
{
    __shared__ float scratch_f[THREADS / 64];
    __shared__ int scratch_i[THREADS / 64];
    const int tid = threadIdx.x;
    const float *x = in + static_cast<size_t>(blockIdx.x) * cols;
    float *y = out + static_cast<size_t>(blockIdx.x) * cols;
    constexpr int W = VEC ? 4 : 1;
    auto load = [&](int c, float (&v)[W]) {
        if constexpr (VEC) {
            const float4 t = *reinterpret_cast<const float4 *>(x + c);
            v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
        } else {
            v[0] = x[c];
        }
    };
    float best = -INFINITY;
    int best_index = 0x7fffffff;
#pragma unroll 4
    for (int c = tid * W; c < cols; c += THREADS * W) {  // ascending columns per thread: the first occurrence wins
        float v[W];
        load(c, v);
#pragma unroll
        for (int e = 0; e < W; ++e) {
            if (v[e] != v[e]) continue;
            if (best_index == 0x7fffffff || v[e] > best) {
                best = v[e];
                best_index = c + e;
            }
        }
    }
    const float row_max = block_reduce<THREADS>(best_index == 0x7fffffff ? -INFINITY : best, scratch_f,
                                                [](float a, float b) { return fmaxf(a, b); });
    const int candidate = block_reduce<THREADS>((best_index != 0x7fffffff && best == row_max) ? best_index : 0x7fffffff,
                                                scratch_i, [](int a, int b) { return min(a, b); });
    const bool found = candidate != 0x7fffffff;
    const float base = (found && isfinite(row_max)) ? row_max : 0.0f;
    float denom = 0.0f;
#pragma unroll 4
    for (int c = tid * W; c < cols; c += THREADS * W) {
        float v[W];
        load(c, v);
#pragma unroll
        for (int e = 0; e < W; ++e) denom += (!found || v[e] != v[e]) ? 0.0f : __expf(v[e] - base);
    }
    denom = block_reduce<THREADS>(denom, scratch_f, [](float a, float b) { return a + b; });
    const bool normal = isfinite(denom) && denom > 1.1920929e-7f;
    const float inv = normal ? 1.0f / denom : 0.0f;
#pragma unroll 4
    for (int c = tid * W; c < cols; c += THREADS * W) {
        float v[W], o[W];
        load(c, v);
#pragma unroll
        for (int e = 0; e < W; ++e) {
            const float weight = (!found || v[e] != v[e]) ? 0.0f : __expf(v[e] - base);
            o[e] = weight * inv;
            if (found && !normal) o[e] = (c + e == candidate) ? 1.0f : 0.0f;
        }
        if constexpr (VEC) *reinterpret_cast<float4 *>(y + c) = make_float4(o[0], o[1], o[2], o[3]);
        else y[c] = o[0];
    }
}

// A few very long rows (a handful of sequences over a vocabulary): a workgroup per row would leave most of the chip
// idle, so the grid's x cuts every row into segments.  First launch: each segment's maximum (first position, NaN
// skipped) and the sum of its weights relative to that maximum; second launch: every workgroup combines its row's
// segment results — in segment order, so the same bits every time — and writes its own segment.  Same edge rules
// as the single-workgroup kernels (the base is the maximum when that is finite, else 0; a row whose sum is not a
// normal number becomes one-hot at the first maximum).
struct SoftmaxSegment {
    float best;   // maximum of the segment's non-NaN values
    int index;    // its first column, 0x7fffffff when the segment has none
    float sum;    // sum of exp(v - base), base = best if finite else 0
};

// Four adjacent values of a row at any 4-byte alignment; past `end` they read as NaN, which every phase skips.
__device__ __forceinline__ void load_quad_or_nan(const float *x, int c, int end, float (&v)[4])
{
    if (c + 4 <= end) {
        const f32x4_a4 t = *reinterpret_cast<const f32x4_a4 *>(x + c);
        v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3];
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (c + e < end) ? x[c + e] : __builtin_nanf("");
    }
}

__global__ __launch_bounds__(256) void row_softmax_split_partial_kernel(int cols, int segment, const float *in, SoftmaxSegment *parts)
{
    __shared__ float scratch_f[4];
    __shared__ int scratch_i[4];
    const int tid = threadIdx.x;
    const float *x = in + static_cast<size_t>(blockIdx.y) * cols;
    const int c_begin = static_cast<int>(blockIdx.x) * segment, c_end = min(cols, c_begin + segment);
    float best = -INFINITY;
    int best_index = 0x7fffffff;
#pragma unroll 4
    for (int c = c_begin + tid * 4; c < c_end; c += 1024) {
        float v[4];
        load_quad_or_nan(x, c, c_end, v);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (v[e] != v[e]) continue;
            if (best_index == 0x7fffffff || v[e] > best) {
                best = v[e];
                best_index = c + e;
            }
        }
    }
    const float seg_max = block_reduce<256>(best_index == 0x7fffffff ? -INFINITY : best, scratch_f,
                                            [](float a, float b) { return fmaxf(a, b); });
    const int candidate = block_reduce<256>((best_index != 0x7fffffff && best == seg_max) ? best_index : 0x7fffffff, scratch_i,
                                            [](int a, int b) { return min(a, b); });
    const bool found = candidate != 0x7fffffff;
    const float base = (found && isfinite(seg_max)) ? seg_max : 0.0f;
    float sum = 0.0f;
#pragma unroll 4
    for (int c = c_begin + tid * 4; c < c_end; c += 1024) {
        float v[4];
        load_quad_or_nan(x, c, c_end, v);
#pragma unroll
        for (int e = 0; e < 4; ++e) sum += (!found || v[e] != v[e]) ? 0.0f : __expf(v[e] - base);
    }
    sum = block_reduce<256>(sum, scratch_f, [](float a, float b) { return a + b; });
    if (tid == 0) parts[static_cast<size_t>(blockIdx.y) * gridDim.x + blockIdx.x] = SoftmaxSegment{seg_max, candidate, sum};
}

__global__ __launch_bounds__(256) void row_softmax_split_write_kernel(int cols, int segment, const float *in,
                                                                      const SoftmaxSegment *parts, float *out)
{
    const int tid = threadIdx.x;
    const float *x = in + static_cast<size_t>(blockIdx.y) * cols;
    float *y = out + static_cast<size_t>(blockIdx.y) * cols;
    const int c_begin = static_cast<int>(blockIdx.x) * segment, c_end = min(cols, c_begin + segment);
    const SoftmaxSegment *row_parts = parts + static_cast<size_t>(blockIdx.y) * gridDim.x;
    // The (at most 64) segment results go through LDS, one load each; every thread then combines them itself, in order.
    __shared__ SoftmaxSegment staged[64];
    if (tid < static_cast<int>(gridDim.x)) staged[tid] = row_parts[tid];
    __syncthreads();
    float row_max = -INFINITY;
    int candidate = 0x7fffffff;
    for (unsigned s = 0; s < gridDim.x; ++s) {
        const SoftmaxSegment part = staged[s];
        if (part.index == 0x7fffffff) continue;
        if (candidate == 0x7fffffff || part.best > row_max) {  // segments ascend: the first occurrence wins
            row_max = part.best;
            candidate = part.index;
        }
    }
    const bool found = candidate != 0x7fffffff;
    const float base = (found && isfinite(row_max)) ? row_max : 0.0f;
    float denom = 0.0f;
    for (unsigned s = 0; s < gridDim.x; ++s) {
        const SoftmaxSegment part = staged[s];
        if (part.index == 0x7fffffff || part.sum == 0.0f) continue;
        const float part_base = isfinite(part.best) ? part.best : 0.0f;
        denom += part.sum * __expf(part_base - base);
    }
    const bool normal = isfinite(denom) && denom > 1.1920929e-7f;
    const float inv = normal ? 1.0f / denom : 0.0f;
#pragma unroll 4
    for (int c = c_begin + tid * 4; c < c_end; c += 1024) {
        float v[4], o[4];
        load_quad_or_nan(x, c, c_end, v);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float weight = (!found || v[e] != v[e]) ? 0.0f : __expf(v[e] - base);
            o[e] = weight * inv;
            if (found && !normal) o[e] = (c + e == candidate) ? 1.0f : 0.0f;
        }
        if (c + 4 <= c_end) {
            *reinterpret_cast<f32x4_a4 *>(y + c) = f32x4_a4{o[0], o[1], o[2], o[3]};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (c + e < c_end) y[c + e] = o[e];
        }
    }
}

// The same for softmax: the row stays in the registers of a 1024-thread workgroup through all three phases.
template <int CH>
__global__ __launch_bounds__(1024) void row_softmax_block_kernel(int cols, const float *in, float *out)
{
    __shared__ float scratch_f[16];
    __shared__ int scratch_i[16];
    const int tid = threadIdx.x;
    const float *x = in + static_cast<size_t>(blockIdx.x) * cols;
    float *y = out + static_cast<size_t>(blockIdx.x) * cols;
    float v[CH][4];
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int c = (tid + 1024 * i) * 4;
        if (c + 4 <= cols) {
            const f32x4_a4 t = *reinterpret_cast<const f32x4_a4 *>(x + c);
            v[i][0] = t[0]; v[i][1] = t[1]; v[i][2] = t[2]; v[i][3] = t[3];
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[i][e] = c + e < cols ? x[c + e] : __builtin_nanf("");  // skipped like NaN entries
        }
    }
    float best = -INFINITY;
    int best_index = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < CH; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {  // ascending columns per thread: the first occurrence wins
            const float value = v[i][e];
            if (value != value) continue;
            if (best_index == 0x7fffffff || value > best) {
                best = value;
                best_index = (tid + 1024 * i) * 4 + e;
            }
        }
    const float row_max = block_reduce<1024>(best_index == 0x7fffffff ? -INFINITY : best, scratch_f,
                                             [](float a, float b) { return fmaxf(a, b); });
    const int candidate = block_reduce<1024>((best_index != 0x7fffffff && best == row_max) ? best_index : 0x7fffffff, scratch_i,
                                             [](int a, int b) { return min(a, b); });
    const bool found = candidate != 0x7fffffff;
    const float base = (found && isfinite(row_max)) ? row_max : 0.0f;
    float denom = 0.0f;
#pragma unroll
    for (int i = 0; i < CH; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float value = v[i][e];
            const float weight = (!found || value != value) ? 0.0f : __expf(value - base);
            v[i][e] = weight;
            denom += weight;
        }
    denom = block_reduce<1024>(denom, scratch_f, [](float a, float b) { return a + b; });
    const bool normal = isfinite(denom) && denom > 1.1920929e-7f;
    const float inv = normal ? 1.0f / denom : 0.0f;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int c = (tid + 1024 * i) * 4;
        if (c >= cols) continue;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            o[e] = v[i][e] * inv;
            if (found && !normal) o[e] = (c + e == candidate) ? 1.0f : 0.0f;
        }
        if (c + 4 <= cols) {
            *reinterpret_cast<f32x4_a4 *>(y + c) = f32x4_a4{o[0], o[1], o[2], o[3]};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (c + e < cols) y[c + e] = o[e];
        }
    }
}

// Gelu::forward, crates/st-nn/src/layers/gelu.rs:78-94 (the tanh form of crates/st-tensor/src/pure.rs:12026-12031).
__global__ __launch_bounds__(256) void gelu_forward_kernel(size_t count, const float *in, float *out)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count; i += stride) out[i] = gelu_tanh(in[i]);
}

// Four values per thread and access when the buffers are 16-byte aligned.
__global__ __launch_bounds__(256) void gelu_forward_vec_kernel(size_t count4, const float4 *in, float4 *out)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count4; i += stride) {
        const float4 v = in[i];
        out[i] = make_float4(gelu_tanh(v.x), gelu_tanh(v.y), gelu_tanh(v.z), gelu_tanh(v.w));
    }
}

// status[0] = number of non-finite values, status[1] = smallest index of one (status[1] must start at ~0).
// The first workgroup resets nothing: the caller clears the two words before the launch.
__global__ __launch_bounds__(256) void nonfinite_probe_kernel(size_t count, const float *data, unsigned long long *status)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    unsigned long long found = 0, first = ~0ull;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count; i += stride) {
        if (!isfinite(data[i])) {
            ++found;
            if (i < first) first = i;
        }
    }
    if (found) {
        atomicAdd(&status[0], found);
        atomicMin(&status[1], first);
    }
}

// gelu_prime(z)·g, crates/st-tensor/src/pure.rs:12033-12040 and :6549-6552.
__global__ __launch_bounds__(256) void gelu_backward_kernel(size_t count, const float *z, const float *grad, float *out)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count; i += stride) {
        const float x = z[i];
        const float x2 = x * x;
        const float inner = 0.7978846f * (x + (0.044715f * x) * x2);
        const float t = tanhf(inner);
        const float prime = 0.5f * (1.0f + t) + (((0.5f * x) * (1.0f - t * t)) * 0.7978846f) * (1.0f + (3.0f * 0.044715f) * x2);
        out[i] = prime * grad[i];
    }
}

// 128-bit forms of the element-wise kernels (count a multiple of 4, 16-byte aligned pointers): one float4 per
// thread and as many workgroups as that takes, which is the access pattern that streams fastest on this chip.
__global__ __launch_bounds__(256) void gelu_backward_vec_kernel(size_t count4, const float4 *z, const float4 *grad, float4 *out)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count4; i += stride) {
        const float4 x4 = z[i], g4 = grad[i];
        const float xs[4] = {x4.x, x4.y, x4.z, x4.w}, gs[4] = {g4.x, g4.y, g4.z, g4.w};
        float r[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float x = xs[e];
            const float x2 = x * x;
            const float inner = 0.7978846f * (x + (0.044715f * x) * x2);
            const float t = tanhf(inner);
            const float prime = 0.5f * (1.0f + t) + (((0.5f * x) * (1.0f - t * t)) * 0.7978846f) * (1.0f + (3.0f * 0.044715f) * x2);
            r[e] = prime * gs[e];
        }
        out[i] = make_float4(r[0], r[1], r[2], r[3]);
    }
}

__global__ __launch_bounds__(256) void scale_vec_kernel(size_t count4, const float4 *in, float scale, float4 *out)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count4; i += stride) {
        const float4 v = in[i];
        out[i] = make_float4(v.x * scale, v.y * scale, v.z * scale, v.w * scale);
    }
}

// cols a multiple of 4: a float4 never straddles a row
__global__ __launch_bounds__(256) void add_row_vec_kernel(size_t count4, int cols4, float4 *data, const float4 *bias)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count4; i += stride) {
        float4 v = data[i];
        const float4 b = bias[i % static_cast<size_t>(cols4)];
        v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w;
        data[i] = v;
    }
}

__global__ __launch_bounds__(256) void f32_to_bf16_vec_kernel(size_t count4, const float4 *in, uint2 *out)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count4; i += stride) {
        const float4 v = in[i];
        out[i] = make_uint2(pack_bf16x2_rne(v.x, v.y), pack_bf16x2_rne(v.z, v.w));
    }
}

// scale_inplace, crates/st-tensor/src/pure.rs:11993-11997 (out may alias in).
__global__ __launch_bounds__(256) void scale_kernel(size_t count, const float *in, float scale, float *out)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count; i += stride) out[i] = in[i] * scale;
}

// add_row_inplace, crates/st-tensor/src/pure.rs:6196-6290: data[r][c] += bias[c].
__global__ __launch_bounds__(256) void add_row_kernel(size_t count, int cols, float *data, const float *bias)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count; i += stride)
        data[i] += bias[i % static_cast<size_t>(cols)];
}

// Column sums, crates/st-tensor/src/pure.rs:7201-7210: stage one adds the rows of one chunk per workgroup row
// (threads along columns, so loads are coalesced); stage two adds the chunks in order and applies the scale.
__global__ __launch_bounds__(256) void sum_axis0_partial_kernel(int rows, int cols, int rows_per_chunk, const float *in,
                                                                float *partial)
{
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= cols) return;
    const int r0 = blockIdx.y * rows_per_chunk;
    const int r1 = min(rows, r0 + rows_per_chunk);
    float sum = 0.0f;
    for (int r = r0; r < r1; ++r) sum += in[static_cast<size_t>(r) * cols + c];
    partial[static_cast<size_t>(blockIdx.y) * cols + c] = sum;
}

// 16-byte aligned rows: a workgroup covers 256 columns (64 lanes × 4) and its four wavefronts take every fourth
// row of the chunk, eight independent loads in flight each; the four partial rows are added through LDS.
// ALIGNED: every row starts on a 16-byte boundary (cols a multiple of 4, aligned base).  Otherwise the 16-byte accesses
// go through a vector type that says 4-byte alignment (global memory takes them), and the last group of a row, which
// may hang over its end, is read value by value.
template <bool ALIGNED>
__global__ __launch_bounds__(256) void sum_axis0_partial_vec_kernel(int rows, int cols, int rows_per_chunk, const float *in,
                                                                    float *partial)
{
    __shared__ float4 stage[4][64];
    const int lane = threadIdx.x & 63, sub = threadIdx.x >> 6;
    const int c = (blockIdx.x * 64 + lane) * 4;
    const int r0 = blockIdx.y * rows_per_chunk;
    const int r1 = min(rows, r0 + rows_per_chunk);
    const bool whole = c + 4 <= cols;  // all four columns exist
    auto load = [&](const float *p) {
        if constexpr (ALIGNED) {
            return *reinterpret_cast<const float4 *>(p);
        } else {
            if (whole) {
                const f32x4_a4 t = *reinterpret_cast<const f32x4_a4 *>(p);
                return make_float4(t[0], t[1], t[2], t[3]);
            }
            return make_float4(p[0], c + 1 < cols ? p[1] : 0.0f, c + 2 < cols ? p[2] : 0.0f, 0.0f);
        }
    };
    float4 acc[2] = {make_float4(0.f, 0.f, 0.f, 0.f), make_float4(0.f, 0.f, 0.f, 0.f)};
    if (c < cols) {
        const float *src = in + c;
        int r = r0 + sub;
        for (; r + 28 < r1; r += 32) {
            float4 t[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) t[u] = load(src + static_cast<size_t>(r + 4 * u) * cols);
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                acc[u & 1].x += t[u].x; acc[u & 1].y += t[u].y; acc[u & 1].z += t[u].z; acc[u & 1].w += t[u].w;
            }
        }
        for (; r < r1; r += 4) {
            const float4 t = load(src + static_cast<size_t>(r) * cols);
            acc[0].x += t.x; acc[0].y += t.y; acc[0].z += t.z; acc[0].w += t.w;
        }
    }
    stage[sub][lane] = make_float4(acc[0].x + acc[1].x, acc[0].y + acc[1].y, acc[0].z + acc[1].z, acc[0].w + acc[1].w);
    __syncthreads();
    if (sub == 0 && c < cols) {
        float4 total = stage[0][lane];
#pragma unroll
        for (int k = 1; k < 4; ++k) {
            total.x += stage[k][lane].x; total.y += stage[k][lane].y; total.z += stage[k][lane].z; total.w += stage[k][lane].w;
        }
        float *dst = partial + static_cast<size_t>(blockIdx.y) * cols + c;
        if constexpr (ALIGNED) {
            *reinterpret_cast<float4 *>(dst) = total;
        } else {
            dst[0] = total.x;
            if (c + 1 < cols) dst[1] = total.y;
            if (c + 2 < cols) dst[2] = total.z;
            if (c + 3 < cols) dst[3] = total.w;
        }
    }
}

// out[c] = scale · Σ_k partial[k][c]: 16 columns per workgroup, sixteen groups of lanes take every sixteenth chunk
// with four loads in flight each; the sixteen partial sums are added in a fixed order through LDS.
__global__ __launch_bounds__(256) void sum_axis0_final_wide_kernel(int chunks, int cols, const float *partial, float scale,
                                                                   float *out)
{
    __shared__ float stage[16][17];
    const int col = threadIdx.x & 15, sub = threadIdx.x >> 4;
    const int c = blockIdx.x * 16 + col;
    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (c < cols) {
        int k = sub;
        for (; k + 48 < chunks; k += 64) {
            float t[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) t[u] = partial[static_cast<size_t>(k + 16 * u) * cols + c];
#pragma unroll
            for (int u = 0; u < 4; ++u) sum[u] += t[u];
        }
        for (; k < chunks; k += 16) sum[0] += partial[static_cast<size_t>(k) * cols + c];
    }
    stage[sub][col] = (sum[0] + sum[1]) + (sum[2] + sum[3]);
    __syncthreads();
    if (sub == 0 && c < cols) {
        float total = stage[0][col];
#pragma unroll
        for (int k = 1; k < 16; ++k) total += stage[k][col];
        out[c] = total * scale;
    }
}

unsigned grid_vec_for(size_t count4)
{
    const size_t blocks = (count4 + 255) / 256;
    return static_cast<unsigned>(blocks < 0x7fffffffull ? (blocks ? blocks : 1) : 0x7fffffffull);
}

bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

unsigned grid_for(size_t count)
{
    const size_t blocks = (count + 255) / 256;
    return static_cast<unsigned>(blocks < 65536 ? (blocks ? blocks : 1) : 65536);
}

}  // namespace

// A count that is a multiple of four takes the 128-bit kernels as a whole; a large one that is not takes them for all
// but its last one to three values, which a second, one-workgroup launch of the scalar kernel finishes (the two
// kernels compute the same bits).
bool vec_with_tail(size_t count) { return count % 4 == 0 || count >= (1u << 20); }

hipError_t launch_layer_norm_f32(size_t rows, size_t cols, const float *x, const float *residual, const float *gamma,
                                 const float *beta, float epsilon, float *out_f32, uint16_t *out_bf16,
                                 hipStream_t stream)
{
    if (rows == 0 || cols == 0) return hipSuccess;
    const dim3 grid(static_cast<unsigned>((rows + 3) / 4)), block(256);
    auto aligned = [](const void *ptr, uintptr_t a) { return (reinterpret_cast<uintptr_t>(ptr) & (a - 1)) == 0; };
    const bool vec = cols % 4 == 0 && cols <= 2048 && aligned(x, 16) && aligned(residual, 16) && aligned(gamma, 16) &&
                     aligned(beta, 16) && aligned(out_f32, 16) && aligned(out_bf16, 8);
    const int r = static_cast<int>(rows), c = static_cast<int>(cols);
    // Two rows per wavefront once there are enough rows to fill the chip that way.
    const bool two_rows = rows >= 8192;
    const dim3 grid2(static_cast<unsigned>((rows + 7) / 8));
    if (vec && cols <= 512 && two_rows)
        hipLaunchKernelGGL((layer_norm_vec_kernel<2, 2>), grid2, block, 0, stream, r, c, x, residual, gamma, beta, epsilon,
                           out_f32, out_bf16, RowGather{});
    else if (vec && cols <= 512)
        hipLaunchKernelGGL((layer_norm_vec_kernel<2, 1>), grid, block, 0, stream, r, c, x, residual, gamma, beta, epsilon,
                           out_f32, out_bf16, RowGather{});
    else if (vec && cols <= 1024 && two_rows)
        hipLaunchKernelGGL((layer_norm_vec_kernel<4, 2>), grid2, block, 0, stream, r, c, x, residual, gamma, beta, epsilon,
                           out_f32, out_bf16, RowGather{});
    else if (vec && cols <= 1024)
        hipLaunchKernelGGL((layer_norm_vec_kernel<4, 1>), grid, block, 0, stream, r, c, x, residual, gamma, beta, epsilon,
                           out_f32, out_bf16, RowGather{});
    else if (vec)
        hipLaunchKernelGGL((layer_norm_vec_kernel<8, 1>), grid, block, 0, stream, r, c, x, residual, gamma, beta, epsilon,
                           out_f32, out_bf16, RowGather{});
    else if (cols > 4096 && cols <= 65536) {
        // The row in the registers of a 1024-thread workgroup: 2 to 16 pieces of 16 bytes per thread.
        const dim3 rows_grid(static_cast<unsigned>(rows));
        const size_t pieces = (cols + 4095) / 4096;
#define ST_LN_BLOCK(CH)                                                                                                     \
    hipLaunchKernelGGL((layer_norm_block_kernel<CH>), rows_grid, dim3(1024), 0, stream, c, x, residual, gamma, beta, epsilon, \
                       out_f32, out_bf16)
        if (pieces <= 2) ST_LN_BLOCK(2);
        else if (pieces <= 4) ST_LN_BLOCK(4);
        else if (pieces <= 8) ST_LN_BLOCK(8);
        else if (pieces <= 12) ST_LN_BLOCK(12);
        else ST_LN_BLOCK(16);
#undef ST_LN_BLOCK
    } else if (cols > 2048) {
        // A workgroup per row: 1024 threads while the rows are few, 256 once the rows alone fill the chip.
        const bool vec_long = cols % 4 == 0 && aligned(x, 16) && aligned(residual, 16) && aligned(out_f32, 16) && aligned(out_bf16, 8);
        const dim3 rows_grid(static_cast<unsigned>(rows));
        if (rows < 2048) {
            if (vec_long) hipLaunchKernelGGL((layer_norm_long_kernel<1024, true>), rows_grid, dim3(1024), 0, stream, c, x, residual, gamma, beta, epsilon, out_f32, out_bf16);
            else hipLaunchKernelGGL((layer_norm_long_kernel<1024, false>), rows_grid, dim3(1024), 0, stream, c, x, residual, gamma, beta, epsilon, out_f32, out_bf16);
        } else {
            if (vec_long) hipLaunchKernelGGL((layer_norm_long_kernel<256, true>), rows_grid, dim3(256), 0, stream, c, x, residual, gamma, beta, epsilon, out_f32, out_bf16);
            else hipLaunchKernelGGL((layer_norm_long_kernel<256, false>), rows_grid, dim3(256), 0, stream, c, x, residual, gamma, beta, epsilon, out_f32, out_bf16);
        }
    } else
        hipLaunchKernelGGL(layer_norm_kernel, grid, block, 0, stream, r, c, x, residual, gamma, beta, epsilon, out_f32,
                           out_bf16);
    return hipGetLastError();
}

// Embedding lookup followed by the layer norm of the looked-up rows: `embedded` receives the rows (the residual stream
// of a pre-norm stack), `out_bf16` their layer norm.  One launch where the 128-bit row kernel applies, two otherwise;
// same values either way.
hipError_t launch_embedding_layer_norm_f32(size_t tokens, size_t vocab, size_t dim, const float *token_ids, const float *table,
                                           float *embedded, const float *gamma, const float *beta, float epsilon,
                                           uint16_t *out_bf16, hipStream_t stream)
{
    if (tokens == 0 || dim == 0) return hipSuccess;
    const bool vec = dim % 4 == 0 && dim <= 2048 && aligned16(table) && aligned16(embedded) && aligned16(gamma) && aligned16(beta) &&
                     (reinterpret_cast<uintptr_t>(out_bf16) & 7u) == 0 && tokens < 0x7fffffffull && vocab < 0x7fffffffull;
    if (!vec) {
        const hipError_t rc = launch_embedding_f32(tokens, vocab, dim, token_ids, table, embedded, stream);
        if (rc != hipSuccess) return rc;
        return launch_layer_norm_f32(tokens, dim, embedded, nullptr, gamma, beta, epsilon, nullptr, out_bf16, stream);
    }
    const RowGather gather{token_ids, embedded, static_cast<int>(vocab)};
    const int r = static_cast<int>(tokens), c = static_cast<int>(dim);
    const dim3 grid(static_cast<unsigned>((tokens + 3) / 4)), grid2(static_cast<unsigned>((tokens + 7) / 8)), block(256);
    const bool two_rows = tokens >= 8192;  // the same choice of kernel as launch_layer_norm_f32: the same sums in the same order
#define ST_LN_GATHER(CHUNKS, ROWS, GRID)                                                                                  \
    hipLaunchKernelGGL((layer_norm_vec_kernel<CHUNKS, ROWS, true>), GRID, block, 0, stream, r, c, table, nullptr, gamma, beta, \
                       epsilon, nullptr, out_bf16, gather)
    if (dim <= 512 && two_rows) ST_LN_GATHER(2, 2, grid2);
    else if (dim <= 512) ST_LN_GATHER(2, 1, grid);
    else if (dim <= 1024 && two_rows) ST_LN_GATHER(4, 2, grid2);
    else if (dim <= 1024) ST_LN_GATHER(4, 1, grid);
    else ST_LN_GATHER(8, 1, grid);
#undef ST_LN_GATHER
    return hipGetLastError();
}

hipError_t launch_embedding_f32(size_t tokens, size_t vocab, size_t dim, const float *token_ids, const float *table,
                                float *out, hipStream_t stream)
{
    if (tokens == 0 || dim == 0) return hipSuccess;
    const size_t chunks = tokens * (dim / 4);
    if (dim % 4 == 0 && aligned16(table) && aligned16(out) && (chunks + 255) / 256 < 0x7fffffffull) {
        hipLaunchKernelGGL(embedding_vec_kernel, dim3(static_cast<unsigned>((chunks + 255) / 256)), dim3(256), 0, stream, chunks,
                           static_cast<int>(vocab), static_cast<int>(dim / 4), token_ids,
                           reinterpret_cast<const float4 *>(table), reinterpret_cast<float4 *>(out));
        return hipGetLastError();
    }
    hipLaunchKernelGGL(embedding_kernel, dim3(static_cast<unsigned>(tokens)), dim3(256), 0, stream,
                       static_cast<int>(tokens), static_cast<int>(vocab), static_cast<int>(dim), token_ids, table, out);
    return hipGetLastError();
}

hipError_t launch_f32_to_bf16(size_t count, const float *in, uint16_t *out, hipStream_t stream)
{
    if (count == 0) return hipSuccess;
    if (vec_with_tail(count) && aligned16(in) && (reinterpret_cast<uintptr_t>(out) & 7u) == 0) {
        const size_t body = count / 4 * 4;
        hipLaunchKernelGGL(f32_to_bf16_vec_kernel, dim3(grid_vec_for(count / 4)), dim3(256), 0, stream, count / 4,
                           reinterpret_cast<const float4 *>(in), reinterpret_cast<uint2 *>(out));
        if (body < count) hipLaunchKernelGGL(f32_to_bf16_kernel, dim3(1), dim3(256), 0, stream, count - body, in + body, out + body);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(f32_to_bf16_kernel, dim3(grid_for(count)), dim3(256), 0, stream, count, in, out);
    return hipGetLastError();
}

hipError_t launch_split_heads_f32(size_t batch, size_t seq, size_t heads, size_t head_dim, const float *qkv, float *q,
                                  float *k, float *v, bool round_to_bf16, hipStream_t stream)
{
    const size_t total = batch * seq * heads * head_dim;
    if (total == 0) return hipSuccess;
    if (round_to_bf16)
        hipLaunchKernelGGL(split_heads_kernel<true>, dim3(grid_for(total)), dim3(256), 0, stream, static_cast<int>(batch),
                           static_cast<int>(seq), static_cast<int>(heads), static_cast<int>(head_dim), qkv, q, k, v);
    else
        hipLaunchKernelGGL(split_heads_kernel<false>, dim3(grid_for(total)), dim3(256), 0, stream, static_cast<int>(batch),
                           static_cast<int>(seq), static_cast<int>(heads), static_cast<int>(head_dim), qkv, q, k, v);
    return hipGetLastError();
}

hipError_t launch_merge_heads_f32(size_t batch, size_t seq, size_t heads, size_t head_dim, const float *contexts_in,
                                  float *out_f32, uint16_t *out_bf16, hipStream_t stream)
{
    const size_t total = batch * seq * heads * head_dim;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(merge_heads_kernel, dim3(grid_for(total)), dim3(256), 0, stream, static_cast<int>(batch),
                       static_cast<int>(seq), static_cast<int>(heads), static_cast<int>(head_dim), contexts_in, out_f32,
                       out_bf16);
    return hipGetLastError();
}

hipError_t launch_row_softmax_f32(size_t rows, size_t cols, const float *in, float *out, hipStream_t stream)
{
    if (rows == 0 || cols == 0) return hipSuccess;
    const dim3 grid(static_cast<unsigned>((rows + 3) / 4)), block(256);
    const int r = static_cast<int>(rows), c = static_cast<int>(cols);
    const bool vec = cols % 4 == 0 && cols <= 2048 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    if (vec && cols <= 512)
        hipLaunchKernelGGL(row_softmax_vec_kernel<2>, grid, block, 0, stream, r, c, in, out);
    else if (vec && cols <= 1024)
        hipLaunchKernelGGL(row_softmax_vec_kernel<4>, grid, block, 0, stream, r, c, in, out);
    else if (vec)
        hipLaunchKernelGGL(row_softmax_vec_kernel<8>, grid, block, 0, stream, r, c, in, out);
    else if (cols > 65536 && rows <= 128) {
        // Few rows too long for a workgroup's registers: segments of at least 8192 values, up to about 1024 workgroups,
        // at most 64 segments a row (4 × 1000000: 34 µs; 16 × 128256: 20 µs; 100 × 100000: 35 → 30 µs.  Up to 65536
        // values the register kernel below is as fast or faster from a handful of rows on: 128 × 50257 19 against 23 µs).
        size_t segments = std::min<size_t>(std::min<size_t>(64, cols / 8192), std::max<size_t>(2, 1024 / rows));
        const size_t segment = ((cols + segments - 1) / segments + 3) / 4 * 4;
        segments = (cols + segment - 1) / segment;
        void *workspace = nullptr;
        const hipError_t rc = stream_workspace(stream, rows * segments * sizeof(SoftmaxSegment), &workspace);
        if (rc != hipSuccess) return rc;
        SoftmaxSegment *parts = static_cast<SoftmaxSegment *>(workspace);
        const dim3 split_grid(static_cast<unsigned>(segments), static_cast<unsigned>(rows));
        const int seg = static_cast<int>(segment);
        hipLaunchKernelGGL(row_softmax_split_partial_kernel, split_grid, dim3(256), 0, stream, c, seg, in, parts);
        hipLaunchKernelGGL(row_softmax_split_write_kernel, split_grid, dim3(256), 0, stream, c, seg, in, parts, out);
    } else if (cols > 4096 && cols <= 65536) {
        // The row in the registers of a 1024-thread workgroup: 2 to 16 pieces of 16 bytes per thread.
        const dim3 rows_grid(static_cast<unsigned>(rows));
        const size_t pieces = (cols + 4095) / 4096;
        if (pieces <= 2) hipLaunchKernelGGL(row_softmax_block_kernel<2>, rows_grid, dim3(1024), 0, stream, c, in, out);
        else if (pieces <= 4) hipLaunchKernelGGL(row_softmax_block_kernel<4>, rows_grid, dim3(1024), 0, stream, c, in, out);
        else if (pieces <= 8) hipLaunchKernelGGL(row_softmax_block_kernel<8>, rows_grid, dim3(1024), 0, stream, c, in, out);
        else if (pieces <= 12) hipLaunchKernelGGL(row_softmax_block_kernel<12>, rows_grid, dim3(1024), 0, stream, c, in, out);
        else hipLaunchKernelGGL(row_softmax_block_kernel<16>, rows_grid, dim3(1024), 0, stream, c, in, out);
    } else if (cols > 2048) {
        // A workgroup per row: 1024 threads while the rows are few, 256 once the rows alone fill the chip.
        const bool vec_long = cols % 4 == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
        const dim3 rows_grid(static_cast<unsigned>(rows));
        if (rows < 2048) {
            if (vec_long) hipLaunchKernelGGL((row_softmax_long_kernel<1024, true>), rows_grid, dim3(1024), 0, stream, c, in, out);
            else hipLaunchKernelGGL((row_softmax_long_kernel<1024, false>), rows_grid, dim3(1024), 0, stream, c, in, out);
        } else {
            if (vec_long) hipLaunchKernelGGL((row_softmax_long_kernel<256, true>), rows_grid, dim3(256), 0, stream, c, in, out);
            else hipLaunchKernelGGL((row_softmax_long_kernel<256, false>), rows_grid, dim3(256), 0, stream, c, in, out);
        }
    } else
        hipLaunchKernelGGL(row_softmax_kernel, grid, block, 0, stream, r, c, in, out);
    return hipGetLastError();
}

hipError_t launch_gelu_f32(size_t count, const float *in, float *out, hipStream_t stream)
{
    if (count == 0) return hipSuccess;
    if (vec_with_tail(count) && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0) {
        const size_t body = count / 4 * 4;
        hipLaunchKernelGGL(gelu_forward_vec_kernel, dim3(grid_for(count / 4)), dim3(256), 0, stream, count / 4,
                           reinterpret_cast<const float4 *>(in), reinterpret_cast<float4 *>(out));
        if (body < count) hipLaunchKernelGGL(gelu_forward_kernel, dim3(1), dim3(256), 0, stream, count - body, in + body, out + body);
    } else {
        hipLaunchKernelGGL(gelu_forward_kernel, dim3(grid_for(count)), dim3(256), 0, stream, count, in, out);
    }
    return hipGetLastError();
}

hipError_t launch_nonfinite_probe_f32(size_t count, const float *data, unsigned long long *status, hipStream_t stream)
{
    hipLaunchKernelGGL(nonfinite_probe_kernel, dim3(count ? grid_for(count) : 1), dim3(256), 0, stream, count, data, status);
    return hipGetLastError();
}

hipError_t launch_gelu_backward_f32(size_t count, const float *z, const float *grad, float *out, hipStream_t stream)
{
    if (count == 0) return hipSuccess;
    if (vec_with_tail(count) && aligned16(z) && aligned16(grad) && aligned16(out)) {
        const size_t body = count / 4 * 4;
        hipLaunchKernelGGL(gelu_backward_vec_kernel, dim3(grid_vec_for(count / 4)), dim3(256), 0, stream, count / 4,
                           reinterpret_cast<const float4 *>(z), reinterpret_cast<const float4 *>(grad),
                           reinterpret_cast<float4 *>(out));
        if (body < count)
            hipLaunchKernelGGL(gelu_backward_kernel, dim3(1), dim3(256), 0, stream, count - body, z + body, grad + body, out + body);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(gelu_backward_kernel, dim3(grid_for(count)), dim3(256), 0, stream, count, z, grad, out);
    return hipGetLastError();
}

hipError_t launch_scale_f32(size_t count, const float *in, float scale, float *out, hipStream_t stream)
{
    if (count == 0) return hipSuccess;
    if (vec_with_tail(count) && aligned16(in) && aligned16(out)) {
        const size_t body = count / 4 * 4;
        hipLaunchKernelGGL(scale_vec_kernel, dim3(grid_vec_for(count / 4)), dim3(256), 0, stream, count / 4,
                           reinterpret_cast<const float4 *>(in), scale, reinterpret_cast<float4 *>(out));
        if (body < count) hipLaunchKernelGGL(scale_kernel, dim3(1), dim3(256), 0, stream, count - body, in + body, scale, out + body);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(scale_kernel, dim3(grid_for(count)), dim3(256), 0, stream, count, in, scale, out);
    return hipGetLastError();
}

hipError_t launch_add_row_f32(size_t rows, size_t cols, float *data, const float *bias, hipStream_t stream)
{
    if (rows == 0 || cols == 0) return hipSuccess;
    if (cols % 4 == 0 && aligned16(data) && aligned16(bias)) {
        hipLaunchKernelGGL(add_row_vec_kernel, dim3(grid_vec_for(rows * cols / 4)), dim3(256), 0, stream, rows * cols / 4,
                           static_cast<int>(cols / 4), reinterpret_cast<float4 *>(data), reinterpret_cast<const float4 *>(bias));
        return hipGetLastError();
    }
    hipLaunchKernelGGL(add_row_kernel, dim3(grid_for(rows * cols)), dim3(256), 0, stream, rows * cols,
                       static_cast<int>(cols), data, bias);
    return hipGetLastError();
}

hipError_t launch_sum_axis0_f32(size_t rows, size_t cols, const float *in, float scale, float *out, hipStream_t stream)
{
    if (cols == 0) return hipSuccess;
    const bool vec = cols % 4 == 0 && (reinterpret_cast<uintptr_t>(in) & 15u) == 0;
    // Row chunks: about four workgroups per compute unit, at least 64 rows each (measured best on 16384 × 512: 9.0 µs
    // with 128-row chunks, 6.8 µs with 64, 9.0 µs with 32); the partial sums live in the stream's workspace and are
    // added in a fixed order.
    const size_t col_blocks = (cols + 255) / 256;
    size_t chunks = (1024 + col_blocks - 1) / col_blocks;
    const size_t max_chunks = (rows + 63) / 64;
    if (chunks > max_chunks) chunks = max_chunks;
    if (chunks == 0) chunks = 1;
    const size_t rows_per_chunk = (rows + chunks - 1) / chunks;
    if (rows_per_chunk > 0) chunks = (rows + rows_per_chunk - 1) / rows_per_chunk;
    if (chunks == 0) chunks = 1;
    void *workspace = nullptr;
    hipError_t rc = stream_workspace(stream, chunks * cols * sizeof(float), &workspace);
    if (rc != hipSuccess) return rc;
    float *partial = static_cast<float *>(workspace);
    const dim3 grid(static_cast<unsigned>(col_blocks), static_cast<unsigned>(chunks));
    if (vec)
        hipLaunchKernelGGL(sum_axis0_partial_vec_kernel<true>, grid, dim3(256), 0, stream, static_cast<int>(rows),
                           static_cast<int>(cols), static_cast<int>(rows_per_chunk), in, partial);
    else if (cols >= 64)
        hipLaunchKernelGGL(sum_axis0_partial_vec_kernel<false>, grid, dim3(256), 0, stream, static_cast<int>(rows),
                           static_cast<int>(cols), static_cast<int>(rows_per_chunk), in, partial);
    else
        hipLaunchKernelGGL(sum_axis0_partial_kernel, grid, dim3(256), 0, stream, static_cast<int>(rows),
                           static_cast<int>(cols), static_cast<int>(rows_per_chunk), in, partial);
    rc = hipGetLastError();
    if (rc != hipSuccess) return rc;
    hipLaunchKernelGGL(sum_axis0_final_wide_kernel, dim3(static_cast<unsigned>((cols + 15) / 16)), dim3(256), 0, stream,
                       static_cast<int>(chunks), static_cast<int>(cols), partial, scale, out);
    return hipGetLastError();
}

}  // namespace sthip
