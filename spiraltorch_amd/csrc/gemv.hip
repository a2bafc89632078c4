// Matrix times a few columns: C(m×n) = epilogue(A·B) with n <= 3 (f32) or n <= 7 (bf16, f32 accumulate), and
// Aᵀ·B for an f32 A stored k×m with n <= 4 (further down).
//
// The same entry points as the tiled GEMMs serve these shapes (hip_sgemm, crates/st-backend-hip/src/real.rs:598-646,
// and the bf16 GEMM beside it); a tile kernel would spend its loads on 64-byte row segments of A and its matrix
// instructions on padding.  Here the product is what it is, a stream over A: a wavefront (or, when there are few rows,
// a whole workgroup) owns one row of A, its lanes walk the row 16 bytes at a time with four loads in flight each, every
// lane keeps n partial sums, and a butterfly over the lanes finishes the row.  B (k×n, a few KB to a few hundred KB) is
// read through the caches by every row.  The order of the additions is fixed by the shape alone.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>

#include "device_math.h"
#include "kernels.h"

namespace sthip {

namespace {

struct GemvArgs {
    const void *A;
    const void *B;
    float *C32;
    uint16_t *C16;
    const float *bias;
    const float *residual;
    int M, N, K;
    float scale;
    int activation;
};

constexpr int kUnroll = 4;  // 16-byte loads of A in flight per lane

__device__ __forceinline__ float bf16_lo(uint32_t pair) { return __builtin_bit_cast(float, pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return __builtin_bit_cast(float, pair & 0xffff0000u); }

// Sum over the 64 lanes, the same tree in every wavefront.
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
    return v;
}

// Finishes a row: the cross-wavefront sum when the workgroup shares the row (WIDE), then the epilogue, written by lane 0.
template <int NC, bool WIDE>
__device__ __forceinline__ void finish_row(const GemvArgs &p, int row, bool active, float (&acc)[NC])
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] = wave_sum(acc[c]);
    if (WIDE) {
        __shared__ float part[4][NC];
        if (lane == 0)
#pragma unroll
            for (int c = 0; c < NC; ++c) part[wave][c] = acc[c];
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[c] = (part[0][c] + part[1][c]) + (part[2][c] + part[3][c]);
    }
    if (!active || lane != 0) return;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const size_t idx = static_cast<size_t>(row) * p.N + c;
        float value = acc[c] * p.scale + (p.bias ? p.bias[c] : -0.0f);
        if (p.residual) value += p.residual[idx];
        value = apply_activation(value, p.activation);
        if (p.C32) p.C32[idx] = value;
        if (p.C16) p.C16[idx] = f32_to_bf16_rne(value);
    }
}

// f32: K a multiple of 4, A and B 16-byte aligned.  NC = N, the columns of B.
// WIDE: one row per workgroup, the four wavefronts taking every fourth 256-wide piece of it.
template <int NC, bool WIDE>
__global__ __launch_bounds__(256) void gemv_f32_kernel(GemvArgs p)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = WIDE ? static_cast<int>(blockIdx.x) : static_cast<int>(blockIdx.x) * 4 + wave;
    const bool active = row < p.M;
    const int K = p.K;
    float acc[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] = 0.0f;
    if (active) {
        const float *a = static_cast<const float *>(p.A) + static_cast<size_t>(row) * K;
        const float *b = static_cast<const float *>(p.B);
        constexpr int PIECE = 256;  // floats one wavefront covers per load
        const int stride = (WIDE ? 4 : 1) * PIECE;
        for (int k0 = (WIDE ? wave : 0) * PIECE + lane * 4; k0 < K; k0 += stride * kUnroll) {
            float4 av[kUnroll];
            float bv[kUnroll][4 * NC];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int k = k0 + u * stride;
                av[u] = k < K ? *reinterpret_cast<const float4 *>(a + k) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int k = k0 + u * stride;
                // rows k .. k+3 of B are 4·N neighbouring floats
                const float4 *src = reinterpret_cast<const float4 *>(b + static_cast<size_t>(k) * NC);
#pragma unroll
                for (int q = 0; q < NC; ++q) {
                    const float4 v = k < K ? src[q] : make_float4(0.f, 0.f, 0.f, 0.f);
                    bv[u][4 * q + 0] = v.x; bv[u][4 * q + 1] = v.y; bv[u][4 * q + 2] = v.z; bv[u][4 * q + 3] = v.w;
                }
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const float ae[4] = {av[u].x, av[u].y, av[u].z, av[u].w};
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int c = 0; c < NC; ++c) acc[c] = fmaf(ae[j], bv[u][j * NC + c], acc[c]);
            }
        }
    }
    finish_row<NC, WIDE>(p, row, active, acc);
}

// bf16: K a multiple of 8, A and B 16-byte aligned; B row-major (k×n) or packed (n×k).  N == NC exactly.
template <int NC, bool WIDE, bool PACKED>
__global__ __launch_bounds__(256) void gemv_bf16_kernel(GemvArgs p)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = WIDE ? static_cast<int>(blockIdx.x) : static_cast<int>(blockIdx.x) * 4 + wave;
    const bool active = row < p.M;
    const int K = p.K;
    float acc[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] = 0.0f;
    if (active) {
        const uint16_t *a = static_cast<const uint16_t *>(p.A) + static_cast<size_t>(row) * K;
        const uint16_t *b = static_cast<const uint16_t *>(p.B);
        constexpr int PIECE = 512;  // bf16 values one wavefront covers per load
        const int stride = (WIDE ? 4 : 1) * PIECE;
        constexpr int U = NC > 4 ? 2 : kUnroll;
        for (int k0 = (WIDE ? wave : 0) * PIECE + lane * 8; k0 < K; k0 += stride * U) {
            uint4 av[U];
            uint4 bv[U][NC];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int k = k0 + u * stride;
                av[u] = k < K ? *reinterpret_cast<const uint4 *>(a + k) : make_uint4(0u, 0u, 0u, 0u);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int k = k0 + u * stride;
#pragma unroll
                for (int q = 0; q < NC; ++q) {
                    // packed: the 8 k-values of column q; row-major: 16-byte piece q of the 8·N values of rows k .. k+7
                    const uint16_t *src = PACKED ? b + static_cast<size_t>(q) * K + k : b + static_cast<size_t>(k) * NC + 8 * q;
                    bv[u][q] = k < K ? *reinterpret_cast<const uint4 *>(src) : make_uint4(0u, 0u, 0u, 0u);
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t aw[4] = {av[u].x, av[u].y, av[u].z, av[u].w};
                float ae[8];
#pragma unroll
                for (int j = 0; j < 4; ++j) { ae[2 * j] = bf16_lo(aw[j]); ae[2 * j + 1] = bf16_hi(aw[j]); }
                uint32_t bw[4 * NC];
#pragma unroll
                for (int q = 0; q < NC; ++q) { bw[4 * q] = bv[u][q].x; bw[4 * q + 1] = bv[u][q].y; bw[4 * q + 2] = bv[u][q].z; bw[4 * q + 3] = bv[u][q].w; }
#pragma unroll
                for (int j = 0; j < 8; ++j)
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        const int e = PACKED ? c * 8 + j : j * NC + c;  // bf16 index inside the 8·NC values
                        const float be = (e & 1) ? bf16_hi(bw[e >> 1]) : bf16_lo(bw[e >> 1]);
                        acc[c] = fmaf(ae[j], be, acc[c]);
                    }
            }
        }
    }
    finish_row<NC, WIDE>(p, row, active, acc);
}

bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

// One wavefront per row once that gives every SIMD a few rows; below that a workgroup per row.
bool wide_rows(size_t m, size_t k, size_t piece) { return m < 4096 && k >= 8 * piece; }

template <int NC>
hipError_t launch_f32(const GemvArgs &args, hipStream_t stream)
{
    const bool wide = wide_rows(args.M, args.K, 256);
    const unsigned groups = wide ? static_cast<unsigned>(args.M) : static_cast<unsigned>((args.M + 3) / 4);
    if (wide) hipLaunchKernelGGL((gemv_f32_kernel<NC, true>), dim3(groups), dim3(256), 0, stream, args);
    else hipLaunchKernelGGL((gemv_f32_kernel<NC, false>), dim3(groups), dim3(256), 0, stream, args);
    return hipGetLastError();
}

template <int NC>
hipError_t launch_bf16(const GemvArgs &args, bool packed, hipStream_t stream)
{
    const bool wide = wide_rows(args.M, args.K, 512);
    const unsigned groups = wide ? static_cast<unsigned>(args.M) : static_cast<unsigned>((args.M + 3) / 4);
    if (wide) {
        if (packed) hipLaunchKernelGGL((gemv_bf16_kernel<NC, true, true>), dim3(groups), dim3(256), 0, stream, args);
        else hipLaunchKernelGGL((gemv_bf16_kernel<NC, true, false>), dim3(groups), dim3(256), 0, stream, args);
    } else {
        if (packed) hipLaunchKernelGGL((gemv_bf16_kernel<NC, false, true>), dim3(groups), dim3(256), 0, stream, args);
        else hipLaunchKernelGGL((gemv_bf16_kernel<NC, false, false>), dim3(groups), dim3(256), 0, stream, args);
    }
    return hipGetLastError();
}

GemvArgs make_args(size_t m, size_t n, size_t k, const void *lhs, const void *rhs, float *out_f32, uint16_t *out_bf16,
                   const GemmEpilogue &epilogue)
{
    GemvArgs args;
    args.A = lhs;
    args.B = rhs;
    args.C32 = out_f32;
    args.C16 = out_bf16;
    args.bias = epilogue.bias;
    args.residual = epilogue.residual;
    args.M = static_cast<int>(m);
    args.N = static_cast<int>(n);
    args.K = static_cast<int>(k);
    args.scale = epilogue.scale;
    args.activation = epilogue.activation;
    return args;
}

// -------------------------------------------------------------------------------------------------
// Aᵀ·B with A stored k×m (the gradient of a matrix-vector product with respect to the vector): the rows of the stored
// matrix run along the OUTPUT, so a lane owns four adjacent outputs and walks down the k rows of its slice, a wavefront
// reading 1 KB of one stored row per load.  The four wavefronts of a workgroup take eight rows each of every 32, the
// grid's second dimension cuts k into slices, and every (slice, output) sum goes to scratch memory: the reduction
// kernel adds the slices in order and applies the epilogue.  Rows need no alignment (16-byte loads take any address
// here); the last lanes of a row whose four outputs straddle its end load one value at a time.
// -------------------------------------------------------------------------------------------------
typedef float gemv_f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

struct GemvTArgs {
    const float *A;   // k × m
    const float *B;   // k × n
    float *partial;   // slices × m × n
    int M, K;
    int rows_per_slice;  // a multiple of 32
};

template <int NC>
__global__ __launch_bounds__(256) void gemv_t_f32_kernel(GemvTArgs p)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
    const int M = p.M;
    const int col = static_cast<int>(blockIdx.x) * 256 + lane * 4;
    const int valid = min(4, M - col);  // <= 0: nothing of this lane's quad exists
    const int k_begin = static_cast<int>(blockIdx.y) * p.rows_per_slice;
    const int k_end = min(p.K, k_begin + p.rows_per_slice);
    float acc[NC][4];
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[c][e] = 0.0f;
    for (int k0 = k_begin + wave * 8; k0 < k_end; k0 += 32) {
        float a[8][4];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int row = k0 + j;
            const float *src = p.A + static_cast<size_t>(row) * M + col;
#pragma unroll
            for (int e = 0; e < 4; ++e) a[j][e] = 0.0f;
            if (row < k_end) {
                if (valid == 4) {
                    const gemv_f32x4_a4 t = *reinterpret_cast<const gemv_f32x4_a4 *>(src);
                    a[j][0] = t[0]; a[j][1] = t[1]; a[j][2] = t[2]; a[j][3] = t[3];
                } else {
#pragma unroll
                    for (int e = 0; e < 3; ++e)
                        if (e < valid) a[j][e] = src[e];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int row = k0 + j;  // the same for the whole wavefront: B comes through the scalar cache
            if (row < k_end) {
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const float b = p.B[static_cast<size_t>(row) * NC + c];
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[c][e] = fmaf(a[j][e], b, acc[c][e]);
                }
            }
        }
    }
    __shared__ float part[4][NC][256];
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int e = 0; e < 4; ++e) part[wave][c][lane * 4 + e] = acc[c][e];
    __syncthreads();
    const int out_col = static_cast<int>(blockIdx.x) * 256 + static_cast<int>(threadIdx.x);
    if (out_col >= M) return;
    float *dst = p.partial + (static_cast<size_t>(blockIdx.y) * M + out_col) * NC;
#pragma unroll
    for (int c = 0; c < NC; ++c)
        dst[c] = (part[0][c][threadIdx.x] + part[1][c][threadIdx.x]) + (part[2][c][threadIdx.x] + part[3][c][threadIdx.x]);
}

struct GemvTReduceArgs {
    const float *partial;
    float *C;
    const float *bias;
    const float *residual;
    size_t plane;  // m · n
    int N, slices;
    float scale;
    int activation;
};

__global__ __launch_bounds__(256) void gemv_t_reduce_kernel(GemvTReduceArgs p)
{
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= p.plane) return;
    float value = 0.0f;
    for (int s0 = 0; s0 < p.slices; s0 += 8) {
        float piece[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) piece[j] = (s0 + j < p.slices) ? p.partial[(s0 + j) * p.plane + idx] : 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) value += piece[j];
    }
    value = value * p.scale + (p.bias ? p.bias[idx % p.N] : -0.0f);
    if (p.residual) value += p.residual[idx];
    p.C[idx] = apply_activation(value, p.activation);
}

template <int NC>
hipError_t launch_t_f32(const GemvTArgs &args, unsigned col_blocks, unsigned slices, hipStream_t stream)
{
    hipLaunchKernelGGL(gemv_t_f32_kernel<NC>, dim3(col_blocks, slices), dim3(256), 0, stream, args);
    return hipGetLastError();
}

}  // namespace

bool gemv_f32_applies(size_t m, size_t n, size_t k, const float *lhs, const float *rhs)
{
    // k: at least one full 256-wide piece per row, or most lanes of a wavefront idle
    return n >= 1 && n <= 3 && m >= 64 && k >= 256 && k % 4 == 0 && aligned16(lhs) && aligned16(rhs) && m < (1ull << 31) &&
           k < (1ull << 31);
}

hipError_t launch_gemv_f32(size_t m, size_t n, size_t k, const float *lhs, const float *rhs, float *out,
                           const GemmEpilogue &epilogue, hipStream_t stream)
{
    const GemvArgs args = make_args(m, n, k, lhs, rhs, out, nullptr, epilogue);
    if (n == 1) return launch_f32<1>(args, stream);
    if (n == 2) return launch_f32<2>(args, stream);
    return launch_f32<3>(args, stream);
}

bool gemv_bf16_applies(size_t m, size_t n, size_t k, const uint16_t *lhs, const uint16_t *rhs)
{
    // Eight columns are faster on the tile kernel (4096×8×4096: 21 µs against 35), five to seven are not: their rows
    // of B are not 16-byte aligned there.
    return n >= 1 && n <= 7 && m >= 64 && k >= 512 && k % 8 == 0 && aligned16(lhs) && aligned16(rhs) && m < (1ull << 31) &&
           k < (1ull << 31);
}

hipError_t launch_gemv_bf16(size_t m, size_t n, size_t k, const uint16_t *lhs, const uint16_t *rhs, bool rhs_packed,
                            float *out_f32, uint16_t *out_bf16, const GemmEpilogue &epilogue, hipStream_t stream)
{
    const GemvArgs args = make_args(m, n, k, lhs, rhs, out_f32, out_bf16, epilogue);
    switch (n) {
    case 1: return launch_bf16<1>(args, rhs_packed, stream);
    case 2: return launch_bf16<2>(args, rhs_packed, stream);
    case 3: return launch_bf16<3>(args, rhs_packed, stream);
    case 4: return launch_bf16<4>(args, rhs_packed, stream);
    case 5: return launch_bf16<5>(args, rhs_packed, stream);
    case 6: return launch_bf16<6>(args, rhs_packed, stream);
    default: return launch_bf16<7>(args, rhs_packed, stream);
    }
}

bool gemv_t_f32_applies(size_t m, size_t n, size_t k)
{
    return n >= 1 && n <= 4 && m >= 1024 && k >= 64 && m < (1ull << 31) && k < (1ull << 31);
}

hipError_t launch_gemv_t_f32(size_t m, size_t n, size_t k, const float *lhs, const float *rhs, float *out,
                             const GemmEpilogue &epilogue, hipStream_t stream)
{
    const size_t col_blocks = (m + 255) / 256;
    // About 2048 workgroups (eight per compute unit), slices of at least 64 rows.
    size_t slices = std::max<size_t>(1, std::min((2048 + col_blocks - 1) / col_blocks, k / 64));
    slices = std::min<size_t>(slices, 65535);
    const size_t rows_per_slice = ((k + slices - 1) / slices + 31) / 32 * 32;
    slices = (k + rows_per_slice - 1) / rows_per_slice;
    const size_t plane = m * n;
    void *workspace = nullptr;
    hipError_t rc = stream_workspace(stream, slices * plane * sizeof(float), &workspace);
    if (rc != hipSuccess) return rc;
    GemvTArgs args;
    args.A = lhs;
    args.B = rhs;
    args.partial = static_cast<float *>(workspace);
    args.M = static_cast<int>(m);
    args.K = static_cast<int>(k);
    args.rows_per_slice = static_cast<int>(rows_per_slice);
    const unsigned blocks = static_cast<unsigned>(col_blocks), cuts = static_cast<unsigned>(slices);
    switch (n) {
    case 1: rc = launch_t_f32<1>(args, blocks, cuts, stream); break;
    case 2: rc = launch_t_f32<2>(args, blocks, cuts, stream); break;
    case 3: rc = launch_t_f32<3>(args, blocks, cuts, stream); break;
    default: rc = launch_t_f32<4>(args, blocks, cuts, stream); break;
    }
    if (rc != hipSuccess) return rc;
    GemvTReduceArgs reduce;
    reduce.partial = args.partial;
    reduce.C = out;
    reduce.bias = epilogue.bias;
    reduce.residual = epilogue.residual;
    reduce.plane = plane;
    reduce.N = static_cast<int>(n);
    reduce.slices = static_cast<int>(slices);
    reduce.scale = epilogue.scale;
    reduce.activation = epilogue.activation;
    hipLaunchKernelGGL(gemv_t_reduce_kernel, dim3(static_cast<unsigned>((plane + 255) / 256)), dim3(256), 0, stream, reduce);
    return hipGetLastError();
}

}  // namespace sthip
