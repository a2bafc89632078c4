// f32 GEMM on the native f32 matrix cores of gfx950 (v_mfma_f32_32x32x2_f32) with the fused
// scale / bias / residual / activation epilogue.
//
// Replaces rocBLAS sgemm + st_gemm_epilogue_f32 in crates/st-backend-hip/src/real.rs:598-646,817-957
// and crates/st-backend-hip/src/hip_kernels/hip_gemm_epilogue.cu:19-71.
//
// Tiling: a workgroup of WM×WN wavefronts owns a BM×BN tile of C and walks K in steps of 16 through two
// LDS stages; global loads for step t+1 are issued into registers before the MFMAs of step t and written
// to the other stage afterwards, so a step costs one barrier.  The f32 MFMA is slow (64 cycles for
// 32x32x2) and needs two LDS values per lane, so register blocking buys nothing here; what keeps the
// matrix pipe busy is MANY wavefronts with small tiles (measured: 32×32 or 64×64 per wavefront, 4 to 16
// wavefronts per workgroup, beat 2×2 wavefronts with 64×64 tiles by 1.5×).
//
// MFMA operand layout (32x32x2): lane l supplies A[l%32][l/32] and B[l/32][l%32]; accumulator register
// r of lane l is C[(r/4)*8 + (l/32)*4 + r%4][l%32].  Because the sum over k is order-free, each group
// of 8 k-values is issued as the pairs {s, s+4}: lane half h = l/32 then needs k = 4h..4h+3 of the
// group, which is ONE 128-bit LDS read per operand row when the tile is stored k-contiguous.
#include "device_math.h"
#include "kernels.h"

#include <algorithm>
#include <type_traits>

namespace sthip {

namespace {

struct GemmF32Args {
    const float *A;
    const float *B;
    float *C;
    const float *bias;
    const float *residual;
    int M, N, K;
    int tiles_m, tiles_n;  // the grid is one-dimensional over (tile_m, tile_n)
    float scale;
    int activation;
    // k-sliced form (few tiles, long k): workgroup (tile, blockIdx.y) covers k in [y·slice_k, (y+1)·slice_k) and writes
    // its raw sums to plane y of C (the launch passes the workspace of partial planes as C, scale 1 and no bias,
    // residual or activation); gemm_f32_slice_reduce_kernel adds the planes in order and applies the epilogue.
    int slice_k = 0;  // 0: one slice, the whole of K
    // Batched form: product blockIdx.z reads A + z·a_batch and writes C + z·c_batch (B is shared).
    size_t a_batch = 0, c_batch = 0;
};

constexpr int kBK = 16;

template <bool VEC>
__device__ __forceinline__ float4 load_row4(const float *base, size_t row_offset, int col, int col_limit,
                                            bool row_valid)
{
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (!row_valid) return v;
    const float *src = base + row_offset + col;
    if (VEC) {
        if (col < col_limit) v = *reinterpret_cast<const float4 *>(src);
    } else if (col + 4 <= col_limit) {
        // Four values inside the row at any 4-byte alignment: still one 16-byte load (global memory takes wide
        // accesses at any alignment; the type says so, and the compiler keeps the single instruction).
        typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
        const f32x4_a4 w = *reinterpret_cast<const f32x4_a4 *>(src);
        v = make_float4(w[0], w[1], w[2], w[3]);
    } else {
        if (col + 0 < col_limit) v.x = src[0];
        if (col + 1 < col_limit) v.y = src[1];
        if (col + 2 < col_limit) v.z = src[2];
        if (col + 3 < col_limit) v.w = src[3];
    }
    return v;
}

template <int BM, int BN, int WM, int WN, bool AT, bool VEC>
__global__ __launch_bounds__(64 * WM * WN) void gemm_f32_kernel(GemmF32Args p)
{
    constexpr int T = 64 * WM * WN;
    constexpr int WTM = BM / WM, WTN = BN / WN;  // wavefront tile
    constexpr int TM = WTM / 32, TN = WTN / 32;  // 32×32 MFMA tiles per wavefront
    static_assert(TM >= 1 && TN >= 1, "wavefront tile must be at least 32×32");
    constexpr int A_STRIDE = AT ? (BM + 8) : (kBK + 4);
    constexpr int A_ELEMS = AT ? kBK * A_STRIDE : BM * A_STRIDE;
    constexpr int B_STRIDE = BN + 8;
    constexpr int B_ELEMS = kBK * B_STRIDE;
    constexpr int A_VECS = BM * kBK / 4, B_VECS = kBK * BN / 4;  // float4 per stage
    constexpr int A_LOADS = (A_VECS + T - 1) / T, B_LOADS = (B_VECS + T - 1) / T;
    __shared__ __attribute__((aligned(16))) float As[2][A_ELEMS];
    __shared__ __attribute__((aligned(16))) float Bs[2][B_ELEMS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int li = lane & 31, lh = lane >> 5;
    // Workgroup ids go round-robin over the 8 XCDs, each with its own L2.  Give every XCD one contiguous run of
    // tile ids, and walk the tiles in groups of GROUP_M tile-rows (column by column inside a group), so the
    // tiles resident on one XCD at a time share their A row panels and B column panels through that L2.
    constexpr int GROUP_M = BM >= 256 ? 4 : 8;
    const int grid = static_cast<int>(gridDim.x), xcd = static_cast<int>(blockIdx.x) & 7;
    const int tile_id = xcd * (grid >> 3) + min(xcd, grid & 7) + (static_cast<int>(blockIdx.x) >> 3);
    const int group_size = GROUP_M * p.tiles_n;
    const int first_m = (tile_id / group_size) * GROUP_M, in_group = tile_id % group_size;
    const int group_rows = min(p.tiles_m - first_m, GROUP_M);
    const int tile_m = first_m + in_group % group_rows, tile_n = in_group / group_rows;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int M = p.M, N = p.N;
    // This workgroup's k range [k_lo, K): K below is the END of the range, p.K stays the row stride of A.
    const int k_lo = p.slice_k ? static_cast<int>(blockIdx.y) * p.slice_k : 0;
    const int K = p.slice_k ? min(p.K, k_lo + p.slice_k) : p.K;
    float *const C = p.C + static_cast<size_t>(blockIdx.y) * M * N + static_cast<size_t>(blockIdx.z) * p.c_batch;
    const float *const A = p.A + static_cast<size_t>(blockIdx.z) * p.a_batch;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
            acc[a][b] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    float4 ra[A_LOADS], rb[B_LOADS];

    // Fast-path source pointers (k-tile 0): rows/columns outside the matrix are clamped to the last valid
    // one instead of being masked — what they load only reaches output elements that are never stored.
    // Only a ragged last k-tile needs real zero-fill, and it takes the checked path below.
    const float *a_src[A_LOADS];
    const float *b_src[B_LOADS];
    if (VEC) {
#pragma unroll
        for (int r = 0; r < A_LOADS; ++r) {
            const int f = tid + T * r;
            if (!AT) {
                const int row = min(m0 + (f >> 2), M - 1), c4 = (f & 3) * 4;
                a_src[r] = A + static_cast<size_t>(row) * p.K + c4;
            } else {
                const int krow = f / (BM / 4), col = min(m0 + (f % (BM / 4)) * 4, M - 4);
                a_src[r] = A + static_cast<size_t>(krow) * M + col;
            }
        }
#pragma unroll
        for (int r = 0; r < B_LOADS; ++r) {
            const int f = tid + T * r;
            const int krow = f / (BN / 4), col = min(n0 + (f % (BN / 4)) * 4, N - 4);
            b_src[r] = p.B + static_cast<size_t>(krow) * N + col;
        }
    }
    const int full_steps = (K - k_lo) / kBK;  // k-tiles that lie completely inside the range

    auto load_fast = [&](int k0) {
#pragma unroll
        for (int r = 0; r < A_LOADS; ++r) {
            if (A_VECS % T != 0 && tid + T * r >= A_VECS) continue;
            ra[r] = *reinterpret_cast<const float4 *>(a_src[r] + (AT ? static_cast<size_t>(k0) * M : static_cast<size_t>(k0)));
        }
#pragma unroll
        for (int r = 0; r < B_LOADS; ++r) {
            if (B_VECS % T != 0 && tid + T * r >= B_VECS) continue;
            rb[r] = *reinterpret_cast<const float4 *>(b_src[r] + static_cast<size_t>(k0) * N);
        }
    };
    auto load_checked = [&](int k0) {
#pragma unroll
        for (int r = 0; r < A_LOADS; ++r) {
            const int f = tid + T * r;
            if (A_VECS % T != 0 && f >= A_VECS) continue;
            if (!AT) {
                const int row = f >> 2, c4 = (f & 3) * 4;
                ra[r] = load_row4<VEC>(A, static_cast<size_t>(m0 + row) * p.K, k0 + c4, K, m0 + row < M);
            } else {
                const int krow = f / (BM / 4), c4 = (f % (BM / 4)) * 4;
                ra[r] = load_row4<VEC>(A, static_cast<size_t>(k0 + krow) * M, m0 + c4, M, k0 + krow < K);
            }
        }
#pragma unroll
        for (int r = 0; r < B_LOADS; ++r) {
            const int f = tid + T * r;
            if (B_VECS % T != 0 && f >= B_VECS) continue;
            const int krow = f / (BN / 4), c4 = (f % (BN / 4)) * 4;
            rb[r] = load_row4<VEC>(p.B, static_cast<size_t>(k0 + krow) * N, n0 + c4, N, k0 + krow < K);
        }
    };
    auto store_lds = [&](int stage) {
#pragma unroll
        for (int r = 0; r < A_LOADS; ++r) {
            const int f = tid + T * r;
            if (A_VECS % T != 0 && f >= A_VECS) continue;
            if (!AT) {
                const int row = f >> 2, c4 = (f & 3) * 4;
                *reinterpret_cast<float4 *>(&As[stage][row * A_STRIDE + c4]) = ra[r];
            } else {
                const int krow = f / (BM / 4), c4 = (f % (BM / 4)) * 4;
                *reinterpret_cast<float4 *>(&As[stage][krow * A_STRIDE + c4]) = ra[r];
            }
        }
#pragma unroll
        for (int r = 0; r < B_LOADS; ++r) {
            const int f = tid + T * r;
            if (B_VECS % T != 0 && f >= B_VECS) continue;
            const int krow = f / (BN / 4), c4 = (f % (BN / 4)) * 4;
            *reinterpret_cast<float4 *>(&Bs[stage][krow * B_STRIDE + c4]) = rb[r];
        }
    };
    auto compute = [&](int stage) {
        const float *as = As[stage];
        const float *bs = Bs[stage];
#pragma unroll
        for (int kk = 0; kk < kBK / 8; ++kk) {
            float a[TM][4], b[TN][4];
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                const int row = wm * WTM + tm * 32 + li;
                if (!AT) {
                    const float4 v = *reinterpret_cast<const float4 *>(&as[row * A_STRIDE + kk * 8 + lh * 4]);
                    a[tm][0] = v.x; a[tm][1] = v.y; a[tm][2] = v.z; a[tm][3] = v.w;
                } else {
#pragma unroll
                    for (int s = 0; s < 4; ++s) a[tm][s] = as[(kk * 8 + lh * 4 + s) * A_STRIDE + row];
                }
            }
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
                const int col = wn * WTN + tn * 32 + li;
#pragma unroll
                for (int s = 0; s < 4; ++s) b[tn][s] = bs[(kk * 8 + lh * 4 + s) * B_STRIDE + col];
            }
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn)
                        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[tm][s], b[tn][s], acc[tm][tn], 0, 0, 0);
        }
    };

    const int steps = (K - k_lo + kBK - 1) / kBK;
    if (steps > 0) {
        if (VEC && full_steps > 0) load_fast(k_lo); else load_checked(k_lo);
        store_lds(0);
    }
    __syncthreads();
    int t = 0;
    if (VEC) {
        // Steady state: the next k-tile lies completely inside K, so its loads need no checks.
        for (; t + 1 < full_steps; ++t) {
            load_fast(k_lo + (t + 1) * kBK);
            compute(t & 1);
            store_lds((t + 1) & 1);
            __syncthreads();
        }
    }
    for (; t < steps; ++t) {
        const bool more = t + 1 < steps;
        if (more) load_checked(k_lo + (t + 1) * kBK);
        compute(t & 1);
        if (more) store_lds((t + 1) & 1);
        __syncthreads();
    }

    // Epilogue: value = acc*scale; (value + bias[col]) + residual; activation.
    // scale 1.0f and the bias stand-in -0.0f leave every value as it is, so neither needs a branch.
    with_epilogue_ops(p.activation, p.residual != nullptr, [&](auto &&act, auto has_residual) {
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const int col = n0 + wn * WTN + tn * 32 + li;
            const bool col_ok = col < N;
            const float bias = (p.bias && col_ok) ? p.bias[col] : -0.0f;
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                const f32x16 tile = acc[tm][tn];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = m0 + wm * WTM + tm * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                    if (col_ok && row < M) {
                        const size_t idx = static_cast<size_t>(row) * N + col;
                        float value = tile[r] * p.scale + bias;
                        if constexpr (decltype(has_residual)::value) value += p.residual[idx];
                        C[idx] = act(value);
                    }
                }
            }
        }
    });
}

// Adds the partial planes of a k-sliced launch in slice order (so the result does not depend on scheduling) and applies
// the epilogue.  One thread per output element; eight planes are requested together so the loads overlap.
struct SliceReduceArgs {
    const float *partial;
    float *C;
    const float *bias;
    const float *residual;
    size_t plane;
    int N, slices;
    float scale;
    int activation;
};
__global__ __launch_bounds__(256) void gemm_f32_slice_reduce_kernel(SliceReduceArgs p)
{
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= p.plane) return;
    float value = 0.0f;
    for (int s0 = 0; s0 < p.slices; s0 += 8) {
        float part[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) part[j] = (s0 + j < p.slices) ? p.partial[(s0 + j) * p.plane + idx] : 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) value += part[j];
    }
    value = value * p.scale + (p.bias ? p.bias[idx % p.N] : -0.0f);
    if (p.residual) value += p.residual[idx];
    p.C[idx] = apply_activation(value, p.activation);
}

// The same for many slices of a small plane (64×64×100000 is 128 slices of 4096 values: one thread per value would walk
// 128 loads in sixteen dependent rounds on sixteen workgroups): sixteen lanes per output value, lane j adding slices
// j, j + 16, ... in order, then a butterfly over the sixteen — a fixed tree, so still independent of scheduling.
__global__ __launch_bounds__(256) void gemm_f32_slice_reduce_wide_kernel(SliceReduceArgs p)
{
    const int lane16 = threadIdx.x & 15;
    const size_t idx = static_cast<size_t>(blockIdx.x) * 16 + (threadIdx.x >> 4);
    const bool valid = idx < p.plane;
    float value = 0.0f;
    for (int s0 = lane16; s0 < p.slices; s0 += 128) {
        float part[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) part[j] = (valid && s0 + 16 * j < p.slices) ? p.partial[(s0 + 16 * j) * p.plane + idx] : 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) value += part[j];
    }
#pragma unroll
    for (int offset = 8; offset > 0; offset >>= 1) value += __shfl_xor(value, offset, 16);
    if (!valid || lane16 != 0) return;
    value = value * p.scale + (p.bias ? p.bias[idx % p.N] : -0.0f);
    if (p.residual) value += p.residual[idx];
    p.C[idx] = apply_activation(value, p.activation);
}

// How many k-slices a launch of `tiles` workgroups, each walking `k_steps` k-tiles, is cut into: none while the tiles
// alone give every other compute unit a workgroup; otherwise enough for about two workgroups per compute unit, each
// slice keeping at least `min_steps` k-tiles, and the partial planes (written once, read once) staying below the
// operands' bytes.
size_t choose_k_slices(size_t m, size_t n, size_t k, size_t tiles, size_t k_steps, size_t min_steps, size_t most_tiles = 128,
                       size_t most_groups = 512)
{
    if (tiles > most_tiles || k_steps < 2 * min_steps) return 1;
    size_t slices = std::min<size_t>(most_groups / tiles, k_steps / min_steps);
    while (slices > 1 && slices * m * n * 2 > m * k + k * n) --slices;
    return std::max<size_t>(slices, 1);
}

// Runs `launch(args)` k-sliced: partial planes in the stream's workspace, then the reduction with the epilogue.
template <class Launch>
hipError_t launch_k_sliced(GemmF32Args args, size_t slices, size_t k_steps, int bk, hipStream_t stream, Launch &&launch)
{
    const size_t steps_per_slice = (k_steps + slices - 1) / slices;
    slices = (k_steps + steps_per_slice - 1) / steps_per_slice;
    const size_t plane = static_cast<size_t>(args.M) * args.N;
    void *workspace = nullptr;
    hipError_t rc = stream_workspace(stream, slices * plane * sizeof(float), &workspace);
    if (rc != hipSuccess) return rc;
    SliceReduceArgs reduce;
    reduce.partial = static_cast<const float *>(workspace);
    reduce.C = args.C;
    reduce.bias = args.bias;
    reduce.residual = args.residual;
    reduce.plane = plane;
    reduce.N = args.N;
    reduce.slices = static_cast<int>(slices);
    reduce.scale = args.scale;
    reduce.activation = args.activation;
    args.C = static_cast<float *>(workspace);
    args.bias = nullptr;
    args.residual = nullptr;
    args.scale = 1.0f;
    args.activation = ST_HIP_ACT_NONE;
    args.slice_k = static_cast<int>(steps_per_slice) * bk;
    rc = launch(args, static_cast<unsigned>(slices));
    if (rc != hipSuccess) return rc;
    if (slices >= 32 && plane <= 65536)
        hipLaunchKernelGGL(gemm_f32_slice_reduce_wide_kernel, dim3(static_cast<unsigned>((plane + 15) / 16)), dim3(256), 0, stream,
                           reduce);
    else
        hipLaunchKernelGGL(gemm_f32_slice_reduce_kernel, dim3(static_cast<unsigned>((plane + 255) / 256)), dim3(256), 0, stream,
                           reduce);
    return hipGetLastError();
}

template <int BM, int BN, int WM, int WN>
hipError_t launch_tile(GemmF32Args args, bool lhs_transposed, bool vec, hipStream_t stream, unsigned slices = 1, unsigned batch = 1)
{
    args.tiles_n = (args.N + BN - 1) / BN;
    args.tiles_m = (args.M + BM - 1) / BM;
    const size_t tiles = static_cast<size_t>(args.tiles_n) * static_cast<size_t>(args.tiles_m);
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    const dim3 grid(static_cast<unsigned>(tiles), slices, batch);
    const dim3 block(64 * WM * WN);
    if (lhs_transposed) {
        if (vec)
            hipLaunchKernelGGL((gemm_f32_kernel<BM, BN, WM, WN, true, true>), grid, block, 0, stream, args);
        else
            hipLaunchKernelGGL((gemm_f32_kernel<BM, BN, WM, WN, true, false>), grid, block, 0, stream, args);
    } else {
        if (vec)
            hipLaunchKernelGGL((gemm_f32_kernel<BM, BN, WM, WN, false, true>), grid, block, 0, stream, args);
        else
            hipLaunchKernelGGL((gemm_f32_kernel<BM, BN, WM, WN, false, false>), grid, block, 0, stream, args);
    }
    return hipGetLastError();
}


bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

// -------------------------------------------------------------------------------------------------
// Ring kernel for K % 16 == 0 and 16-byte aligned rows.  On a SIMD the f32 MFMAs and ordinary vector
// instructions do not overlap — measured, every VALU, LDS or memory instruction a wavefront issues takes
// roughly 8 to 15 cycles away from the matrix pipe — so this loop issues as few of them as possible:
// both operands go global memory -> LDS with buffer_load ... lds (16 bytes per lane, no registers, no
// ds_write) into a three-deep ring of 16-wide k-tiles; the per-lane memory offsets are loop constants and
// the k-tile advance rides in the instruction's scalar offset; the ring slot is a compile-time constant of
// the 3x unrolled loop, so the fragment reads use immediate offsets.  What is left per k-tile and wavefront
// is the fragment reads, LOADS load instructions and the MFMAs.
//
// Everything that could read outside a matrix is flagged through the vector offset alone (rows past M or
// columns past N get an offset beyond the buffer's range and read as zero); K needs no guard.
//
// A (row-major m×k): stage rows hold 16 k-values (64 B); 16-byte chunk c of row r sits at c ^ ((r >> 2) & 3).
// A stored k×m (lhs_transposed) and B (k×n): stage rows are k, BM or BN floats long, unpadded.
// BT: B is given prepacked as n×k (the column-major packing of PackedB, crates/st-tensor/src/pure.rs:1285-1323)
// and is staged exactly like a row-major A, so its fragments are 128-bit reads too.
// -------------------------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void *lds_void_ptr;

#define ST_F32_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (7 << 4) | (15 << 8) | ((((n) >> 4) & 3) << 14))

template <int BM, int BN, int WM, int WN, bool AT, bool BT>
__device__ __forceinline__ void gemm_f32_ring_body(const GemmF32Args &p)
{
    constexpr int BK = 16, RING = 3;
    constexpr int WAVES = WM * WN;
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(TM >= 1 && TN >= 1, "wavefront tile must be at least 32×32");
    constexpr int NA = BM / 16, NB = BN / 16;  // 1 KB load instructions per stage and operand
    static_assert(NA % WAVES == 0 && NB % WAVES == 0, "load instructions divide evenly over the wavefronts");
    constexpr int LOADS_A = NA / WAVES, LOADS = (NA + NB) / WAVES;  // per wavefront: first the A loads, then B
    constexpr int A_BYTES = BM * BK * 4, B_BYTES = BK * BN * 4;
    constexpr int STAGE = A_BYTES + B_BYTES;
    static_assert(RING * STAGE <= 65536, "fragment reads address the ring with 16-bit immediates");

    extern __shared__ __attribute__((aligned(16))) unsigned char ring_lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int li = lane & 31, lh = lane >> 5;
    const int M = p.M, N = p.N, K = p.K;

    constexpr int GROUP_M = 8;
    const int grid = static_cast<int>(gridDim.x), xcd = static_cast<int>(blockIdx.x) & 7;
    const int tile_id = xcd * (grid >> 3) + min(xcd, grid & 7) + (static_cast<int>(blockIdx.x) >> 3);
    const int group_size = GROUP_M * p.tiles_n;
    const int first_m = (tile_id / group_size) * GROUP_M, in_group = tile_id % group_size;
    const int group_rows = min(p.tiles_m - first_m, GROUP_M);
    const int tile_m = first_m + in_group % group_rows, tile_n = in_group / group_rows;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(p.A + static_cast<size_t>(blockIdx.z) * p.a_batch), 0, static_cast<int>(static_cast<size_t>(M) * K * 4),
        0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(p.B), 0, static_cast<int>(static_cast<size_t>(K) * N * 4), 0x00020000);
    constexpr unsigned kOutside = 0x80000000u;

    // This wavefront's load instructions: A instructions wave, wave + WAVES, ..., then B instructions likewise.
    unsigned load_off[LOADS];     // per-lane byte offset at k-tile 0
    int load_lds[LOADS];          // LDS byte offset of the instruction's 1 KB within a stage (wavefront-uniform)
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        if (i < LOADS_A) {
            const int idx = wave + i * WAVES;
            load_lds[i] = idx * 1024;
            if (AT) {  // tile [16 k][BM]: lane covers floats idx*256 + lane*4 .. +3
                const int f = idx * 256 + lane * 4;
                const int k = f / BM, col = f % BM;
                load_off[i] = (m0 + col < M) ? (static_cast<unsigned>(k) * M + m0 + col) * 4u : kOutside;
            } else {   // tile [BM][16 k]: lane lands at row idx*16 + lane/4, chunk position lane%4
                const int row = idx * 16 + (lane >> 2);
                const int chunk = (lane & 3) ^ ((row >> 2) & 3);
                load_off[i] = (m0 + row < M) ? (static_cast<unsigned>(m0 + row) * K + chunk * 4) * 4u : kOutside;
            }
        } else {
            const int j = wave + (i - LOADS_A) * WAVES;
            load_lds[i] = A_BYTES + j * 1024;
            if (BT) {  // tile [BN][16 k]: lane lands at row j*16 + lane/4, chunk position lane%4
                const int row = j * 16 + (lane >> 2);
                const int chunk = (lane & 3) ^ ((row >> 2) & 3);
                load_off[i] = (n0 + row < N) ? (static_cast<unsigned>(n0 + row) * K + chunk * 4) * 4u : kOutside;
            } else {
                const int f = j * 256 + lane * 4;
                const int k = f / BN, col = f % BN;
                load_off[i] = (n0 + col < N) ? (static_cast<unsigned>(k) * N + n0 + col) * 4u : kOutside;
            }
        }
    }
    const unsigned a_step = AT ? static_cast<unsigned>(BK) * M * 4u : BK * 4u;  // bytes per k-tile
    const unsigned b_step = BT ? BK * 4u : static_cast<unsigned>(BK) * N * 4u;

    auto issue = [&](auto slot_tag, int t) {
        constexpr int SLOT = decltype(slot_tag)::value;
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            lds_void_ptr dst = (lds_void_ptr)(ring_lds + SLOT * STAGE + load_lds[i]);
            if (i < LOADS_A)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, load_off[i], t * a_step, 0, 0);
            else
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, load_off[i], t * b_step, 0, 0);
        }
    };

    // Per-lane fragment offsets within a stage.
    unsigned a_lane[BK / 8][TM], b_lane[BK / 8][TN];
#pragma unroll
    for (int kk = 0; kk < BK / 8; ++kk) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const int row = wm * WTM + tm * 32 + li;
            a_lane[kk][tm] = AT ? ((kk * 8 + lh * 4) * BM + row) * 4
                                : row * 64 + (((kk * 2 + lh) ^ ((row >> 2) & 3)) * 16);
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const int col = wn * WTN + tn * 32 + li;
            b_lane[kk][tn] = A_BYTES + (BT ? col * 64 + (((kk * 2 + lh) ^ ((col >> 2) & 3)) * 16)
                                           : ((kk * 8 + lh * 4) * BN + col) * 4);
        }
    }

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    auto compute = [&](auto slot_tag) {
        constexpr int SLOT = decltype(slot_tag)::value;
        const unsigned char *stage = ring_lds + SLOT * STAGE;
        float a[BK / 8][TM][4], b[BK / 8][TN][4];
#pragma unroll
        for (int kk = 0; kk < BK / 8; ++kk) {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                if (AT) {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        a[kk][tm][t] = *reinterpret_cast<const float *>(stage + a_lane[kk][tm] + t * BM * 4);
                } else {
                    const f32x4 v = *reinterpret_cast<const f32x4 *>(stage + a_lane[kk][tm]);
                    a[kk][tm][0] = v[0]; a[kk][tm][1] = v[1]; a[kk][tm][2] = v[2]; a[kk][tm][3] = v[3];
                }
            }
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
                if (BT) {
                    const f32x4 v = *reinterpret_cast<const f32x4 *>(stage + b_lane[kk][tn]);
                    b[kk][tn][0] = v[0]; b[kk][tn][1] = v[1]; b[kk][tn][2] = v[2]; b[kk][tn][3] = v[3];
                } else {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        b[kk][tn][t] = *reinterpret_cast<const float *>(stage + b_lane[kk][tn] + t * BN * 4);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(2);
#pragma unroll
        for (int kk = 0; kk < BK / 8; ++kk)
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn)
                        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kk][tm][t], b[kk][tn][t], acc[tm][tn], 0, 0, 0);
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
    };

    // k-tiles of this workgroup: all of them, or slice blockIdx.y of a k-sliced launch (first k-tile t0).
    const int slice_steps = p.slice_k / BK;
    const int t0 = __builtin_amdgcn_readfirstlane(static_cast<int>(blockIdx.y) * slice_steps);
    const int steps = p.slice_k ? min(K / BK - t0, slice_steps) : K / BK;
    if (steps > 0) issue(std::integral_constant<int, 0>{}, t0);
    if (steps > 1) issue(std::integral_constant<int, 1>{}, t0 + 1);
    // Drain the prologue once: loads still counted as outstanding at the loop header make the compiler's
    // wait-count insertion fall back to a full vmcnt(0) inside the loop.
    ST_F32_WAIT_VMCNT(0);
    auto step = [&](auto slot_tag, int t) {
        constexpr int SLOT = decltype(slot_tag)::value;
        // This wavefront's loads of k-tile t have landed once only those of k-tile t+1 are outstanding; the
        // barrier extends that to every wavefront and says that all are done reading the slot k-tile t+2
        // overwrites.  It is a bare s_barrier: __syncthreads() carries a release fence that makes the
        // compiler wait for every outstanding load, including the k-tile just requested.  No ordinary store
        // writes LDS in the loop, and a wavefront's reads of a slot have returned before its next barrier.
        if (t + 1 < steps) ST_F32_WAIT_VMCNT(LOADS);
        else ST_F32_WAIT_VMCNT(0);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (t + 2 < steps) issue(std::integral_constant<int, (SLOT + 2) % RING>{}, t0 + t + 2);
        compute(slot_tag);
    };
    int t = 0;
    for (; t + 3 <= steps; t += 3) {
        step(std::integral_constant<int, 0>{}, t);
        step(std::integral_constant<int, 1>{}, t + 1);
        step(std::integral_constant<int, 2>{}, t + 2);
    }
    if (t < steps) step(std::integral_constant<int, 0>{}, t);
    if (t + 1 < steps) step(std::integral_constant<int, 1>{}, t + 1);

    // scale 1.0f and the bias stand-in -0.0f leave every value as it is, so neither needs a branch.
    float *const C = p.C + static_cast<size_t>(blockIdx.y) * M * N + static_cast<size_t>(blockIdx.z) * p.c_batch;
    with_epilogue_ops(p.activation, p.residual != nullptr, [&](auto &&act, auto has_residual) {
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const int col = n0 + wn * WTN + tn * 32 + li;
            const bool col_ok = col < N;
            const float bias = (p.bias && col_ok) ? p.bias[col] : -0.0f;
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                const f32x16 tile = acc[tm][tn];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = m0 + wm * WTM + tm * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                    if (col_ok && row < M) {
                        const size_t idx = static_cast<size_t>(row) * N + col;
                        float value = tile[r] * p.scale + bias;
                        if constexpr (decltype(has_residual)::value) value += p.residual[idx];
                        C[idx] = act(value);
                    }
                }
            }
        }
    });
}

// (Plain kernels around the templated body: a kernel template whose body uses the LDS-load builtins loses
// its host-side launch stub with this compiler.)
__global__ __launch_bounds__(512) void gemm_f32_ring_128x128_kernel(GemmF32Args p) { gemm_f32_ring_body<128, 128, 4, 2, false, false>(p); }
__global__ __launch_bounds__(512) void gemm_f32_ring_128x128_at_kernel(GemmF32Args p) { gemm_f32_ring_body<128, 128, 4, 2, true, false>(p); }
__global__ __launch_bounds__(512) void gemm_f32_ring_128x128_bt_kernel(GemmF32Args p) { gemm_f32_ring_body<128, 128, 4, 2, false, true>(p); }
__global__ __launch_bounds__(256) void gemm_f32_ring_64x64_kernel(GemmF32Args p) { gemm_f32_ring_body<64, 64, 2, 2, false, false>(p); }
__global__ __launch_bounds__(256) void gemm_f32_ring_64x64_at_kernel(GemmF32Args p) { gemm_f32_ring_body<64, 64, 2, 2, true, false>(p); }
__global__ __launch_bounds__(256) void gemm_f32_ring_64x64_bt_kernel(GemmF32Args p) { gemm_f32_ring_body<64, 64, 2, 2, false, true>(p); }

// Small problems (fewer 64×64 tiles than compute units): 32×32 tiles, and the four wavefronts of a workgroup
// split K between them — wavefront w takes k-tiles w, w+4, w+8, ... through a ring of its own, so the loop has
// no barrier at all (a wavefront only waits for its own loads) — and add their partial tiles through LDS at the
// end.  Same direct-to-LDS staging and layouts as the ring kernel above.
__global__ __launch_bounds__(256) void gemm_f32_ring_32x32_splitk_kernel(GemmF32Args p)
{
    constexpr int BM = 32, BN = 32, BK = 16, RING = 3, LOADS = 4;
    constexpr int A_BYTES = BM * BK * 4, STAGE = A_BYTES + BK * BN * 4;
    constexpr int WAVE_BYTES = RING * STAGE;
    __shared__ __attribute__((aligned(16))) unsigned char lds[4 * WAVE_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int M = p.M, N = p.N, K = p.K;
    const int tile_m = blockIdx.x / p.tiles_n, tile_n = blockIdx.x % p.tiles_n;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(p.A), 0, static_cast<int>(static_cast<size_t>(M) * K * 4), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(p.B), 0, static_cast<int>(static_cast<size_t>(K) * N * 4), 0x00020000);
    constexpr unsigned kOutside = 0x80000000u;
    unsigned a_off[2], b_off[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int row = j * 16 + (lane >> 2);
        const int chunk = (lane & 3) ^ ((row >> 2) & 3);
        a_off[j] = (m0 + row < M) ? (static_cast<unsigned>(m0 + row) * K + chunk * 4) * 4u : kOutside;
        const int f = j * 256 + lane * 4;
        const int k = f / BN, col = f % BN;
        b_off[j] = (n0 + col < N) ? (static_cast<unsigned>(k) * N + n0 + col) * 4u : kOutside;
    }
    const unsigned b_step = static_cast<unsigned>(BK) * N * 4u;
    unsigned char *ring = lds + wave * WAVE_BYTES;

    auto issue = [&](auto slot_tag, int t) {  // t: global k-tile index
        constexpr int SLOT = decltype(slot_tag)::value;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_ptr)(ring + SLOT * STAGE + j * 1024), 16, a_off[j],
                                                     t * (BK * 4), 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_ptr)(ring + SLOT * STAGE + A_BYTES + j * 1024), 16,
                                                     b_off[j], t * b_step, 0, 0);
        }
    };
    unsigned a_lane[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) a_lane[kk] = li * 64 + (((kk * 2 + lh) ^ ((li >> 2) & 3)) * 16);
    const unsigned b_lane = A_BYTES + (lh * 4 * BN + li) * 4;

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    auto compute = [&](auto slot_tag) {
        constexpr int SLOT = decltype(slot_tag)::value;
        const unsigned char *stage = ring + SLOT * STAGE;
        f32x4 a[2];
        float b[2][4];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            a[kk] = *reinterpret_cast<const f32x4 *>(stage + a_lane[kk]);
#pragma unroll
            for (int t = 0; t < 4; ++t) b[kk][t] = *reinterpret_cast<const float *>(stage + b_lane + (kk * 8 + t) * BN * 4);
        }
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kk][t], b[kk][t], acc, 0, 0, 0);
    };

    // k-tiles of this workgroup: all of them, or slice blockIdx.y of a k-sliced launch.
    const int slice_steps = p.slice_k / BK;
    const int t0 = __builtin_amdgcn_readfirstlane(static_cast<int>(blockIdx.y) * slice_steps) + wave;
    const int steps = p.slice_k ? min(K / BK - static_cast<int>(blockIdx.y) * slice_steps, slice_steps) : K / BK;
    const int my_steps = steps > wave ? (steps - wave + 3) / 4 : 0;  // k-tiles t0, t0+4, ...
    if (my_steps > 0) issue(std::integral_constant<int, 0>{}, t0);
    if (my_steps > 1) issue(std::integral_constant<int, 1>{}, t0 + 4);
    ST_F32_WAIT_VMCNT(0);
    auto step = [&](auto slot_tag, int i) {
        constexpr int SLOT = decltype(slot_tag)::value;
        if (i + 1 < my_steps) ST_F32_WAIT_VMCNT(LOADS);
        else ST_F32_WAIT_VMCNT(0);
        asm volatile("" ::: "memory");
        // slot (i+2)%3 was last read by this same wavefront in step i-1, whose reads have returned
        if (i + 2 < my_steps) issue(std::integral_constant<int, (SLOT + 2) % RING>{}, t0 + 4 * (i + 2));
        compute(slot_tag);
    };
    int i = 0;
    for (; i + 3 <= my_steps; i += 3) {
        step(std::integral_constant<int, 0>{}, i);
        step(std::integral_constant<int, 1>{}, i + 1);
        step(std::integral_constant<int, 2>{}, i + 2);
    }
    if (i < my_steps) step(std::integral_constant<int, 0>{}, i);
    if (i + 1 < my_steps) step(std::integral_constant<int, 1>{}, i + 1);

    // Add the four partial tiles: each wavefront writes its 32×32 accumulators to LDS, then thread t finishes
    // row t/8, columns 4·(t%8) .. +3.
    __syncthreads();
    float *partial = reinterpret_cast<float *>(lds);  // [4][32][32 + 4]
    constexpr int P_STRIDE = BN + 4;
#pragma unroll
    for (int r = 0; r < 16; ++r)
        partial[(wave * 32 + (r >> 2) * 8 + lh * 4 + (r & 3)) * P_STRIDE + li] = acc[r];
    __syncthreads();
    const int row = tid >> 3, c4 = (tid & 7) * 4;
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const f32x4 v = *reinterpret_cast<const f32x4 *>(&partial[(w * 32 + row) * P_STRIDE + c4]);
        sum[0] += v[0]; sum[1] += v[1]; sum[2] += v[2]; sum[3] += v[3];
    }
    float *const C = p.C + static_cast<size_t>(blockIdx.y) * M * N;
    if (m0 + row < M) {
        with_epilogue_ops(p.activation, p.residual != nullptr, [&](auto &&act, auto has_residual) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int col = n0 + c4 + e;
                if (col >= N) continue;
                const size_t idx = static_cast<size_t>(m0 + row) * N + col;
                float value = sum[e] * p.scale + (p.bias ? p.bias[col] : -0.0f);
                if constexpr (decltype(has_residual)::value) value += p.residual[idx];
                C[idx] = act(value);
            }
        });
    }
}

hipError_t launch_splitk32(GemmF32Args args, hipStream_t stream, bool scratch_free)
{
    args.tiles_n = (args.N + 31) / 32;
    args.tiles_m = (args.M + 31) / 32;
    const size_t tiles = static_cast<size_t>(args.tiles_n) * static_cast<size_t>(args.tiles_m);
    auto launch = [&](const GemmF32Args &a, unsigned slices) {
        hipLaunchKernelGGL(gemm_f32_ring_32x32_splitk_kernel, dim3(static_cast<unsigned>(tiles), slices), dim3(256), 0, stream, a);
        return hipGetLastError();
    };
    // A long k over few tiles (64×64×100000, 256×256×16384) is cut over workgroups as well: 64 k-tiles per slice keep
    // 16 for each wavefront's ring.
    const size_t k_steps = static_cast<size_t>(args.K) / 16;
    const size_t slices = scratch_free ? choose_k_slices(args.M, args.N, args.K, tiles, k_steps, 64) : 1;
    if (slices > 1) return launch_k_sliced(args, slices, k_steps, 16, stream, launch);
    return launch(args, 1);
}

hipError_t launch_ring(GemmF32Args args, bool lhs_transposed, bool rhs_packed, bool big, hipStream_t stream, bool scratch_free,
                       unsigned batch = 1)
{
    const int bm = big ? 128 : 64, bn = big ? 128 : 64;
    args.tiles_n = (args.N + bn - 1) / bn;
    args.tiles_m = (args.M + bm - 1) / bm;
    const size_t tiles = static_cast<size_t>(args.tiles_n) * static_cast<size_t>(args.tiles_m);
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    const size_t lds_bytes = 3 * static_cast<size_t>(bm + bn) * 16 * 4;
    auto kernel = big ? (rhs_packed ? gemm_f32_ring_128x128_bt_kernel
                                    : lhs_transposed ? gemm_f32_ring_128x128_at_kernel : gemm_f32_ring_128x128_kernel)
                      : (rhs_packed ? gemm_f32_ring_64x64_bt_kernel
                                    : lhs_transposed ? gemm_f32_ring_64x64_at_kernel : gemm_f32_ring_64x64_kernel);
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    auto launch = [&](const GemmF32Args &a, unsigned slices) {
        hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(tiles), slices, batch), dim3(big ? 512 : 256), lds_bytes, stream, a);
        return hipGetLastError();
    };
    // Few tiles and a long k (a weight gradient Xᵀ·dY of a small layer over many rows): cut along k over workgroups.
    const size_t k_steps = static_cast<size_t>(args.K) / 16;
    // (768 of the 64×64 workgroups are resident at a time, and with fewer than half of that a 16-wide k-tile costs a
    // workgroup half a microsecond of load latency: 1576×768×3072, 300 tiles of 192 k-tiles, took 102 µs.)
    const size_t slices = big || !scratch_free ? 1 : choose_k_slices(args.M, args.N, args.K, tiles, k_steps, 16, 384, 768);
    if (slices > 1) return launch_k_sliced(args, slices, k_steps, 16, stream, launch);
    return launch(args, 1);
}


// out(cols×rows) = in(rows×cols)ᵀ through a 32×33 LDS tile (PackedB::from_row_major, pure.rs:1299-1316, and back).
__global__ __launch_bounds__(256) void transpose_f32_kernel(int rows, int cols, const float *in, float *out)
{
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 × 8
    const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = r0 + ty + 8 * i, c = c0 + tx;
        if (r < rows && c < cols) tile[ty + 8 * i][tx] = in[static_cast<size_t>(r) * cols + c];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = c0 + ty + 8 * i, r = r0 + tx;
        if (r < rows && c < cols) out[static_cast<size_t>(c) * rows + r] = tile[tx][ty + 8 * i];
    }
}

// Copies rows × cols f32 matrices into rows_pad × cols_pad ones, zeros in the new rows and columns: two matrices (the
// operands of a product) in one launch, the first `first_blocks` workgroups on the first.  A thread moves four
// adjacent values of one output row (16-byte accesses at any alignment).
struct PadJobF32 {
    const float *in;
    float *out;
    unsigned rows, cols, rows_pad, cols_pad;
};

__global__ __launch_bounds__(256) void pad_f32_pair_kernel(PadJobF32 first, PadJobF32 second, unsigned first_blocks)
{
    typedef float pad_f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
    const bool is_first = blockIdx.x < first_blocks;
    const PadJobF32 &job = is_first ? first : second;
    const unsigned chunks = (job.cols_pad + 3) / 4;
    const unsigned idx = (blockIdx.x - (is_first ? 0u : first_blocks)) * 256u + threadIdx.x;  // below 2^29: the copies are below 2 GiB
    const unsigned r = idx / chunks;
    const unsigned c0 = (idx - r * chunks) * 4;
    if (r >= job.rows_pad) return;
    float *dst = job.out + static_cast<size_t>(r) * job.cols_pad + c0;
    const float *src = job.in + static_cast<size_t>(r) * job.cols + c0;
    if (r < job.rows && c0 + 4 <= job.cols) {
        *reinterpret_cast<pad_f32x4_a4 *>(dst) = *reinterpret_cast<const pad_f32x4_a4 *>(src);
        return;
    }
#pragma unroll
    for (unsigned e = 0; e < 4; ++e) {
        const unsigned c = c0 + e;
        if (c < job.cols_pad) dst[e] = (r < job.rows && c < job.cols) ? src[e] : 0.0f;
    }
}

hipError_t launch_pad_f32_pair(const PadJobF32 &first, const PadJobF32 &second, hipStream_t stream)
{
    auto blocks = [](const PadJobF32 &job) {
        return static_cast<unsigned>((static_cast<size_t>(job.rows_pad) * ((job.cols_pad + 3) / 4) + 255) / 256);
    };
    const unsigned first_blocks = blocks(first), all = first_blocks + blocks(second);
    if (all == 0) return hipSuccess;
    hipLaunchKernelGGL(pad_f32_pair_kernel, dim3(all), dim3(256), 0, stream, first, second, first_blocks);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_gemm_f32(size_t m, size_t n, size_t k, bool lhs_transposed, const float *lhs,
                           const float *rhs, float *out, const GemmEpilogue &epilogue, hipStream_t stream, bool scratch_free)
{
    if (m == 0 || n == 0) return hipSuccess;
    if (!lhs_transposed && gemv_f32_applies(m, n, k, lhs, rhs)) return launch_gemv_f32(m, n, k, lhs, rhs, out, epilogue, stream);
    if (lhs_transposed && scratch_free && gemv_t_f32_applies(m, n, k)) return launch_gemv_t_f32(m, n, k, lhs, rhs, out, epilogue, stream);
    // A k that is not a multiple of 4 (a vocabulary of 50257 as the reduction of a backward product): the rows of A start
    // at odd addresses, which the direct-to-LDS kernels do not take, and the general kernel runs at about 0.6 of their
    // speed (1024×1024×4099: 140 µs against 80 µs at 4096).  Where the product is large against its operands, copies
    // of A and B zero-padded along k to a multiple of 16 (exact: the new terms are 0·0) go into the stream's second
    // scratch buffer, one launch for both, and the product runs on them.
    // (Only where the copies then take the fast kernels: B's rows, and A's when it is stored k×m, must be 16-byte aligned.)
    if (k % 4 != 0 && k > 64 && m >= 128 && n >= 128 && n % 4 == 0 && (!lhs_transposed || m % 4 == 0) && scratch_free &&
        2.0 * m * n * k >= 2e9 &&
        m * (k + 16) * sizeof(float) < (1ull << 31) && (k + 16) * n * sizeof(float) < (1ull << 31)) {
        const size_t k_pad = (k + 15) / 16 * 16;
        const size_t a_bytes = (m * k_pad * sizeof(float) + 255) & ~static_cast<size_t>(255);
        void *copies = nullptr;
        hipError_t rc = stream_workspace_slot(stream, 1, a_bytes + k_pad * n * sizeof(float), &copies);
        if (rc != hipSuccess) return rc;
        float *a_pad = static_cast<float *>(copies);
        float *b_pad = reinterpret_cast<float *>(static_cast<unsigned char *>(copies) + a_bytes);
        auto job = [](size_t rows, size_t cols, size_t rows_pad, size_t cols_pad, const float *in, float *to) {
            return PadJobF32{in, to, static_cast<unsigned>(rows), static_cast<unsigned>(cols), static_cast<unsigned>(rows_pad),
                             static_cast<unsigned>(cols_pad)};
        };
        rc = launch_pad_f32_pair(lhs_transposed ? job(k, m, k_pad, m, lhs, a_pad) : job(m, k, m, k_pad, lhs, a_pad),
                                 job(k, n, k_pad, n, rhs, b_pad), stream);
        if (rc != hipSuccess) return rc;
        return launch_gemm_f32(m, n, k_pad, lhs_transposed, a_pad, b_pad, out, epilogue, stream, true);
    }
    // An A of 2 GiB or more (the direct-to-LDS kernels address their operands through 32-bit byte offsets): row blocks
    // of A are independent products, so the launch is cut into blocks that fit and each takes the fast path.
    if (!lhs_transposed && m * k * sizeof(float) >= (1ull << 31) && gemm_row_block(k, sizeof(float)) > 0) {
        const size_t block = gemm_row_block(k, sizeof(float));
        for (size_t row = 0; row < m; row += block) {
            const size_t rows = std::min(block, m - row);
            GemmEpilogue part = epilogue;
            if (part.residual) part.residual += row * n;
            const hipError_t rc = launch_gemm_f32(rows, n, k, false, lhs + row * k, rhs, out + row * n, part, stream, scratch_free);
            if (rc != hipSuccess) return rc;
        }
        return hipSuccess;
    }
    GemmF32Args args;
    args.A = lhs;
    args.B = rhs;
    args.C = out;
    args.bias = epilogue.bias;
    args.residual = epilogue.residual;
    args.M = static_cast<int>(m);
    args.N = static_cast<int>(n);
    args.K = static_cast<int>(k);
    args.scale = epilogue.scale;
    args.activation = epilogue.activation;
    // 128-bit global loads need every row start 16-byte aligned.
    const size_t lhs_ld = lhs_transposed ? m : k;
    const bool vec = (lhs_ld % 4 == 0) && (n % 4 == 0) && aligned16(lhs) && aligned16(rhs);
    // 256×256 tiles (16 wavefronts of 64×64) once they give every compute unit a full tile without padding
    // waste; otherwise 64×64 tiles (4 wavefronts of 32×32), which spread small and narrow problems over the chip.
    // The ring kernel wants whole 16-wide k-tiles, 16-byte aligned rows and 32-bit byte offsets.
    const bool ring_ok = vec && k >= 16 && k % 16 == 0 && m * k * 4 < (1ull << 31) && k * n * 4 < (1ull << 31) &&
                         (!lhs_transposed || m % 4 == 0);
    const size_t big_tiles = ((m + 255) / 256) * ((n + 255) / 256);
    const bool little_padding = (m % 256 == 0 || m >= 2048) && (n % 256 == 0 || n >= 2048);
    // ... and in rounds of 256 that are mostly full: 300 tiles are two rounds for the work of 1.17 (6304×3072×768: 399 µs
    // on these tiles, 74 TFLOP/s; the ring kernel's 128×128 tiles, 768 resident, quantise finer).
    const double rounds_fill = static_cast<double>(big_tiles) / static_cast<double>((big_tiles + 255) / 256 * 256);
    if (big_tiles >= 256 && little_padding && (rounds_fill >= 0.8 || !ring_ok))
        return launch_tile<256, 256, 4, 4>(args, lhs_transposed, vec, stream);
    if (ring_ok) {
        // 128×128 tiles (three workgroups per compute unit, 768 at a time) when they come in full rounds or many
        // rounds; 64×64 tiles otherwise, which spread small problems and leave a shorter tail.
        const size_t tiles128 = ((m + 127) / 128) * ((n + 127) / 128);
        const bool big = tiles128 >= 512 && (tiles128 >= 3072 || tiles128 % 768 == 0 || tiles128 % 768 >= 384);
        // Fewer 64×64 tiles than two per compute unit: 32×32 tiles with K split over the wavefronts of a workgroup.
        const size_t tiles64 = ((m + 63) / 64) * ((n + 63) / 64);
        // (Up to 448: with one or two 64×64 workgroups on a compute unit a SIMD holds a single wavefront and its
        // fragment reads and MFMAs do not overlap — 1576×768×768, 300 tiles: 28.4 µs on them, 20.2 µs on 32×32 tiles;
        // from 512 tiles on the larger tiles are ahead again: 1024×2048×512 21.7 against 24.5 µs.)
        if (!lhs_transposed && tiles64 <= 448 && k >= 128) return launch_splitk32(args, stream, scratch_free);
        return launch_ring(args, lhs_transposed, false, big, stream, scratch_free);
    }
    // Shapes the ring kernels do not take.  Few tiles and a long k (a matrix-vector product, n < 4, is the common case):
    // k-sliced, so that the whole chip streams A and B.
    const size_t tiles64 = ((m + 63) / 64) * ((n + 63) / 64), k_steps = (k + kBK - 1) / kBK;
    const size_t slices = scratch_free ? choose_k_slices(m, n, k, tiles64, k_steps, 16) : 1;
    if (slices > 1)
        return launch_k_sliced(args, slices, k_steps, kBK, stream, [&](const GemmF32Args &a, unsigned count) {
            return launch_tile<64, 64, 2, 2>(a, lhs_transposed, vec, stream, count);
        });
    return launch_tile<64, 64, 2, 2>(args, lhs_transposed, vec, stream);
}

hipError_t launch_gemm_f32_batched(size_t batch, size_t m, size_t n, size_t k, bool lhs_transposed, const float *lhs,
                                   size_t lhs_stride, const float *rhs, float *out, size_t out_stride, hipStream_t stream)
{
    if (batch == 0 || m == 0 || n == 0) return hipSuccess;
    GemmF32Args args;
    args.A = lhs;
    args.B = rhs;
    args.C = out;
    args.bias = nullptr;
    args.residual = nullptr;
    args.M = static_cast<int>(m);
    args.N = static_cast<int>(n);
    args.K = static_cast<int>(k);
    args.scale = 1.0f;
    args.activation = ST_HIP_ACT_NONE;
    args.a_batch = lhs_stride;
    args.c_batch = out_stride;
    const size_t lhs_ld = lhs_transposed ? m : k;
    const bool vec = (lhs_ld % 4 == 0) && (n % 4 == 0) && aligned16(lhs) && aligned16(rhs) && lhs_stride % 4 == 0;
    const bool ring_ok = vec && k >= 16 && k % 16 == 0 && m * k * 4 < (1ull << 31) && k * n * 4 < (1ull << 31) &&
                         (!lhs_transposed || m % 4 == 0);
    const size_t tiles128 = ((m + 127) / 128) * ((n + 127) / 128) * batch;
    const bool big = tiles128 >= 512 && (tiles128 >= 3072 || tiles128 % 768 == 0 || tiles128 % 768 >= 384);
    // The grid's third dimension holds at most 65535 products.
    for (size_t first = 0; first < batch; first += 65535) {
        const unsigned count = static_cast<unsigned>(std::min<size_t>(65535, batch - first));
        args.A = lhs + first * lhs_stride;
        args.C = out + first * out_stride;
        const hipError_t rc = ring_ok ? launch_ring(args, lhs_transposed, false, big, stream, /*scratch_free=*/false, count)
                                      : launch_tile<64, 64, 2, 2>(args, lhs_transposed, vec, stream, 1, count);
        if (rc != hipSuccess) return rc;
    }
    return hipSuccess;
}

hipError_t launch_transpose_f32(size_t rows, size_t cols, const float *in, float *out, hipStream_t stream)
{
    if (rows == 0 || cols == 0) return hipSuccess;
    const dim3 grid(static_cast<unsigned>((cols + 31) / 32), static_cast<unsigned>((rows + 31) / 32));
    hipLaunchKernelGGL(transpose_f32_kernel, grid, dim3(256), 0, stream, static_cast<int>(rows), static_cast<int>(cols), in,
                       out);
    return hipGetLastError();
}

hipError_t launch_gemm_f32_packed(size_t m, size_t n, size_t k, const float *lhs, const float *packed_rhs, float *out,
                                  const GemmEpilogue &epilogue, hipStream_t stream)
{
    if (m == 0 || n == 0) return hipSuccess;
    const bool ring_ok = k >= 16 && k % 16 == 0 && aligned16(lhs) && aligned16(packed_rhs) && m * k * 4 < (1ull << 31) &&
                         k * n * 4 < (1ull << 31);
    if (!ring_ok) {
        // Ragged k: unpack into the stream's workspace and take the general path.
        void *workspace = nullptr;
        hipError_t rc = stream_workspace(stream, k * n * sizeof(float), &workspace);
        if (rc != hipSuccess) return rc;
        rc = launch_transpose_f32(n, k, packed_rhs, static_cast<float *>(workspace), stream);
        if (rc != hipSuccess) return rc;
        return launch_gemm_f32(m, n, k, false, lhs, static_cast<const float *>(workspace), out, epilogue, stream,
                               /*scratch_free=*/false);  // the scratch buffer holds the unpacked B
    }
    GemmF32Args args;
    args.A = lhs;
    args.B = packed_rhs;
    args.C = out;
    args.bias = epilogue.bias;
    args.residual = epilogue.residual;
    args.M = static_cast<int>(m);
    args.N = static_cast<int>(n);
    args.K = static_cast<int>(k);
    args.scale = epilogue.scale;
    args.activation = epilogue.activation;
    const size_t tiles128 = ((m + 127) / 128) * ((n + 127) / 128);
    const bool big = tiles128 >= 512 && (tiles128 >= 3072 || tiles128 % 768 == 0 || tiles128 % 768 >= 384);
    return launch_ring(args, false, true, big, stream, true);
}

}  // namespace sthip
