// bf16 GEMM with f32 accumulation on the gfx950 matrix cores (v_mfma_f32_32x32x16_bf16), with the
// fused bias / residual / activation epilogue and f32 and/or bf16 output.
//
// The reference has no bf16 path (docs/backend_matrix.md lists it as roadmap); the operator contract is
// the f32 one of crates/st-backend-hip/src/lib.rs:607-720 with bf16 operand storage.
//
// Tiling: a 256-thread workgroup (4 wavefronts, 2×2) owns a BM×BN tile of C.  A (row-major, k
// contiguous) is staged as As[BM][BK+8]; B (row-major, n contiguous) is staged UNTRANSPOSED as
// Bs[BK][BN+32] and read with the gfx950 LDS transpose load (ds_read_b64_tr_b16), which hands lane
// (column j, k-half h) the four k-consecutive values of column j out of a 4×16 block whose rows are
// stored n-contiguous.  Two such reads make the 8-value B operand of the 32x32x16 MFMA.
//
// MFMA operand layout (32x32x16): lane l supplies A[l%32][8*(l/32) .. +7] and B[8*(l/32) .. +7][l%32];
// accumulator register r of lane l is C[(r/4)*8 + (l/32)*4 + r%4][l%32].
#include "device_math.h"
#include "kernels.h"

namespace sthip {

namespace {

struct GemmBf16Args {
    const uint16_t *A;
    const uint16_t *B;
    float *C32;
    uint16_t *C16;
    const float *bias;
    const float *residual;
    int M, N, K;
    int tiles_m, tiles_n;
    int swizzle;  // 1: remap workgroup ids so each XCD (id % 8) works on a compact block of tiles
    float scale;
    int activation;
};

typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;

template <bool VEC>
__device__ __forceinline__ uint4 load_row8(const uint16_t *base, size_t row_offset, int col, int col_limit,
                                           bool row_valid)
{
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (!row_valid) return v;
    const uint16_t *src = base + row_offset + col;
    if (VEC) {
        if (col < col_limit) v = *reinterpret_cast<const uint4 *>(src);
    } else {
        uint16_t e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) e[i] = (col + i < col_limit) ? src[i] : static_cast<uint16_t>(0);
        v.x = e[0] | (static_cast<uint32_t>(e[1]) << 16);
        v.y = e[2] | (static_cast<uint32_t>(e[3]) << 16);
        v.z = e[4] | (static_cast<uint32_t>(e[5]) << 16);
        v.w = e[6] | (static_cast<uint32_t>(e[7]) << 16);
    }
    return v;
}

template <int BM, int BN, int BK, bool VEC>
__global__ __launch_bounds__(256) void gemm_bf16_kernel(GemmBf16Args p)
{
    constexpr int WTM = BM / 2, WTN = BN / 2;  // wavefront tile
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int A_STRIDE = BK + 8;   // bf16 elements; keeps 128-bit row reads conflict-light
    constexpr int B_STRIDE = BN + 32;  // 64 B skew per k-row spreads the transpose reads over banks
    constexpr int A_CHUNKS = BM * BK / 8 / 256;
    constexpr int B_CHUNKS = BK * BN / 8 / 256;
    static_assert(A_CHUNKS >= 1 && B_CHUNKS >= 1, "tile too small for 256 threads");
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
    uint16_t *As = lds;                         // [2][BM * A_STRIDE]
    uint16_t *Bs = lds + 2 * BM * A_STRIDE;     // [2][BK * B_STRIDE]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, lh = lane >> 5;
    const int M = p.M, N = p.N, K = p.K;

    int logical = blockIdx.x;
    if (p.swizzle) {
        const int per_xcd = gridDim.x >> 3;
        logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    }
    // Grouped ordering: consecutive ids walk 4 tile-rows before moving along N, so the 32 tiles an XCD
    // holds at a time share 4 row panels of A and 8 column panels of B in its L2.
    constexpr int GROUP_M = 4;
    const int width = GROUP_M * p.tiles_n;
    const int group = logical / width;
    const int first_m = group * GROUP_M;
    const int group_size = min(p.tiles_m - first_m, GROUP_M);
    const int tile_m = first_m + (logical % width) % group_size;
    const int tile_n = (logical % width) / group_size;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    uint4 ra[A_CHUNKS], rb[B_CHUNKS];

    auto load_global = [&](int k0) {
#pragma unroll
        for (int r = 0; r < A_CHUNKS; ++r) {
            const int f = tid + 256 * r;
            const int row = f / (BK / 8), c8 = (f % (BK / 8)) * 8;
            ra[r] = load_row8<VEC>(p.A, static_cast<size_t>(m0 + row) * K, k0 + c8, K, m0 + row < M);
        }
#pragma unroll
        for (int r = 0; r < B_CHUNKS; ++r) {
            const int f = tid + 256 * r;
            const int krow = f / (BN / 8), c8 = (f % (BN / 8)) * 8;
            rb[r] = load_row8<VEC>(p.B, static_cast<size_t>(k0 + krow) * N, n0 + c8, N, k0 + krow < K);
        }
    };
    auto store_lds = [&](int stage) {
        uint16_t *as = As + stage * BM * A_STRIDE;
        uint16_t *bs = Bs + stage * BK * B_STRIDE;
#pragma unroll
        for (int r = 0; r < A_CHUNKS; ++r) {
            const int f = tid + 256 * r;
            const int row = f / (BK / 8), c8 = (f % (BK / 8)) * 8;
            *reinterpret_cast<uint4 *>(&as[row * A_STRIDE + c8]) = ra[r];
        }
#pragma unroll
        for (int r = 0; r < B_CHUNKS; ++r) {
            const int f = tid + 256 * r;
            const int krow = f / (BN / 8), c8 = (f % (BN / 8)) * 8;
            *reinterpret_cast<uint4 *>(&bs[krow * B_STRIDE + c8]) = rb[r];
        }
    };
    // Transpose-read lane roles: within each 16-lane group, lane i16 supplies the address of row
    // i16/4 (k) and 4-column chunk i16%4, and receives column i16 of that 4×16 block.
    const int i16 = lane & 15;
    const int c16 = (lane >> 4) & 1;
    const int b_row = lh * 8 + (i16 >> 2);
    const int b_col = wn * WTN + c16 * 16 + (i16 & 3) * 4;
    auto compute = [&](int stage) {
        const uint16_t *as = As + stage * BM * A_STRIDE;
        const uint16_t *bs = Bs + stage * BK * B_STRIDE;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            bf16x8 a[TM], b[TN];
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                const int row = wm * WTM + tm * 32 + li;
                a[tm] = *reinterpret_cast<const bf16x8 *>(&as[row * A_STRIDE + kk * 16 + lh * 8]);
            }
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
                const uint16_t *src = &bs[(kk * 16 + b_row) * B_STRIDE + b_col + tn * 32];
                union {
                    s16x4 half[2];
                    bf16x8 full;
                } frag;
                frag.half[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(src));
                frag.half[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(src + 4 * B_STRIDE));
                b[tn] = frag.full;
            }
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < TN; ++tn)
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[tm], b[tn], acc[tm][tn], 0, 0, 0);
        }
    };

    const int steps = (K + BK - 1) / BK;
    if (steps > 0) {
        load_global(0);
        store_lds(0);
    }
    __syncthreads();
    for (int t = 0; t < steps; ++t) {
        const bool more = t + 1 < steps;
        if (more) load_global((t + 1) * BK);
        compute(t & 1);
        if (more) store_lds((t + 1) & 1);
        __syncthreads();
    }

    const bool scaled = p.scale != 1.0f;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        const int col = n0 + wn * WTN + tn * 32 + li;
        if (col >= N) continue;
        const float bias = p.bias ? p.bias[col] : 0.0f;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm * WTM + tm * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                if (row >= M) continue;
                const size_t idx = static_cast<size_t>(row) * N + col;
                float value = acc[tm][tn][r];
                if (scaled) value *= p.scale;
                if (p.bias) value += bias;
                if (p.residual) value += p.residual[idx];
                value = apply_activation(value, p.activation);
                if (p.C32) p.C32[idx] = value;
                if (p.C16) p.C16[idx] = f32_to_bf16_rne(value);
            }
        }
    }
}

template <int BM, int BN, int BK>
hipError_t launch_tile(GemmBf16Args args, bool vec, hipStream_t stream)
{
    args.tiles_m = (args.M + BM - 1) / BM;
    args.tiles_n = (args.N + BN - 1) / BN;
    const size_t tiles = static_cast<size_t>(args.tiles_m) * static_cast<size_t>(args.tiles_n);
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    args.swizzle = (tiles % 8 == 0) ? 1 : 0;
    constexpr size_t lds_bytes = 2 * (static_cast<size_t>(BM) * (BK + 8) + static_cast<size_t>(BK) * (BN + 32)) * 2;
    const dim3 grid(static_cast<unsigned>(tiles));
    const dim3 block(256);
    hipError_t rc;
    if (vec) {
        auto kernel = gemm_bf16_kernel<BM, BN, BK, true>;
        rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                 static_cast<int>(lds_bytes));
        if (rc != hipSuccess) return rc;
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, args);
    } else {
        auto kernel = gemm_bf16_kernel<BM, BN, BK, false>;
        rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                 static_cast<int>(lds_bytes));
        if (rc != hipSuccess) return rc;
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, args);
    }
    return hipGetLastError();
}

bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

}  // namespace

hipError_t launch_gemm_bf16(size_t m, size_t n, size_t k, const uint16_t *lhs, const uint16_t *rhs,
                            float *out_f32, uint16_t *out_bf16, const GemmEpilogue &epilogue,
                            hipStream_t stream)
{
    if (m == 0 || n == 0) return hipSuccess;
    GemmBf16Args args;
    args.A = lhs;
    args.B = rhs;
    args.C32 = out_f32;
    args.C16 = out_bf16;
    args.bias = epilogue.bias;
    args.residual = epilogue.residual;
    args.M = static_cast<int>(m);
    args.N = static_cast<int>(n);
    args.K = static_cast<int>(k);
    args.tiles_m = args.tiles_n = 0;
    args.swizzle = 0;
    args.scale = epilogue.scale;
    args.activation = epilogue.activation;
    const bool vec = (k % 8 == 0) && (n % 8 == 0) && aligned16(lhs) && aligned16(rhs);
    const size_t big_tiles = ((m + 255) / 256) * ((n + 255) / 256);
    if (big_tiles >= 192) return launch_tile<256, 256, 64>(args, vec, stream);
    return launch_tile<128, 128, 32>(args, vec, stream);
}

}  // namespace sthip
