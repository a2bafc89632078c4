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
#include <algorithm>
#include <mutex>
#include <type_traits>
#include <vector>

#include "device_math.h"
#include "kernels.h"

namespace sthip {

namespace {

// Geometry of a convolution run as a GEMM with M = c_out, N = batch·oh·ow output pixels and K = kh·kw·c_pad, k ordered
// (ky, kx, channel): a 64-wide k-tile is one tap and 64 consecutive channels, i.e. one contiguous 128-byte piece of the
// channels-last image copy for every output pixel.
struct ConvBf16Geometry {
    int ohow, ow;          // output plane
    int hp, wp, c_pad;     // padded image copy: hp × wp positions of c_pad channels (a multiple of 64)
    int stride_h, stride_w, dil_h, dil_w;
    int kw;                // taps per kernel row
    int c_blocks;          // c_pad / 64: k-tiles per tap
    int c_out;
    unsigned image_bytes;  // bytes of the whole padded copy (the buffer range of operand B)
};

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
    // Split-k form of the 256-row kernels (launches of few tiles with a long k): workgroup (tile, split) covers
    // tiles_per_split k-tiles and leaves its raw sums in partial[split][M][N]; gemm_bf16_skinny_reduce_kernel adds the
    // splits in order and applies the epilogue.
    int k_splits = 1;
    int tiles_per_split = 0;
    float *partial = nullptr;
    // Convolution form of the packed kernels (CONV = true): A is the weight matrix re-laid as (c_out, kh·kw·c_pad), B the
    // zero-padded channels-last copy of the images, addressed per output pixel — see conv_bf16 below.
    ConvBf16Geometry conv = {};
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
    } else if (col + 8 <= col_limit) {
        // Eight values inside the row at any 2-byte alignment: still one 16-byte load (global memory takes wide
        // accesses at any alignment; the type says so, and the compiler keeps the single instruction).
        typedef uint32_t u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
        const u32x4_a2 w = *reinterpret_cast<const u32x4_a2 *>(src);
        v = make_uint4(w[0], w[1], w[2], w[3]);
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
    const int M = p.M, N = p.N;
    // This workgroup's k range [k_lo, K): slice blockIdx.y of a k-sliced launch (few tiles, long k), whose raw sums go
    // to plane blockIdx.y of C32 (the launch passes the workspace of partial planes as C32 and no epilogue);
    // K below is the END of the range, p.K stays the row stride of A.
    const int k_lo = static_cast<int>(blockIdx.y) * p.tiles_per_split * BK;
    const int K = p.k_splits > 1 ? min(p.K, k_lo + p.tiles_per_split * BK) : p.K;
    float *const C32 = p.C32 ? p.C32 + static_cast<size_t>(blockIdx.y) * M * N : nullptr;

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
            acc[a][b] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    uint4 ra[A_CHUNKS], rb[B_CHUNKS];

    auto load_global = [&](int k0) {
#pragma unroll
        for (int r = 0; r < A_CHUNKS; ++r) {
            const int f = tid + 256 * r;
            const int row = f / (BK / 8), c8 = (f % (BK / 8)) * 8;
            ra[r] = load_row8<VEC>(p.A, static_cast<size_t>(m0 + row) * p.K, k0 + c8, K, m0 + row < M);
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
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(src));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(src + 4 * B_STRIDE));
                typedef short s16x8 __attribute__((ext_vector_type(8)));
                const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                b[tn] = __builtin_bit_cast(bf16x8, both);
            }
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < TN; ++tn)
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[tm], b[tn], acc[tm][tn], 0, 0, 0);
        }
    };

    const int steps = (K - k_lo + BK - 1) / BK;
    if (steps > 0) {
        load_global(k_lo);
        store_lds(0);
    }
    __syncthreads();
    for (int t = 0; t < steps; ++t) {
        const bool more = t + 1 < steps;
        if (more) load_global(k_lo + (t + 1) * BK);
        compute(t & 1);
        if (more) store_lds((t + 1) & 1);
        __syncthreads();
    }

    // Epilogue.  The loops carry no early exits so that they unroll completely and the accumulators
    // stay in registers.
    const bool scaled = p.scale != 1.0f;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        const int col = n0 + wn * WTN + tn * 32 + li;
        const bool col_ok = col < N;
        const float bias = (p.bias && col_ok) ? p.bias[col] : 0.0f;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const f32x16 tile = acc[tm][tn];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm * WTM + tm * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                if (col_ok && row < M) {
                    const size_t idx = static_cast<size_t>(row) * N + col;
                    float value = tile[r];
                    if (scaled) value *= p.scale;
                    value += bias;
                    if (p.residual) value += p.residual[idx];
                    value = apply_activation(value, p.activation);
                    if (C32) C32[idx] = value;
                    if (p.C16) p.C16[idx] = f32_to_bf16_rne(value);
                }
            }
        }
    }
}


// -------------------------------------------------------------------------------------------------
// Large-problem kernels: 256×256×64 (or 256×128×64) tiles, eight wavefronts (two per SIMD, 64 × BN/2 of C each), K a
// multiple of 64, N a multiple of 128 (M may be ragged: rows past the end read as zero through the buffer
// descriptor's range check and are never stored).  Two forms, by the layout of B: packed (n×k) and row-major (k×n).
//
// LDS is the scarce resource (per k-tile a compute unit writes 64 KB and reads 192 KB of it while the matrix pipes
// need 2048 cycles; measured rates: 160 B/clk for 128-bit reads, 70 B/clk for 128-bit writes, 120 B/clk for a 2:1
// mix), so both operands are laid out for 128-bit, conflict-free reads and neither is padded:
//   * every operand row holds the tile's 64 k-values (128 B = 8 chunks of 16 B); chunk q of row r is
//     stored at chunk position q ^ swz(r), swz(r) = ((r >> 1) ^ (r >> 4)) & 7, which spreads the 16 rows
//     a 128-bit read touches per cycle, and the rows the B writes touch, over all banks;
//   * a k-contiguous operand (A; packed B) goes from global memory straight into LDS with buffer_load ... lds;
//     the swizzle is applied by choosing which 16 bytes each lane fetches.  A has three stages, B two;
//   * a row-major B is transposed in registers (v_perm_b32) and stored as rows of Bᵀ, so its fragments are
//     128-bit reads too (the LDS transpose read, ds_read_b64_tr_b16, moves a third of the bytes per cycle).
// Fragment reads run one 16-wide k sub-step ahead of the MFMAs and cross the tile boundary; there is one
// barrier per k-tile.  The epilogue goes through LDS (each wavefront owns a 32-row f32 strip) so that
// bias/residual loads and the stores are 128-bit and row-contiguous.
// -------------------------------------------------------------------------------------------------
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void *lds_void_ptr;

// s_waitcnt vmcnt(n) only (expcnt and lgkmcnt left at their maxima), gfx9 encoding.
#define ST_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (7 << 4) | (15 << 8) | ((((n) >> 4) & 3) << 14))

// Epilogue of the 256-row kernels.  The main loops form the product transposed (the MFMA's first operand is the Bᵀ
// fragment), so accumulator register 4g + j of lane (li, lh) in tile (tm, tn) is
//     C[row_first + 32·tm + li][col_base + 32·tn + 8g + 4·lh + j]:
// four neighbouring columns of one row, i.e. one 128-bit (f32) or 64-bit (bf16) LDS write.  Every wavefront sends its
// accumulators through a strip of LDS of its own and reads them back row-contiguous, so that the global stores (and
// the residual loads) are 128-bit and cover whole 256- or 512-byte row segments.
//   * bf16 is the only output and there is no residual: scale, bias and activation are applied in the accumulator
//     layout, the values are rounded to bf16 first and all 32·TM rows go through LDS in one pass (row = WTN·2 bytes,
//     unpadded; the 8-byte chunk q of row r sits at chunk q ^ swz(r), which spreads the 32 rows a write instruction
//     touches, and the rows a read instruction touches, over all banks);
//   * otherwise: f32 strips of 32 rows (row stride WTN + 4 floats), bias / residual / activation after the read-back.
// `lds`: start of the workgroup's LDS (the operand stages are dead by now); `wave`: this wavefront's index.
// Everything the epilogue decides per launch (activation, bias, residual) is a template parameter of the bodies below
// and is dispatched once per wavefront: with those decisions made per element the epilogue compiled to several
// hundred basic blocks whose loads, conversions and stores could not be scheduled across each other.
template <int ACT>
__device__ __forceinline__ float activate(float value)
{
    if constexpr (ACT == ST_HIP_ACT_RELU) return value > 0.0f ? value : 0.0f;
    else if constexpr (ACT == ST_HIP_ACT_GELU) return gelu_tanh(value);
    else return value;
}

template <int WTN, int TM, int ACT, bool FULL>
__device__ __forceinline__ void gemm_bf16_epilogue_bf16(const GemmBf16Args &p, const f32x16 (&acc)[TM][WTN / 32],
                                                        unsigned char *lds, int wave, int row_first, int col_base, int lane)
{
    constexpr int TN = WTN / 32;
    const int li = lane & 31, lh = lane >> 5;
    const int M = p.M, N = p.N;
    const float scale = p.scale;
    constexpr int ROW_BYTES = WTN * 2;
    constexpr int LPR8 = WTN / 8, ROWS8_PER_PASS = 64 / LPR8;  // read-back: 16 bytes (8 columns) per lane
    unsigned char *strip = lds + wave * (TM * 32 * ROW_BYTES);
    auto swz = [](int row) { return WTN == 128 ? (row & 31) : ((row >> 1) & 15); };
    // Without a bias the addend is -0.0f, which leaves every value (either zero included) as it is.
    float4 bias4[TN][4];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int g = 0; g < 4; ++g) bias4[tn][g] = make_float4(-0.0f, -0.0f, -0.0f, -0.0f);
    if (p.bias) {
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                bias4[tn][g] = *reinterpret_cast<const float4 *>(p.bias + col_base + tn * 32 + g * 8 + lh * 4);
    }
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int q = tn * 8 + g * 2 + lh;
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                float v0 = acc[tm][tn][4 * g + 0] * scale, v1 = acc[tm][tn][4 * g + 1] * scale;
                float v2 = acc[tm][tn][4 * g + 2] * scale, v3 = acc[tm][tn][4 * g + 3] * scale;
                v0 += bias4[tn][g].x; v1 += bias4[tn][g].y; v2 += bias4[tn][g].z; v3 += bias4[tn][g].w;
                uint2 packed;
                packed.x = pack_bf16x2_rne(activate<ACT>(v0), activate<ACT>(v1));
                packed.y = pack_bf16x2_rne(activate<ACT>(v2), activate<ACT>(v3));
                const int row = tm * 32 + li;
                *reinterpret_cast<uint2 *>(strip + row * ROW_BYTES + ((q ^ swz(row)) << 3)) = packed;
            }
        }
    }
    const int piece = lane & (LPR8 - 1);
#pragma unroll
    for (int j = 0; j < TM * 32 / ROWS8_PER_PASS; ++j) {
        const int local_row = j * ROWS8_PER_PASS + lane / LPR8;
        const int row = row_first + local_row;
        const unsigned char *src = strip + local_row * ROW_BYTES;
        const uint2 lo = *reinterpret_cast<const uint2 *>(src + (((2 * piece) ^ swz(local_row)) << 3));
        const uint2 hi = *reinterpret_cast<const uint2 *>(src + (((2 * piece + 1) ^ swz(local_row)) << 3));
        if (FULL || row < M) {
            u32x4 packed;
            packed.x = lo.x; packed.y = lo.y; packed.z = hi.x; packed.w = hi.y;
            *reinterpret_cast<u32x4 *>(p.C16 + static_cast<size_t>(row) * N + col_base + piece * 8) = packed;
        }
    }
}

template <int WTN, int TM, int ACT, bool RES, bool OUT32, bool OUT16, bool FULL>
__device__ __forceinline__ void gemm_bf16_epilogue_f32(const GemmBf16Args &p, const f32x16 (&acc)[TM][WTN / 32],
                                                       unsigned char *lds, int wave, int row_first, int col_base, int lane)
{
    constexpr int TN = WTN / 32;
    const int li = lane & 31, lh = lane >> 5;
    const int M = p.M, N = p.N;
    const float scale = p.scale;
    constexpr int C_STRIDE = WTN + 4;
    float *strip = reinterpret_cast<float *>(lds) + wave * (32 * C_STRIDE);
    constexpr int LPR = WTN / 4;        // lanes per strip row in the read-back phase (4 columns each)
    constexpr int ROWS_PER_PASS = 64 / LPR;
    constexpr int PASSES = 32 / ROWS_PER_PASS;
    const int col0 = col_base + (lane & (LPR - 1)) * 4;  // this lane's 4 columns in the read-back phase
    float4 bias4 = make_float4(-0.0f, -0.0f, -0.0f, -0.0f);  // x + -0.0f == x for every x
    if (p.bias) bias4 = *reinterpret_cast<const float4 *>(p.bias + col0);
    float *const c32 = p.C32;
    uint16_t *const c16 = p.C16;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
        const int row_base = row_first + tm * 32;
        // The residual rows of this strip are requested before the accumulators go through LDS.
        float4 rr[PASSES];
        if constexpr (RES) {
#pragma unroll
            for (int j = 0; j < PASSES; ++j) {
                const int row = row_base + j * ROWS_PER_PASS + lane / LPR;
                rr[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (FULL || row < M) rr[j] = *reinterpret_cast<const float4 *>(p.residual + static_cast<size_t>(row) * N + col0);
            }
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const f32x16 tile = acc[tm][tn];
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *reinterpret_cast<float4 *>(&strip[li * C_STRIDE + tn * 32 + g * 8 + lh * 4]) =
                    make_float4(tile[4 * g], tile[4 * g + 1], tile[4 * g + 2], tile[4 * g + 3]);
        }
#pragma unroll
        for (int j = 0; j < PASSES; ++j) {
            const int local_row = j * ROWS_PER_PASS + lane / LPR;
            const int row = row_base + local_row;
            float4 v = *reinterpret_cast<const float4 *>(&strip[local_row * C_STRIDE + (lane & (LPR - 1)) * 4]);
            if (FULL || row < M) {
                const size_t idx = static_cast<size_t>(row) * N + col0;
                v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
                v.x += bias4.x; v.y += bias4.y; v.z += bias4.z; v.w += bias4.w;
                if constexpr (RES) { v.x += rr[j].x; v.y += rr[j].y; v.z += rr[j].z; v.w += rr[j].w; }
                v.x = activate<ACT>(v.x);
                v.y = activate<ACT>(v.y);
                v.z = activate<ACT>(v.z);
                v.w = activate<ACT>(v.w);
                if constexpr (OUT32) *reinterpret_cast<float4 *>(c32 + idx) = v;
                if constexpr (OUT16) {
                    uint2 packed;
                    packed.x = pack_bf16x2_rne(v.x, v.y);
                    packed.y = pack_bf16x2_rne(v.z, v.w);
                    *reinterpret_cast<uint2 *>(c16 + idx) = packed;
                }
            }
        }
    }
}

template <int WTN, int TM, int ACT, bool FULL>
__device__ __forceinline__ void gemm_bf16_epilogue_act(const GemmBf16Args &p, const f32x16 (&acc)[TM][WTN / 32],
                                                       unsigned char *lds, int wave, int row_first, int col_base, int lane)
{
    const bool bf16_only = p.C32 == nullptr && (reinterpret_cast<uintptr_t>(p.C16) & 15u) == 0;
    if (bf16_only && p.residual == nullptr) {
        gemm_bf16_epilogue_bf16<WTN, TM, ACT, FULL>(p, acc, lds, wave, row_first, col_base, lane);
    } else if (p.residual) {
        if (p.C32 && p.C16) gemm_bf16_epilogue_f32<WTN, TM, ACT, true, true, true, FULL>(p, acc, lds, wave, row_first, col_base, lane);
        else if (p.C32) gemm_bf16_epilogue_f32<WTN, TM, ACT, true, true, false, FULL>(p, acc, lds, wave, row_first, col_base, lane);
        else gemm_bf16_epilogue_f32<WTN, TM, ACT, true, false, true, FULL>(p, acc, lds, wave, row_first, col_base, lane);
    } else {
        if (p.C32 && p.C16) gemm_bf16_epilogue_f32<WTN, TM, ACT, false, true, true, FULL>(p, acc, lds, wave, row_first, col_base, lane);
        else if (p.C32) gemm_bf16_epilogue_f32<WTN, TM, ACT, false, true, false, FULL>(p, acc, lds, wave, row_first, col_base, lane);
        else gemm_bf16_epilogue_f32<WTN, TM, ACT, false, false, true, FULL>(p, acc, lds, wave, row_first, col_base, lane);
    }
}

template <int WTN, int TM, int ACT>
__device__ __forceinline__ void gemm_bf16_epilogue_rows(const GemmBf16Args &p, const f32x16 (&acc)[TM][WTN / 32],
                                                        unsigned char *lds, int wave, int row_first, int col_base, int lane)
{
    // Only the last row of tiles can hang over the end of a ragged M; every other wavefront runs without row checks.
    if (row_first + TM * 32 <= p.M) gemm_bf16_epilogue_act<WTN, TM, ACT, true>(p, acc, lds, wave, row_first, col_base, lane);
    else gemm_bf16_epilogue_act<WTN, TM, ACT, false>(p, acc, lds, wave, row_first, col_base, lane);
}

// Epilogue for an N that is not a multiple of 128 (a vocabulary of 50257, 1000 classes): the rows of C, of the residual
// and the pieces of the bias start at any 4-byte (f32) or 2-byte (bf16) boundary and the last tile hangs over the end.
// Same f32 strips through LDS as above; the four columns a lane owns are stored as one 16-byte (f32) / 8-byte (bf16)
// access where they all exist — global memory takes those at any alignment, and the types say so — and one by one in
// the last piece of a row.  Everything per launch is a run-time value here: this path is bound by its stores.
template <int WTN, int TM>
__device__ __forceinline__ void gemm_bf16_epilogue_ragged(const GemmBf16Args &p, const f32x16 (&acc)[TM][WTN / 32],
                                                          unsigned char *lds, int wave, int row_first, int col_base, int lane)
{
    typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
    typedef uint32_t u32x2_a2 __attribute__((ext_vector_type(2), aligned(2)));
    constexpr int TN = WTN / 32;
    const int li = lane & 31, lh = lane >> 5;
    const int M = p.M, N = p.N;
    const float scale = p.scale;
    constexpr int C_STRIDE = WTN + 4;
    float *strip = reinterpret_cast<float *>(lds) + wave * (32 * C_STRIDE);
    constexpr int LPR = WTN / 4;
    constexpr int ROWS_PER_PASS = 64 / LPR;
    constexpr int PASSES = 32 / ROWS_PER_PASS;
    const int col0 = col_base + (lane & (LPR - 1)) * 4;
    const bool whole = col0 + 4 <= N;  // all four columns exist
    float bias[4] = {-0.0f, -0.0f, -0.0f, -0.0f};
    if (p.bias) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (col0 + e < N) bias[e] = p.bias[col0 + e];
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
        const int row_base = row_first + tm * 32;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const f32x16 tile = acc[tm][tn];
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *reinterpret_cast<float4 *>(&strip[li * C_STRIDE + tn * 32 + g * 8 + lh * 4]) =
                    make_float4(tile[4 * g], tile[4 * g + 1], tile[4 * g + 2], tile[4 * g + 3]);
        }
#pragma unroll
        for (int j = 0; j < PASSES; ++j) {
            const int local_row = j * ROWS_PER_PASS + lane / LPR;
            const int row = row_base + local_row;
            const float4 s4 = *reinterpret_cast<const float4 *>(&strip[local_row * C_STRIDE + (lane & (LPR - 1)) * 4]);
            if (row >= M || col0 >= N) continue;
            const size_t idx = static_cast<size_t>(row) * N + col0;
            float v[4] = {s4.x, s4.y, s4.z, s4.w};
            float res[4] = {0.f, 0.f, 0.f, 0.f};
            if (p.residual) {
                if (whole) {
                    const f32x4_a4 r4 = *reinterpret_cast<const f32x4_a4 *>(p.residual + idx);
                    res[0] = r4[0]; res[1] = r4[1]; res[2] = r4[2]; res[3] = r4[3];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col0 + e < N) res[e] = p.residual[idx + e];
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float value = v[e] * scale + bias[e];
                if (p.residual) value += res[e];
                v[e] = apply_activation(value, p.activation);
            }
            if (whole) {
                if (p.C32) *reinterpret_cast<f32x4_a4 *>(p.C32 + idx) = f32x4_a4{v[0], v[1], v[2], v[3]};
                if (p.C16) *reinterpret_cast<u32x2_a2 *>(p.C16 + idx) = u32x2_a2{pack_bf16x2_rne(v[0], v[1]), pack_bf16x2_rne(v[2], v[3])};
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (col0 + e >= N) continue;
                    if (p.C32) p.C32[idx + e] = v[e];
                    if (p.C16) p.C16[idx + e] = f32_to_bf16_rne(v[e]);
                }
            }
        }
    }
}

template <int WTN, int TM = 2>
__device__ __forceinline__ void gemm_bf16_epilogue(const GemmBf16Args &p, const f32x16 (&acc)[TM][WTN / 32], unsigned char *lds,
                                                   int wave, int row_first, int col_base, int lane)
{
    if (p.N & 127) return gemm_bf16_epilogue_ragged<WTN, TM>(p, acc, lds, wave, row_first, col_base, lane);
    if (p.activation == ST_HIP_ACT_GELU) gemm_bf16_epilogue_rows<WTN, TM, ST_HIP_ACT_GELU>(p, acc, lds, wave, row_first, col_base, lane);
    else if (p.activation == ST_HIP_ACT_RELU) gemm_bf16_epilogue_rows<WTN, TM, ST_HIP_ACT_RELU>(p, acc, lds, wave, row_first, col_base, lane);
    else gemm_bf16_epilogue_rows<WTN, TM, ST_HIP_ACT_NONE>(p, acc, lds, wave, row_first, col_base, lane);
}

// Epilogue of the convolution form: rows of C are output channels, columns output pixels (image-major), and the result
// goes to NCHW — channel o of image i is the contiguous run out[(i·c_out + o)·oh·ow ..].  Same f32 strips through LDS as
// above; a lane's four neighbouring columns are four consecutive pixels, stored as one 16-byte (f32) / 8-byte (bf16)
// access when the plane size is a multiple of four (then they share an image and the address is aligned), one by one
// otherwise.  The bias is per row.
template <int WTN, int TM>
__device__ __forceinline__ void conv_bf16_epilogue(const GemmBf16Args &p, const f32x16 (&acc)[TM][WTN / 32], unsigned char *lds,
                                                   int wave, int row_first, int col_base, int lane)
{
    constexpr int TN = WTN / 32;
    const int li = lane & 31, lh = lane >> 5;
    const int M = p.M, N = p.N;
    constexpr int C_STRIDE = WTN + 4;
    float *strip = reinterpret_cast<float *>(lds) + wave * (32 * C_STRIDE);
    constexpr int LPR = WTN / 4;
    constexpr int ROWS_PER_PASS = 64 / LPR;
    constexpr int PASSES = 32 / ROWS_PER_PASS;
    const int ohow = p.conv.ohow;
    const int pixel0 = col_base + (lane & (LPR - 1)) * 4;  // this lane's four pixels in the read-back phase
    const bool vector_ok = (ohow & 3) == 0;
    // image and position of each of the four pixels (the same for every row this lane stores)
    size_t plane_off[4];
    bool live[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int pixel = pixel0 + e;
        live[e] = pixel < N;
        const int image = pixel / ohow;
        plane_off[e] = static_cast<size_t>(image) * p.conv.c_out * ohow + (pixel - image * ohow);
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
        const int row_base = row_first + tm * 32;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const f32x16 tile = acc[tm][tn];
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *reinterpret_cast<float4 *>(&strip[li * C_STRIDE + tn * 32 + g * 8 + lh * 4]) =
                    make_float4(tile[4 * g], tile[4 * g + 1], tile[4 * g + 2], tile[4 * g + 3]);
        }
#pragma unroll
        for (int j = 0; j < PASSES; ++j) {
            const int local_row = j * ROWS_PER_PASS + lane / LPR;
            const int row = row_base + local_row;  // output channel
            const float4 s4 = *reinterpret_cast<const float4 *>(&strip[local_row * C_STRIDE + (lane & (LPR - 1)) * 4]);
            if (row >= M || !live[0]) continue;
            const float bias = p.bias ? p.bias[row] : -0.0f;
            float v[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = apply_activation(v[e] + bias, p.activation);
            const size_t channel_off = static_cast<size_t>(row) * ohow;
            if (vector_ok) {
                const size_t idx = plane_off[0] + channel_off;
                if (p.C32) *reinterpret_cast<float4 *>(p.C32 + idx) = make_float4(v[0], v[1], v[2], v[3]);
                if (p.C16) *reinterpret_cast<uint2 *>(p.C16 + idx) = make_uint2(pack_bf16x2_rne(v[0], v[1]), pack_bf16x2_rne(v[2], v[3]));
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (!live[e]) continue;
                    const size_t idx = plane_off[e] + channel_off;
                    if (p.C32) p.C32[idx] = v[e];
                    if (p.C16) p.C16[idx] = f32_to_bf16_rne(v[e]);
                }
            }
        }
    }
}

// Epilogue of a 256-row kernel's workgroup: the launch's own, or — when k is split over workgroups — the raw sums of
// this split into its plane of the partial buffer (the reduction kernel applies scale, bias, residual and activation).
template <int WTN, int TM>
__device__ __forceinline__ void gemm_bf16_finish(const GemmBf16Args &p, int split, const f32x16 (&acc)[TM][WTN / 32],
                                                 unsigned char *lds, int wave, int row_first, int col_base, int lane)
{
    GemmBf16Args q = p;
    if (p.k_splits > 1) {
        q.C32 = p.partial + static_cast<size_t>(split) * p.M * p.N;
        q.C16 = nullptr;
        q.bias = nullptr;
        q.residual = nullptr;
        q.scale = 1.0f;
        q.activation = ST_HIP_ACT_NONE;
    }
    gemm_bf16_epilogue<WTN, TM>(q, acc, lds, wave, row_first, col_base, lane);
}

// -------------------------------------------------------------------------------------------------
// Packed-B kernel: B is given prepacked as Bᵀ (n×k row-major, k contiguous — PackedB's column-major layout,
// crates/st-tensor/src/pure.rs:1285-1323).  Same 256×BN×64 tiles, LDS layout, swizzle and epilogue as the kernel
// above, but B needs no transposition: both operands go global memory -> LDS with buffer_load ... lds, every
// wavefront issuing an eighth of the loads of each, and the main loop carries no vector-ALU work at all (the LDS
// destination of each load is wavefront-uniform and computed on the scalar unit).
//
// Issue order is pinned: within a 16-wide k sub-step a wavefront alternates one MFMA with one memory instruction
// (a fragment read of the next sub-step, or a direct load of a later k-tile).  An MFMA occupies the matrix pipe
// for 32 cycles but issues in a few, so the memory instruction rides in its shadow; left to the compiler's own
// order (all reads of a sub-step in a burst right before the MFMAs that use them) both wavefronts of a SIMD sit
// in their read bursts at the same time and the pipe idles (4096³, all-zero operands so that the clock stays at
// 2.4 GHz: 1.22 µs per k-tile against 0.92 with the order pinned; a loop of MFMAs alone needs 0.94).
//
// WAVES = 4 (one wavefront per SIMD, 128×128 of C each, a third less LDS read traffic) is instantiable but
// measured slower (0.997 µs per k-tile on zeros, no gain on random data) and is not built.
// -------------------------------------------------------------------------------------------------
#define ST_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

template <int BN, int WAVES, int BM = 256, bool CONV = false>
__device__ __forceinline__ void gemm_bf16_packed_body(const GemmBf16Args &p)
{
    static_assert(BN == 256 || BN == 128, "tile width");
    static_assert(WAVES == 8 || WAVES == 4, "wavefronts per workgroup");
    static_assert(BM == 256 || (BM == 128 && BN == 128 && WAVES == 4), "tile height");
    constexpr int BK = 64;
    constexpr int WTM = 2 * BM / WAVES;      // wavefront tile: WAVES/2 × 2 wavefronts
    constexpr int WTN = BN / 2;
    constexpr int TM = WTM / 32, TN = WTN / 32;  // 32×32 MFMA tiles per wavefront
    constexpr int NA = BM / 8 / WAVES;       // direct loads per wavefront and k-tile: A ...
    constexpr int NB = BN / 8 / WAVES;       // ... and B (one load fills 8 rows of a stage)
    constexpr int A_STAGE = BM * 128;        // bytes: BM rows × 128 B
    constexpr int B_STAGE = BM == 256 ? 32768 : BN * 128;  // (the 256-row forms give Bᵀ 256 rows' room whatever BN is)
    constexpr int B_REGION = 3 * A_STAGE;    // [A0][A1][A2][B0][B1]
    constexpr int C_STRIDE = WTN + 4;        // floats, epilogue strip
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_bytes[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;  // WAVES/2 × 2 wavefronts, WTM × WTN each
    const int li = lane & 31, lh = lane >> 5;
    const int M = p.M, N = p.N, K = p.K;

    int logical = blockIdx.x;
    if (p.swizzle) logical = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int tiles = p.tiles_m * p.tiles_n;
    const int split = logical / tiles;  // 0 unless k is split over workgroups
    logical -= split * tiles;
    constexpr int GROUP_M = 4;
    const int width = GROUP_M * p.tiles_n;
    const int group = logical / width;
    const int first_m = group * GROUP_M;
    const int group_size = min(p.tiles_m - first_m, GROUP_M);
    const int tile_m = first_m + (logical % width) % group_size;
    const int tile_n = (logical % width) / group_size;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int tile0 = split * p.tiles_per_split;  // first k-tile of this workgroup

    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(p.A), 0, static_cast<int>(static_cast<unsigned>(M) * static_cast<unsigned>(K) * 2u), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(p.B), 0,
        static_cast<int>(CONV ? p.conv.image_bytes : static_cast<unsigned>(K) * static_cast<unsigned>(N) * 2u), 0x00020000);

    // Direct loads: instruction r of wavefront w fills rows (r*WAVES + w)*8 .. +7 of a stage (1 KB of LDS, lane l at
    // chunk position l&7 of row l>>3), so lane l fetches logical chunk (l&7) ^ swz(row), swz(r) = ((r>>1) ^ (r>>4)) & 7.
    constexpr int NMAX = NA > NB ? NA : NB;
    unsigned a_off[NA], b_off[NB];
    {
        const int row_in = wave * 8 + (lane >> 3);
        const int sw_base = ((wave * 4 + (lane >> 4)) ^ (wave >> 1)) & 7;
        const unsigned k_first = static_cast<unsigned>(tile0) * BK;
#pragma unroll
        for (int r = 0; r < NMAX; ++r) {
            const int chunk = ((lane & 7) ^ sw_base ^ ((r * WAVES / 2) & 7)) & 7;
            if (r < NA) a_off[r] = (static_cast<unsigned>(m0 + r * WAVES * 8 + row_in) * K + k_first + chunk * 8) * 2u;
            if (r < NB) {
                if constexpr (CONV) {
                    // Row n of operand B is output pixel n: its 128-byte pieces start at the pixel's first tap in the
                    // padded channels-last copy.  (Pixels past the end repeat the last one; they are never stored.)
                    const int pixel = min(n0 + r * WAVES * 8 + row_in, N - 1);
                    const int image = pixel / p.conv.ohow, rest = pixel - image * p.conv.ohow;
                    const int oy = rest / p.conv.ow, ox = rest - oy * p.conv.ow;
                    const unsigned position = (static_cast<unsigned>(image) * p.conv.hp + oy * p.conv.stride_h) * p.conv.wp + ox * p.conv.stride_w;
                    b_off[r] = (position * p.conv.c_pad + chunk * 8) * 2u;
                } else {
                    b_off[r] = (static_cast<unsigned>(n0 + r * WAVES * 8 + row_in) * K + k_first + chunk * 8) * 2u;
                }
            }
        }
    }
    // CONV: byte offset of the k-tile whose B loads are issued next (tiles are requested strictly in order): tap
    // (ky, kx), channel block cb, kept on the scalar unit and advanced without a division.
    int conv_cb = 0, conv_kx = 0, conv_row_off = 0;  // conv_row_off = ky·dil_h·wp
    unsigned conv_off = 0;
    auto conv_advance = [&]() {
        if (++conv_cb == p.conv.c_blocks) {
            conv_cb = 0;
            if (++conv_kx == p.conv.kw) {
                conv_kx = 0;
                conv_row_off += p.conv.dil_h * p.conv.wp;
            }
        }
        conv_off = (static_cast<unsigned>(conv_row_off + conv_kx * p.conv.dil_w) * p.conv.c_pad + conv_cb * 64) * 2u;
    };
    const int lds_row_block = wave * 1024;  // wavefront-uniform part of every load's LDS destination
    auto load_a1 = [&](int stage, int r, unsigned k_off) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_ptr)(lds_bytes + stage * A_STAGE + r * (WAVES * 1024) + lds_row_block),
                                                 16, a_off[r], k_off, 0, 0);
    };
    auto load_b1 = [&](int stage, int r, unsigned k_off) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrc_b, (lds_void_ptr)(lds_bytes + B_REGION + stage * B_STAGE + r * (WAVES * 1024) + lds_row_block), 16, b_off[r],
            CONV ? conv_off : k_off, 0, 0);
        if constexpr (CONV) {
            if (r == NB - 1) conv_advance();  // the last load of this k-tile: the next ones belong to the next tile
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
            acc[a][b] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // Fragment addresses: row*128 + ((q ^ swz(row)) << 4) with q = 2*kk + lh; for row = base + t*32 + li the
    // swizzle is sw0 ^ 2t, so the four values of (2kk) ^ (2t) select one of four precomputed addresses.
    unsigned a_frag[4], b_frag[4];
    {
        const int sw0 = ((li >> 1) ^ (li >> 4)) & 7;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            a_frag[c] = (wm * WTM + li) * 128 + ((lh ^ sw0 ^ ((wm * WTM / 16) & 7) ^ (2 * c)) & 7) * 16;
            b_frag[c] = B_REGION + (wn * WTN + li) * 128 + ((lh ^ sw0 ^ ((wn * WTN / 16) & 7) ^ (2 * c)) & 7) * 16;
        }
    }
    bf16x8 fa[2][TM], fb[2][TN];
    auto read_a = [&](int buf, int a_stage, int kk, int t) {
        fa[buf][t] = *reinterpret_cast<const bf16x8 *>(lds_bytes + a_frag[kk ^ t] + a_stage * A_STAGE + t * 4096);
    };
    auto read_b = [&](int buf, int b_stage, int kk, int t) {
        fb[buf][t] = *reinterpret_cast<const bf16x8 *>(lds_bytes + b_frag[kk ^ t] + b_stage * B_STAGE + t * 4096);
    };
    auto mfma = [&](int buf, int tm, int tn) {
        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][tn], fa[buf][tm], acc[tm][tn], 0, 0, 0);
    };
    // One sub-step: the TM×TN MFMAs on fragment buffer `buf`, each followed by a slot for memory instructions: the
    // first TM + TN slots issue the fragment reads of the sub-step after it (into the other buffer, in the order
    // that sub-step uses them: A0, B0 .. B(TN-1), A1 ..), the last `loads` slots one direct load each (`load(i)`).
    auto substep = [&](int buf, bool reads, int a_stage_r, int b_stage_r, int kk_r, auto &&load, int loads) {
        constexpr int SLOTS = TM * TN;
        static_assert(TM + TN <= SLOTS, "a sub-step has a slot for each fragment read");
#pragma unroll
        for (int slot = 0; slot < SLOTS; ++slot) {
            mfma(buf, slot / TN, slot % TN);
            ST_SCHED_FENCE();
            if (reads) {
                if (slot == 0) read_a(buf ^ 1, a_stage_r, kk_r, 0);
                else if (slot <= TN) read_b(buf ^ 1, b_stage_r, kk_r, slot - 1);
                else if (slot < TM + TN) read_a(buf ^ 1, a_stage_r, kk_r, slot - TN);
            }
            if (slot >= SLOTS - loads) load(slot - (SLOTS - loads));
            ST_SCHED_FENCE();
        }
    };
    auto no_load = [](int) {};

    // One k-tile t.  On entry fragment buffer 0 holds sub-step 0 of tile t; B(t+1) and A(t+1) are in flight or
    // landed.  Sub-step 0 requests A(t+2) (its stage was freed by the previous barrier); sub-step 3, after this
    // tile's barrier, requests B(t+2) into the B stage this tile was read from.  The wait before the barrier lets
    // the newest NA loads (A(t+2)) stay in flight; every load therefore has at least a whole k-tile to land.
    int a_stage = 0;  // t % 3
    auto iteration = [&](auto more_tag, auto load_tag, int t) {
        constexpr bool MORE = decltype(more_tag)::value;  // a tile t+1 exists
        constexpr bool LOAD = decltype(load_tag)::value;  // a tile t+2 exists
        const int b_stage = t & 1;
        const int a_next = a_stage == 2 ? 0 : a_stage + 1;
        const int a_load = a_next == 2 ? 0 : a_next + 1;
        const unsigned k_load = static_cast<unsigned>(t + 2) * (BK * 2u);
        auto load_a_t2 = [&](int i) { load_a1(a_load, i, k_load); };
        auto load_b_t2 = [&](int i) { load_b1(b_stage, i, k_load); };
        if constexpr (LOAD) substep(0, true, a_stage, b_stage, 1, load_a_t2, NA);
        else substep(0, true, a_stage, b_stage, 1, no_load, 0);
        substep(1, true, a_stage, b_stage, 2, no_load, 0);
        substep(0, true, a_stage, b_stage, 3, no_load, 0);
        if constexpr (MORE) {
            if constexpr (LOAD) ST_WAIT_VMCNT(NA); else ST_WAIT_VMCNT(0);
        }
        // Bare barrier: __syncthreads() would add a wait for every outstanding load.  This wavefront's LDS reads
        // of tile t have returned (lgkmcnt) before anyone may overwrite the stages they came from.
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if constexpr (LOAD) substep(1, MORE, a_next, b_stage ^ 1, 0, load_b_t2, NB);
        else substep(1, MORE, a_next, b_stage ^ 1, 0, no_load, 0);
        a_stage = a_next;
    };

    const int steps = p.k_splits > 1 ? min(p.tiles_per_split, K / BK - tile0) : K / BK;
#pragma unroll
    for (int r = 0; r < NA; ++r) load_a1(0, r, 0u);
#pragma unroll
    for (int r = 0; r < NB; ++r) load_b1(0, r, 0u);
    if (steps > 1) {
#pragma unroll
        for (int r = 0; r < NA; ++r) load_a1(1, r, BK * 2u);
#pragma unroll
        for (int r = 0; r < NB; ++r) load_b1(1, r, BK * 2u);
        ST_WAIT_VMCNT(NA + NB);
    } else {
        ST_WAIT_VMCNT(0);
    }
    __syncthreads();
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) read_a(0, 0, 0, tm);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) read_b(0, 0, 0, tn);
    int t = 0;
    for (; t + 2 < steps; ++t) iteration(std::true_type{}, std::true_type{}, t);
    if (t + 1 < steps) {
        iteration(std::true_type{}, std::false_type{}, t);
        ++t;
    }
    iteration(std::false_type{}, std::false_type{}, t);

    __syncthreads();
    if constexpr (CONV) conv_bf16_epilogue<WTN, TM>(p, acc, lds_bytes, wave, m0 + wm * WTM, n0 + wn * WTN, lane);
    else gemm_bf16_finish<WTN, TM>(p, split, acc, lds_bytes, wave, m0 + wm * WTM, n0 + wn * WTN, lane);
}

// -------------------------------------------------------------------------------------------------
// Row-complete packed-B kernel for N = 512: a workgroup owns 64 whole rows of C (64×512×64 tiles, eight wavefronts as
// 2 × 4, 32×128 of C each), so that what follows the GEMM along a row — the residual add and the layer normalisation of
// a transformer block (crates/st-vision/src/models/vit.rs:256-265) — can run in its epilogue instead of in a kernel of
// its own that reads the rows back from memory.  Same LDS layout, swizzle and direct loads as the kernel above: three
// 8 KB stages of A, two 64 KB stages of Bᵀ.  Every wavefront reads five fragments per four MFMAs, which the LDS cannot
// sustain at the matrix pipe's full rate (the kernel is meant for the memory-bound projections back to d_model).
// -------------------------------------------------------------------------------------------------
struct RowLnArgs {
    GemmBf16Args g;          // C32 = the rows before normalisation (may be null), C16 unused
    const float *gamma;      // null: no normalisation, plain epilogue
    const float *beta;
    float epsilon;
    uint16_t *ln_bf16;       // normalised rows, rounded to bf16
};

__device__ __forceinline__ void gemm_bf16_rowcomplete_body(const RowLnArgs &q)
{
    const GemmBf16Args &p = q.g;
    constexpr int BM = 64, BN = 512, BK = 64;
    constexpr int WTN = 128, TN = 4;
    constexpr int A_STAGE = BM * 128, B_STAGE = BN * 128;
    constexpr int B_REGION = 3 * A_STAGE;  // [A0][A1][A2][B0][B1]
    constexpr int NB = BN / 8 / 8;         // direct loads of B per wavefront and k-tile (one load fills 8 rows); A: one
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_bytes[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    const int li = lane & 31, lh = lane >> 5;
    const int M = p.M, K = p.K;
    const int m0 = blockIdx.x * BM;

    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(p.A), 0, static_cast<int>(static_cast<unsigned>(M) * static_cast<unsigned>(K) * 2u), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(p.B), 0, static_cast<int>(static_cast<unsigned>(K) * static_cast<unsigned>(BN) * 2u), 0x00020000);

    // Direct loads: instruction r of wavefront w fills rows (r*8 + w)*8 .. +7 of a stage, lane l at chunk position l&7 of
    // row l>>3, fetching logical chunk (l&7) ^ swz(row), swz(r) = ((r>>1) ^ (r>>4)) & 7.
    unsigned a_off, b_off[NB];
    {
        const int row_in = wave * 8 + (lane >> 3);
        const int sw_base = ((wave * 4 + (lane >> 4)) ^ (wave >> 1)) & 7;
        a_off = (static_cast<unsigned>(m0 + row_in) * K + (((lane & 7) ^ sw_base) & 7) * 8) * 2u;
#pragma unroll
        for (int r = 0; r < NB; ++r) {
            const int chunk = ((lane & 7) ^ sw_base ^ ((4 * r) & 7)) & 7;
            b_off[r] = (static_cast<unsigned>(r * 64 + row_in) * K + chunk * 8) * 2u;
        }
    }
    const int lds_row_block = wave * 1024;
    auto load_a1 = [&](int stage, unsigned k_off) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_ptr)(lds_bytes + stage * A_STAGE + lds_row_block), 16, a_off, k_off, 0, 0);
    };
    auto load_b1 = [&](int stage, int r, unsigned k_off) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_ptr)(lds_bytes + B_REGION + stage * B_STAGE + r * 8192 + lds_row_block),
                                                 16, b_off[r], k_off, 0, 0);
    };

    f32x16 acc[1][TN];
#pragma unroll
    for (int b = 0; b < TN; ++b) acc[0][b] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // Fragment addresses: row*128 + ((q ^ swz(row)) << 4), q = 2*kk + lh.  A rows are 32*wm + li (swizzle sw0 ^ 2wm), B
    // rows 128*wn + 32*t + li (swizzle sw0 ^ 2t): the four values of (2kk) ^ (2t) pick one of four addresses.
    unsigned a_frag[4], b_frag[4];
    {
        const int sw0 = ((li >> 1) ^ (li >> 4)) & 7;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            a_frag[c] = (wm * 32 + li) * 128 + ((lh ^ sw0 ^ (2 * wm) ^ (2 * c)) & 7) * 16;
            b_frag[c] = B_REGION + (wn * WTN + li) * 128 + ((lh ^ sw0 ^ (2 * c)) & 7) * 16;
        }
    }
    bf16x8 fa[2], fb[2][TN];
    auto read_a = [&](int buf, int a_stage, int kk) {
        fa[buf] = *reinterpret_cast<const bf16x8 *>(lds_bytes + a_frag[kk] + a_stage * A_STAGE);
    };
    auto read_b = [&](int buf, int b_stage, int kk, int t) {
        fb[buf][t] = *reinterpret_cast<const bf16x8 *>(lds_bytes + b_frag[kk ^ t] + b_stage * B_STAGE + t * 4096);
    };
    // One sub-step: four MFMAs on fragment buffer `buf`; behind them the five fragment reads of the sub-step after it
    // and `extra(slot)`.
    auto substep = [&](int buf, bool reads, int a_stage_r, int b_stage_r, int kk_r, auto &&extra) {
#pragma unroll
        for (int slot = 0; slot < TN; ++slot) {
            acc[0][slot] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][slot], fa[buf], acc[0][slot], 0, 0, 0);
            ST_SCHED_FENCE();
            if (reads) {
                if (slot == 0) read_a(buf ^ 1, a_stage_r, kk_r);
                read_b(buf ^ 1, b_stage_r, kk_r, slot);
            }
            extra(slot);
            ST_SCHED_FENCE();
        }
    };
    auto nothing = [](int) {};

    int a_stage = 0;  // t % 3
    auto iteration = [&](auto more_tag, auto load_tag, int t) {
        constexpr bool MORE = decltype(more_tag)::value;  // a tile t+1 exists
        constexpr bool LOAD = decltype(load_tag)::value;  // a tile t+2 exists
        const int b_stage = t & 1;
        const int a_next = a_stage == 2 ? 0 : a_stage + 1;
        const int a_load = a_next == 2 ? 0 : a_next + 1;
        const unsigned k_load = static_cast<unsigned>(t + 2) * (BK * 2u);
        substep(0, true, a_stage, b_stage, 1, [&](int slot) { if (LOAD && slot == 3) load_a1(a_load, k_load); });
        substep(1, true, a_stage, b_stage, 2, nothing);
        substep(0, true, a_stage, b_stage, 3, nothing);
        if constexpr (MORE) {
            if constexpr (LOAD) ST_WAIT_VMCNT(1); else ST_WAIT_VMCNT(0);
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        substep(1, MORE, a_next, b_stage ^ 1, 0, [&](int slot) {
            if (LOAD) {
                load_b1(b_stage, 2 * slot, k_load);
                load_b1(b_stage, 2 * slot + 1, k_load);
            }
        });
        a_stage = a_next;
    };

    const int steps = K / BK;
    load_a1(0, 0u);
#pragma unroll
    for (int r = 0; r < NB; ++r) load_b1(0, r, 0u);
    if (steps > 1) {
        load_a1(1, BK * 2u);
#pragma unroll
        for (int r = 0; r < NB; ++r) load_b1(1, r, BK * 2u);
        ST_WAIT_VMCNT(1 + NB);
    } else {
        ST_WAIT_VMCNT(0);
    }
    __syncthreads();
    read_a(0, 0, 0);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) read_b(0, 0, 0, tn);
    int t = 0;
    for (; t + 2 < steps; ++t) iteration(std::true_type{}, std::true_type{}, t);
    if (t + 1 < steps) {
        iteration(std::true_type{}, std::false_type{}, t);
        ++t;
    }
    iteration(std::false_type{}, std::false_type{}, t);

    __syncthreads();
    if (q.gamma == nullptr) {
        gemm_bf16_epilogue<WTN, 1>(p, acc, lds_bytes, wave, m0 + wm * 32, wn * WTN, lane);
        return;
    }

    // Epilogue with layer normalisation (crates/st-tensor/src/pure.rs:4008-4058 on the rows (acc·scale + bias) + residual).
    // Pass 1: the accumulators go through this wavefront's LDS strip and come back row-contiguous (a lane holds four
    // neighbouring columns of two rows per step), bias and residual are added, the rows are stored when the caller wants
    // them and kept in registers, and every lane leaves the sum and the sum of squares of its four values per row in LDS
    // (over the strips, which are dead by then).  Pass 2 adds a row's 128 partial sums in exactly the order the
    // stand-alone layer-norm kernel uses for a 512-wide row — lane L of its wavefront holds columns 4L.. and 256 + 4L..,
    // i.e. this kernel's column groups (L >> 5) and (L >> 5) + 2 at lane L & 31, and reduces with exchanges over 32, 16,
    // … 1 lanes — so both paths produce the same statistics bit for bit, and normalises from the registers.
    constexpr int C_STRIDE = WTN + 4;
    constexpr int PASSES = 16;  // 32 rows, two per step
    float *strip = reinterpret_cast<float *>(lds_bytes) + wave * (32 * C_STRIDE);
    float2 *partial = reinterpret_cast<float2 *>(lds_bytes);  // [64 rows][4 column groups][32 lanes]
    static_assert(64 * 4 * 32 * sizeof(float2) <= 8 * 32 * C_STRIDE * sizeof(float), "the partial sums overlay the strips");
    const int N = BN;
    const int l32 = lane & 31;
    const int col0 = wn * WTN + l32 * 4;
    const int half = lane >> 5;
    float4 bias4 = make_float4(-0.0f, -0.0f, -0.0f, -0.0f);
    if (p.bias) bias4 = *reinterpret_cast<const float4 *>(p.bias + col0);
    const float4 gamma4 = *reinterpret_cast<const float4 *>(q.gamma + col0);
    const float4 beta4 = *reinterpret_cast<const float4 *>(q.beta + col0);
    const int row_first = m0 + wm * 32;
    float4 rr[PASSES];
    if (p.residual) {
#pragma unroll
        for (int j = 0; j < PASSES; ++j) {
            const int row = row_first + j * 2 + half;
            rr[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (row < M) rr[j] = *reinterpret_cast<const float4 *>(p.residual + static_cast<size_t>(row) * N + col0);
        }
    }
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        const f32x16 tile = acc[0][tn];
#pragma unroll
        for (int g = 0; g < 4; ++g)
            *reinterpret_cast<float4 *>(&strip[li * C_STRIDE + tn * 32 + g * 8 + lh * 4]) =
                make_float4(tile[4 * g], tile[4 * g + 1], tile[4 * g + 2], tile[4 * g + 3]);
    }
    float4 xs[PASSES];
#pragma unroll
    for (int j = 0; j < PASSES; ++j) {
        const int local_row = j * 2 + half;
        const int row = row_first + local_row;
        float4 v = *reinterpret_cast<const float4 *>(&strip[local_row * C_STRIDE + l32 * 4]);
        v.x = v.x * p.scale + bias4.x; v.y = v.y * p.scale + bias4.y; v.z = v.z * p.scale + bias4.z; v.w = v.w * p.scale + bias4.w;
        if (p.residual) { v.x += rr[j].x; v.y += rr[j].y; v.z += rr[j].z; v.w += rr[j].w; }
        xs[j] = v;
        if (p.C32 && row < M) *reinterpret_cast<float4 *>(p.C32 + static_cast<size_t>(row) * N + col0) = v;
    }
    __syncthreads();  // every wavefront has its rows in registers: the strips may be overwritten
#pragma unroll
    for (int j = 0; j < PASSES; ++j) {
        const int tile_row = wm * 32 + j * 2 + half;
        partial[(tile_row * 4 + wn) * 32 + l32] = make_float2(sum4(xs[j]), sumsq4(xs[j]));
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PASSES; ++j) {
        const int tile_row = wm * 32 + j * 2 + half;
        const int row = m0 + tile_row;
        const float2 g0 = partial[(tile_row * 4 + 0) * 32 + l32], g1 = partial[(tile_row * 4 + 1) * 32 + l32];
        const float2 g2 = partial[(tile_row * 4 + 2) * 32 + l32], g3 = partial[(tile_row * 4 + 3) * 32 + l32];
        // lane L = l32 holds g0 + g2, lane L = 32 + l32 holds g1 + g3; the exchange over 32 lanes adds the two
        float sum = (g0.x + g2.x) + (g1.x + g3.x);
        float sumsq = (g0.y + g2.y) + (g1.y + g3.y);
#pragma unroll
        for (int w = 16; w >= 1; w >>= 1) {
            sum += __shfl_xor(sum, w);
            sumsq += __shfl_xor(sumsq, w);
        }
        const float cols_f = static_cast<float>(N);
        const float mean = sum / cols_f;
        const float var = layer_norm_variance(sumsq, mean, cols_f);
        const float denom = layer_norm_denominator(var, q.epsilon);
        // (v - mean) / denom with one division per row: the product with the reciprocal, corrected once by its exact
        // remainder, is the correctly rounded quotient (the stand-alone layer-norm kernel does the same).
        const float inv = 1.0f / denom;
        auto quotient = [&](float a) {
            const float t = a * inv;
            return fmaf(fmaf(-t, denom, a), inv, t);
        };
        const float4 v = xs[j];
        uint2 packed;
        packed.x = pack_bf16x2_rne(layer_norm_scale_shift(quotient(v.x - mean), gamma4.x, beta4.x), layer_norm_scale_shift(quotient(v.y - mean), gamma4.y, beta4.y));
        packed.y = pack_bf16x2_rne(layer_norm_scale_shift(quotient(v.z - mean), gamma4.z, beta4.z), layer_norm_scale_shift(quotient(v.w - mean), gamma4.w, beta4.w));
        if (row < M) *reinterpret_cast<uint2 *>(q.ln_bf16 + static_cast<size_t>(row) * N + col0) = packed;
    }
}

__global__ __launch_bounds__(512) void gemm_bf16_rowcomplete_kernel(RowLnArgs q) { gemm_bf16_rowcomplete_body(q); }

// -------------------------------------------------------------------------------------------------
// Row-major-B kernel in the same pinned style.  B (k×n, n contiguous) has to reach LDS as rows of Bᵀ, so it goes
// through registers: every thread owns KR k-rows × 4 columns of the k-tile (KR × 64-bit loads, a wavefront
// instruction reading 512 contiguous bytes of one k-row), transposes them with v_perm_b32 and writes 4 pieces of
// Bᵀ rows (128-bit for KR = 8, 64-bit for KR = 4) into the stage the previous barrier freed.  The loads of B(t+2)
// are issued in sub-step 2 of tile t and consumed in sub-step 1 of tile t+1; all of it — 4 direct loads of A,
// KR loads, 2·KR permutes and 4 LDS writes per wavefront and k-tile — rides in the slots behind the MFMAs.
// -------------------------------------------------------------------------------------------------
template <int BN, int BM = 256>
__device__ __forceinline__ void gemm_bf16_rowmajor_body(const GemmBf16Args &p)
{
    static_assert(BN == 256 || BN == 128, "tile width");
    static_assert(BM == 256 || (BM == 128 && BN == 128), "tile height");
    constexpr int BK = 64;
    constexpr int WAVES = BM / 32;           // a wavefront owns 64 rows × BN/2 columns of C
    constexpr int WTN = BN / 2;
    constexpr int TN = WTN / 32;
    constexpr int SLOTS = 2 * TN;            // MFMAs (and memory slots) per sub-step
    constexpr int KR = BN / (4 * WAVES);     // k-rows of B per thread: threads × KR × 4 columns = 64 × BN
    constexpr int STAGE = BM * 128;          // bytes per stage of A; a stage of B (BN × 128) never needs more
    constexpr int B_REGION = 3 * STAGE;      // [A0][A1][A2][B0][B1]
    constexpr int C_STRIDE = WTN + 4;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_bytes[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, lh = lane >> 5;
    const int M = p.M, N = p.N, K = p.K;

    int logical = blockIdx.x;
    if (p.swizzle) logical = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int tiles = p.tiles_m * p.tiles_n;
    const int split = logical / tiles;  // 0 unless k is split over workgroups
    logical -= split * tiles;
    constexpr int GROUP_M = 4;
    const int width = GROUP_M * p.tiles_n;
    const int group = logical / width;
    const int first_m = group * GROUP_M;
    const int group_size = min(p.tiles_m - first_m, GROUP_M);
    const int tile_m = first_m + (logical % width) % group_size;
    const int tile_n = (logical % width) / group_size;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int tile0 = split * p.tiles_per_split;  // first k-tile of this workgroup

    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(p.A), 0, static_cast<int>(static_cast<unsigned>(M) * static_cast<unsigned>(K) * 2u), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(p.B), 0, static_cast<int>(static_cast<unsigned>(K) * static_cast<unsigned>(N) * 2u), 0x00020000);

    // A: as in the packed kernel (instruction r of wavefront w fills rows r*8*WAVES + w*8 .. +7 of a stage).
    unsigned a_off[4];
    {
        const int row_in = wave * 8 + (lane >> 3);
        const int sw_base = ((wave * 4 + (lane >> 4)) ^ (wave >> 1)) & 7;
        const unsigned k_first = static_cast<unsigned>(tile0) * BK;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int chunk = ((lane & 7) ^ sw_base ^ ((r * WAVES / 2) & 7)) & 7;
            a_off[r] = (static_cast<unsigned>(m0 + r * 8 * WAVES + row_in) * K + k_first + chunk * 8) * 2u;
        }
    }
    const int lds_row_block = wave * 1024;
    auto load_a1 = [&](int stage, int r, unsigned k_off) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_ptr)(lds_bytes + stage * STAGE + r * (1024 * WAVES) + lds_row_block), 16,
                                                 a_off[r], k_off, 0, 0);
    };

    // B: thread (kg, nc) owns k-rows kg*KR .. +KR-1 and columns nc*4 .. +3 of the k-tile.
    const int nc = tid & (BN / 4 - 1), kg = tid / (BN / 4);
    unsigned b_voff[KR];
#pragma unroll
    for (int j = 0; j < KR; ++j) b_voff[j] = (static_cast<unsigned>(kg * KR + j) * N + n0 + nc * 4) * 2u;
    const unsigned b_tile_step = static_cast<unsigned>(BK) * N * 2u;
    uint2 rb[KR];
    auto load_b1 = [&](int j, unsigned tile) {
        const unsigned soff = __builtin_amdgcn_readfirstlane((tile + static_cast<unsigned>(tile0)) * b_tile_step);
        const auto v = __builtin_amdgcn_raw_buffer_load_b64(rsrc_b, b_voff[j], soff, 0);
        rb[j] = make_uint2(v[0], v[1]);
    };
    // Store instruction s writes column s ^ (nc & 1): odd and even lanes then hit rows of different parity and, with
    // the swizzle, the lanes of one LDS pass cover all banks.
    const unsigned sel_even = (nc & 1) ? 0x07060302u : 0x05040100u;
    const unsigned sel_odd = (nc & 1) ? 0x05040100u : 0x07060302u;
    unsigned b_store[4];
#pragma unroll
    for (int sidx = 0; sidx < 4; ++sidx) {
        const int col = nc * 4 + (sidx ^ (nc & 1));
        const int swz = ((col >> 1) ^ (col >> 4)) & 7;
        if (KR == 8) b_store[sidx] = B_REGION + col * 128 + ((kg ^ swz) & 7) * 16;
        else b_store[sidx] = B_REGION + col * 128 + (((kg >> 1) ^ swz) & 7) * 16 + (kg & 1) * 8;
    }
    // Piece `sidx` of the transposed block: the KR k-values of one column as KR/2 dwords.
    auto store_b1 = [&](int sidx, int stage) {
        const unsigned sel = (sidx & 1) ? sel_odd : sel_even;
        unsigned out[KR / 2];
#pragma unroll
        for (int i = 0; i < KR / 2; ++i) {
            const unsigned hi = (sidx >> 1) ? rb[2 * i + 1].y : rb[2 * i + 1].x;
            const unsigned lo = (sidx >> 1) ? rb[2 * i].y : rb[2 * i].x;
            out[i] = __builtin_amdgcn_perm(hi, lo, sel);
        }
        if constexpr (KR == 8) {
            u32x4 v;
            v.x = out[0]; v.y = out[1]; v.z = out[2]; v.w = out[3];
            *reinterpret_cast<u32x4 *>(lds_bytes + b_store[sidx] + stage * STAGE) = v;
        } else {
            *reinterpret_cast<uint2 *>(lds_bytes + b_store[sidx] + stage * STAGE) = make_uint2(out[0], out[1]);
        }
    };

    f32x16 acc[2][TN];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
            acc[a][b] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    unsigned a_frag[4], b_frag[4];
    {
        const int sw0 = ((li >> 1) ^ (li >> 4)) & 7;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            a_frag[c] = (wm * 64 + li) * 128 + ((lh ^ sw0 ^ ((wm & 1) * 4) ^ (2 * c)) & 7) * 16;
            b_frag[c] = B_REGION + (wn * WTN + li) * 128 + ((lh ^ sw0 ^ ((wn * WTN / 16) & 7) ^ (2 * c)) & 7) * 16;
        }
    }
    bf16x8 fa[2][2], fb[2][TN];
    auto read_a = [&](int buf, int a_stage, int kk, int t) {
        fa[buf][t] = *reinterpret_cast<const bf16x8 *>(lds_bytes + a_frag[kk ^ t] + a_stage * STAGE + t * 4096);
    };
    auto read_b = [&](int buf, int b_stage, int kk, int t) {
        fb[buf][t] = *reinterpret_cast<const bf16x8 *>(lds_bytes + b_frag[kk ^ t] + b_stage * STAGE + t * 4096);
    };
    // One sub-step: the 2×TN MFMAs on fragment buffer `buf`, each followed by a slot: a fragment read of the sub-step
    // after it in the first 2 + TN slots (A0, B0 .. B(TN-1), A1), then whatever `extra(slot)` issues.
    auto substep = [&](int buf, bool reads, int a_stage_r, int b_stage_r, int kk_r, auto &&extra) {
#pragma unroll
        for (int slot = 0; slot < SLOTS; ++slot) {
            acc[slot / TN][slot % TN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][slot % TN], fa[buf][slot / TN],
                                                                              acc[slot / TN][slot % TN], 0, 0, 0);
            ST_SCHED_FENCE();
            if (reads) {
                if (slot == 0) read_a(buf ^ 1, a_stage_r, kk_r, 0);
                else if (slot <= TN) read_b(buf ^ 1, b_stage_r, kk_r, slot - 1);
                else if (slot < 2 + TN) read_a(buf ^ 1, a_stage_r, kk_r, slot - TN);
            }
            extra(slot);
            ST_SCHED_FENCE();
        }
    };
    auto nothing = [](int) {};

    // One k-tile t.  On entry: fragment buffer 0 holds sub-step 0 of tile t, rb holds (or is receiving) B(t+1),
    // A(t+1) is in flight or landed.
    int a_stage = 0;  // t % 3
    auto iteration = [&](auto more_tag, auto load_tag, int t) {
        constexpr bool MORE = decltype(more_tag)::value;  // a tile t+1 exists
        constexpr bool LOAD = decltype(load_tag)::value;  // a tile t+2 exists
        const int b_stage = t & 1;
        const int a_next = a_stage == 2 ? 0 : a_stage + 1;
        const int a_load = a_next == 2 ? 0 : a_next + 1;
        const unsigned k_load = static_cast<unsigned>(t + 2) * (BK * 2u);
        // sub-step 0: A(t+2) into the stage the previous barrier freed
        substep(0, true, a_stage, b_stage, 1, [&](int slot) {
            if (LOAD && slot >= SLOTS - 4) load_a1(a_load, slot - (SLOTS - 4), k_load);
        });
        // sub-step 1: B(t+1) from the registers into the other B stage
        substep(1, true, a_stage, b_stage, 2, [&](int slot) {
            if (!MORE) return;
            if (SLOTS == 8) {
                if (slot & 1) store_b1(slot >> 1, b_stage ^ 1);
            } else {
                store_b1(slot, b_stage ^ 1);
            }
        });
        // sub-step 2: B(t+2) into the registers
        substep(0, true, a_stage, b_stage, 3, [&](int slot) {
            if constexpr (KR > SLOTS) {
                if (LOAD) {
#pragma unroll
                    for (int j = 0; j < KR / SLOTS; ++j) load_b1(slot * (KR / SLOTS) + j, static_cast<unsigned>(t + 2));
                }
            } else {
                if (LOAD && slot < KR) load_b1(slot, static_cast<unsigned>(t + 2));
            }
        });
        if constexpr (MORE) {
            if constexpr (LOAD) ST_WAIT_VMCNT(4 + KR); else ST_WAIT_VMCNT(0);
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wavefront's LDS reads and writes are done
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        substep(1, MORE, a_next, b_stage ^ 1, 0, nothing);
        a_stage = a_next;
    };

    const int steps = p.k_splits > 1 ? min(p.tiles_per_split, K / BK - tile0) : K / BK;
#pragma unroll
    for (int r = 0; r < 4; ++r) load_a1(0, r, 0u);
#pragma unroll
    for (int j = 0; j < KR; ++j) load_b1(j, 0u);
    if (steps > 1) {
#pragma unroll
        for (int r = 0; r < 4; ++r) load_a1(1, r, BK * 2u);
    }
#pragma unroll
    for (int sidx = 0; sidx < 4; ++sidx) store_b1(sidx, 0);
    if (steps > 1) {
#pragma unroll
        for (int j = 0; j < KR; ++j) load_b1(j, 1u);
        ST_WAIT_VMCNT(4 + KR);
    } else {
        ST_WAIT_VMCNT(0);
    }
    __syncthreads();
    read_a(0, 0, 0, 0);
    read_a(0, 0, 0, 1);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) read_b(0, 0, 0, tn);
    int t = 0;
    for (; t + 2 < steps; ++t) iteration(std::true_type{}, std::true_type{}, t);
    if (t + 1 < steps) {
        iteration(std::true_type{}, std::false_type{}, t);
        ++t;
    }
    iteration(std::false_type{}, std::false_type{}, t);

    __syncthreads();
    gemm_bf16_finish<WTN, 2>(p, split, acc, lds_bytes, wave, m0 + wm * 64, n0 + wn * WTN, lane);
}

__global__ __launch_bounds__(512) void gemm_bf16_256rm_kernel(GemmBf16Args p) { gemm_bf16_rowmajor_body<256>(p); }
__global__ __launch_bounds__(512) void gemm_bf16_256x128rm_kernel(GemmBf16Args p) { gemm_bf16_rowmajor_body<128>(p); }
__global__ __launch_bounds__(256, 2) void gemm_bf16_128x128w4_rm_kernel(GemmBf16Args p) { gemm_bf16_rowmajor_body<128, 128>(p); }

__global__ __launch_bounds__(512) void gemm_bf16_256w8_packed_kernel(GemmBf16Args p) { gemm_bf16_packed_body<256, 8>(p); }
__global__ __launch_bounds__(512) void gemm_bf16_256x128w8_packed_kernel(GemmBf16Args p) { gemm_bf16_packed_body<128, 8>(p); }
// 128×128 tiles, four wavefronts (64×64 of C each), 80 KB of LDS: two workgroups per compute unit.  Every MFMA needs a
// fragment read of its own (the 256-row forms need three for four), so its main loop is LDS-bound; it serves launches
// that would otherwise leave most compute units without a tile (1024³ is 16 tiles of 256×256).
__global__ __launch_bounds__(256, 2) void gemm_bf16_128x128w4_packed_kernel(GemmBf16Args p) { gemm_bf16_packed_body<128, 4, 128>(p); }
// Convolution forms (conv_bf16 below): 128 output channels × 128 pixels with four wavefronts, two workgroups per compute
// unit, and 256 output channels × 128 / 256 pixels with eight.
__global__ __launch_bounds__(256, 2) void conv2d_bf16_128x128w4_kernel(GemmBf16Args p) { gemm_bf16_packed_body<128, 4, 128, true>(p); }
__global__ __launch_bounds__(512) void conv2d_bf16_256x128w8_kernel(GemmBf16Args p) { gemm_bf16_packed_body<128, 8, 256, true>(p); }
__global__ __launch_bounds__(512) void conv2d_bf16_256x256w8_kernel(GemmBf16Args p) { gemm_bf16_packed_body<256, 8, 256, true>(p); }

// Zero-padded channels-last copy of NCHW bf16 images: out[image][yp][xp][c_pad], yp = y + pad_h, xp = x + pad_w, channels
// past c_in and the border positions zero.  One workgroup per (64-channel block, padded row, image): the row's
// [64 channels][w] block is read along x, four pixels (8 bytes, at whatever alignment the row has) per lane, and written
// along the channels, 16 bytes per lane, through a transposing LDS tile.  The workgroups behind those of the images
// re-lay the weights in the same launch: OIHW -> (c_out, kh·kw·c_pad) with k ordered (ky, kx, channel), channels past c_in zero.
struct ConvBf16Relayout {
    const uint16_t *in;
    uint16_t *out;
    const uint16_t *weight_in;
    uint16_t *weight_out;
    int batch, c_in, h, w, c_pad, hp, wp, pad_h, pad_w, c_out, taps;
    unsigned image_blocks;  // workgroups that copy image rows; the ones behind them re-lay the weights
};

__global__ __launch_bounds__(256) void conv_bf16_relayout_kernel(ConvBf16Relayout p)
{
    constexpr int TILE_W = 256;
    __shared__ __attribute__((aligned(8))) uint16_t tile[64][TILE_W + 4];
    typedef uint32_t u32x2_a2 __attribute__((ext_vector_type(2), aligned(2)));
    const int tid = threadIdx.x;
    if (blockIdx.x >= p.image_blocks) {  // the weights: 1024 values per workgroup
        const size_t row = static_cast<size_t>(p.taps) * p.c_pad, total = static_cast<size_t>(p.c_out) * row;
        const size_t first = static_cast<size_t>(blockIdx.x - p.image_blocks) * 1024 + tid;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const size_t idx = first + i * 256;
            if (idx >= total) break;
            const int o = static_cast<int>(idx / row);
            const int rest = static_cast<int>(idx - static_cast<size_t>(o) * row);
            const int tap = rest / p.c_pad, c = rest - tap * p.c_pad;
            p.weight_out[idx] = c < p.c_in ? p.weight_in[(static_cast<size_t>(o) * p.c_in + c) * p.taps + tap] : static_cast<uint16_t>(0);
        }
        return;
    }
    const int c_blocks = p.c_pad / 64;
    const int cb = blockIdx.x % c_blocks, yp = (blockIdx.x / c_blocks) % p.hp, image = blockIdx.x / (c_blocks * p.hp);
    const int y = yp - p.pad_h, w = p.w;
    uint16_t *row_out = p.out + ((static_cast<size_t>(image) * p.hp + yp) * p.wp) * p.c_pad + cb * 64;
    const bool row_inside = y >= 0 && y < p.h;
    const int channels = min(64, p.c_in - cb * 64);  // channels of this block that exist
    for (int x0 = 0; x0 < w || x0 == 0; x0 += TILE_W) {  // x0: first image column of this piece
        const int piece_w = min(TILE_W, w - x0), quads = (piece_w + 3) / 4;
        __syncthreads();
        if (row_inside) {
            // sixteen lanes per channel row, four pixels each; sixteen channels per pass
            for (int c = tid >> 4; c < channels; c += 16)
            for (int x = (tid & 15) * 4; x < quads * 4; x += 64) {
                const uint16_t *src = p.in + ((static_cast<size_t>(image) * p.c_in + cb * 64 + c) * p.h + y) * w + x0 + x;
                uint16_t v[4] = {0, 0, 0, 0};
                if (x + 4 <= piece_w) {
                    const u32x2_a2 two = *reinterpret_cast<const u32x2_a2 *>(src);
                    v[0] = static_cast<uint16_t>(two[0]); v[1] = static_cast<uint16_t>(two[0] >> 16);
                    v[2] = static_cast<uint16_t>(two[1]); v[3] = static_cast<uint16_t>(two[1] >> 16);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (x + e < piece_w) v[e] = src[e];
                }
                *reinterpret_cast<uint2 *>(&tile[c][x]) = make_uint2(v[0] | (static_cast<uint32_t>(v[1]) << 16), v[2] | (static_cast<uint32_t>(v[3]) << 16));
            }
        }
        __syncthreads();
        // Padded columns this piece covers: the left border with the first piece, the right border with the last.
        const int first_xp = x0 == 0 ? 0 : x0 + p.pad_w;
        const int last_xp = x0 + piece_w >= w ? p.wp : x0 + piece_w + p.pad_w;
        for (int idx = tid; idx < (last_xp - first_xp) * 8; idx += 256) {
            const int xp = first_xp + (idx >> 3), part = idx & 7;
            const int col = xp - p.pad_w - x0;  // column within the tile (outside [0, piece_w): border)
            uint32_t words[4] = {0u, 0u, 0u, 0u};
            if (row_inside && col >= 0 && col < piece_w) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int c = part * 8 + 2 * e;
                    const uint32_t lo = c < channels ? tile[c][col] : 0u, hi = c + 1 < channels ? tile[c + 1][col] : 0u;
                    words[e] = lo | (hi << 16);
                }
            }
            *reinterpret_cast<uint4 *>(row_out + static_cast<size_t>(xp) * p.c_pad + part * 8) = make_uint4(words[0], words[1], words[2], words[3]);
        }
    }
}

// Epilogue of the persistent kernel: the arithmetic and the strip layout of gemm_bf16_epilogue_bf16<64, 2, ACT, true>
// (same bits), written to need few registers — the kernel runs three wavefronts per SIMD, 168 registers each, and
// anything the compiler spills here is reloaded behind the tile's stores, i.e. waits for them.  Bias and output go
// through buffer descriptors (one 32-bit offset per access instead of a 64-bit address), and the bias of the next
// group of four columns is requested while the current one is used.
template <int ACT>
__device__ __forceinline__ void persistent_epilogue_bf16(const GemmBf16Args &p, const f32x16 (&acc)[2][2], unsigned char *strip,
                                                         int row_first, int col_base, int lane)
{
    const int li = lane & 31, lh = lane >> 5;
    const float scale = p.scale;
    const bool has_bias = p.bias != nullptr;
    const __amdgpu_buffer_rsrc_t rsrc_bias = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(p.bias), 0, has_bias ? static_cast<int>(static_cast<unsigned>(p.N) * 4u) : 0, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(
        p.C16, 0, static_cast<int>(static_cast<unsigned>(p.M) * static_cast<unsigned>(p.N) * 2u), 0x00020000);
    auto load_bias = [&](int group) {  // group = tn*4 + g: columns col_base + 32 tn + 8 g + 4 lh .. +3; zeros without a bias
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        const u32x4 raw = __builtin_amdgcn_raw_buffer_load_b128(
            rsrc_bias, static_cast<unsigned>(col_base + (group >> 2) * 32 + (group & 3) * 8 + lh * 4) * 4u, 0, 0);
        const f32x4 v = __builtin_bit_cast(f32x4, raw);
        return make_float4(v.x, v.y, v.z, v.w);
    };
    const float4 no_bias = make_float4(-0.0f, -0.0f, -0.0f, -0.0f);  // x + -0.0f == x for every x
    float4 bias_now = has_bias ? load_bias(0) : no_bias;
#pragma unroll
    for (int group = 0; group < 8; ++group) {
        const int tn = group >> 2, g = group & 3;
        float4 bias_next = no_bias;
        if (group + 1 < 8 && has_bias) bias_next = load_bias(group + 1);
        const int q = tn * 8 + g * 2 + lh;
#pragma unroll
        for (int tm = 0; tm < 2; ++tm) {
            float v0 = acc[tm][tn][4 * g + 0] * scale, v1 = acc[tm][tn][4 * g + 1] * scale;
            float v2 = acc[tm][tn][4 * g + 2] * scale, v3 = acc[tm][tn][4 * g + 3] * scale;
            v0 += bias_now.x; v1 += bias_now.y; v2 += bias_now.z; v3 += bias_now.w;
            uint2 packed;
            packed.x = pack_bf16x2_rne(activate<ACT>(v0), activate<ACT>(v1));
            packed.y = pack_bf16x2_rne(activate<ACT>(v2), activate<ACT>(v3));
            const int row = tm * 32 + li;
            *reinterpret_cast<uint2 *>(strip + row * 128 + ((q ^ ((row >> 1) & 15)) << 3)) = packed;
        }
        bias_now = bias_next;
    }
    const int piece = lane & 7;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int local_row = j * 8 + (lane >> 3);
        const unsigned char *src = strip + local_row * 128;
        const uint2 lo = *reinterpret_cast<const uint2 *>(src + (((2 * piece) ^ ((local_row >> 1) & 15)) << 3));
        const uint2 hi = *reinterpret_cast<const uint2 *>(src + (((2 * piece + 1) ^ ((local_row >> 1) & 15)) << 3));
        u32x4 packed;
        packed.x = lo.x; packed.y = lo.y; packed.z = hi.x; packed.w = hi.y;
        __builtin_amdgcn_raw_buffer_store_b128(
            packed, rsrc_c, (static_cast<unsigned>(row_first + local_row) * static_cast<unsigned>(p.N) + col_base + piece * 8) * 2u, 0, 0);
    }
}

// The same for f32 output: the wavefront's 64×64 accumulators leave in two passes of 32 rows through the same 8 KB
// strip (32 rows × 256 B; the 16-byte chunk q of row r sits at chunk q ^ (r & 15), which spreads the eight rows a
// 128-bit write touches per cycle and the sixteen chunks of a row a read touches over all banks), are read back
// row-contiguous — sixteen lanes per row, 128 bits each — and stored as whole 256-byte row segments.  Scale, bias and
// activation are applied after the read-back, where a lane keeps the same four columns for all rows.
template <int ACT>
__device__ __forceinline__ void persistent_epilogue_f32(const GemmBf16Args &p, const f32x16 (&acc)[2][2], unsigned char *strip,
                                                        int row_first, int col_base, int lane)
{
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const int li = lane & 31, lh = lane >> 5;
    const float scale = p.scale;
    const bool has_bias = p.bias != nullptr;
    const __amdgpu_buffer_rsrc_t rsrc_bias = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(p.bias), 0, has_bias ? static_cast<int>(static_cast<unsigned>(p.N) * 4u) : 0, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(
        p.C32, 0, static_cast<int>(static_cast<unsigned>(p.M) * static_cast<unsigned>(p.N) * 4u), 0x00020000);
    const int piece = lane & 15, sub_row = lane >> 4;
    f32x4 bias4 = {-0.0f, -0.0f, -0.0f, -0.0f};  // x + -0.0f == x for every x
    if (has_bias)
        bias4 = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_bias, static_cast<unsigned>(col_base + piece * 4) * 4u, 0, 0));
#pragma unroll
    for (int tm = 0; tm < 2; ++tm) {
#pragma unroll
        for (int tn = 0; tn < 2; ++tn)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int q = tn * 8 + g * 2 + lh;
                *reinterpret_cast<f32x4 *>(strip + li * 256 + ((q ^ (li & 15)) << 4)) =
                    f32x4{acc[tm][tn][4 * g], acc[tm][tn][4 * g + 1], acc[tm][tn][4 * g + 2], acc[tm][tn][4 * g + 3]};
            }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int local_row = j * 4 + sub_row;
            f32x4 v = *reinterpret_cast<const f32x4 *>(strip + local_row * 256 + ((piece ^ (local_row & 15)) << 4));
            v = v * scale + bias4;
            v.x = activate<ACT>(v.x);
            v.y = activate<ACT>(v.y);
            v.z = activate<ACT>(v.z);
            v.w = activate<ACT>(v.w);
            __builtin_amdgcn_raw_buffer_store_b128(
                __builtin_bit_cast(u32x4, v), rsrc_c,
                (static_cast<unsigned>(row_first + tm * 32 + local_row) * static_cast<unsigned>(p.N) + col_base + piece * 4) * 4u, 0, 0);
        }
    }
}

// The lane index, from the hardware and opaque to the compiler: what is computed from it can neither be hoisted out of
// a loop nor has an input that must stay in a register until then.
__device__ __forceinline__ int fresh_lane_index()
{
    int lane;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
    return lane;
}

// -------------------------------------------------------------------------------------------------
// Persistent packed-B kernel, 256×128 tiles, bf16 output, M a multiple of 256: one workgroup per compute unit walks
// through its tiles, and four more wavefronts do nothing but request the operands (buffer_load ... lds), always two
// k-tiles ahead of the eight that compute — across tile boundaries too.  What this buys: a wavefront counts its
// loads and its stores in one in-order counter, so a wavefront that both stores a tile's results and loads the next
// tile's operands cannot wait for the loads without waiting for the stores as well.  Here the computing wavefronts
// never wait for memory at all (their stores drain while they are back in the main loop of the next tile) and the
// loading wavefronts never store.  While a tile's results go through the LDS strips of the epilogue, the next tile's
// first two k-tiles are already in their stages: the strips use the A stage the tile finished in (wavefronts 0-3)
// and 32 KB beside the stages (wavefronts 4-7).  Layout, swizzle, fragment reads and issue order of the main loop
// are those of the packed kernel above.
// -------------------------------------------------------------------------------------------------
template <bool OUT32>
__device__ __forceinline__ void gemm_bf16_persistent_body(const GemmBf16Args &p)
{
    constexpr int BM = 256, BN = 128, BK = 64;
    constexpr int WTM = 64, WTN = 64, TM = 2, TN = 2;
    constexpr int A_STAGE = BM * 128, B_STAGE = BN * 128;
    constexpr int B_REGION = 3 * A_STAGE;              // [A0][A1][A2][B0][B1][spare 32 KB]
    constexpr int SPARE = B_REGION + 2 * B_STAGE;
    constexpr int LOADERS = 4;                         // loading wavefronts (a wavefront can have 64 loads in flight)
    constexpr int NA = BM / 8 / LOADERS, NB = BN / 8 / LOADERS;  // direct loads per loading wavefront and k-tile
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_bytes[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int K = p.K, N = p.N;
    const int steps = K / BK;
    const int tiles = p.tiles_m * p.tiles_n;

    // Tile j of this workgroup.  With the XCD mapping each XCD (workgroup id mod 8) owns a contiguous eighth of the
    // tile order and its workgroups take it in rounds; otherwise the launch's workgroups take the order in rounds.
    auto tile_of = [&](int j, int &m0, int &n0) -> bool {
        int logical;
        if (p.swizzle) {
            const int per_xcd = tiles >> 3;
            const int idx = static_cast<int>(blockIdx.x >> 3) + j * static_cast<int>(gridDim.x >> 3);
            if (idx >= per_xcd) return false;
            logical = static_cast<int>(blockIdx.x & 7) * per_xcd + idx;
        } else {
            logical = static_cast<int>(blockIdx.x) + j * static_cast<int>(gridDim.x);
            if (logical >= tiles) return false;
        }
        constexpr int GROUP_M = 4;
        const int width = GROUP_M * p.tiles_n;
        const int group = logical / width;
        const int first_m = group * GROUP_M;
        const int group_size = min(p.tiles_m - first_m, GROUP_M);
        m0 = (first_m + (logical % width) % group_size) * BM;
        n0 = ((logical % width) / group_size) * BN;
        return true;
    };
    int my_tiles = 0;
    {
        int m0, n0;
        while (tile_of(my_tiles, m0, n0)) ++my_tiles;
    }
    const int total = my_tiles * steps;  // k-tiles this workgroup goes through

    if (wave >= 8) {
        // ---- the loading wavefronts ----
        const int loader = wave - 8;
        const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint16_t *>(p.A), 0, static_cast<int>(static_cast<unsigned>(p.M) * static_cast<unsigned>(K) * 2u), 0x00020000);
        const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint16_t *>(p.B), 0, static_cast<int>(static_cast<unsigned>(K) * static_cast<unsigned>(N) * 2u), 0x00020000);
        // Instruction i of loading wavefront w fills rows 8(4i + w) .. +7 of a stage (lane l: row l>>3, chunk position
        // l&7) and fetches the chunk that the swizzle swz(r) = ((r>>1) ^ (r>>4)) & 7 stores there.  The tile's and
        // k-tile's offset is scalar.
        unsigned off[NA];
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            const int row = (i * LOADERS + loader) * 8 + (lane >> 3);
            const int chunk = ((lane & 7) ^ (row >> 1) ^ (row >> 4)) & 7;
            off[i] = (static_cast<unsigned>(row) * K + chunk * 8) * 2u;
        }
        int jp = 0, ktp = 0, m0p = 0, n0p = 0;  // the k-tile requested next
        tile_of(0, m0p, n0p);
        auto advance = [&]() {
            if (++ktp == steps) {
                ktp = 0;
                ++jp;
                tile_of(jp, m0p, n0p);
            }
        };
        auto issue_a = [&](int f) {
            const unsigned soff = __builtin_amdgcn_readfirstlane((static_cast<unsigned>(m0p) * K + ktp * BK) * 2u);
            unsigned char *stage = lds_bytes + (f % 3) * A_STAGE;
#pragma unroll
            for (int i = 0; i < NA; ++i)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_ptr)(stage + (i * LOADERS + loader) * 1024), 16, off[i], soff, 0, 0);
        };
        auto issue_b = [&](int f) {
            const unsigned soff = __builtin_amdgcn_readfirstlane((static_cast<unsigned>(n0p) * K + ktp * BK) * 2u);
            unsigned char *stage = lds_bytes + B_REGION + (f & 1) * B_STAGE;
#pragma unroll
            for (int i = 0; i < NB; ++i)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_ptr)(stage + (i * LOADERS + loader) * 1024), 16, off[i], soff, 0, 0);
        };
        auto barrier = [&]() {
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };
        if (total > 0) {
            issue_a(0);
            issue_b(0);
            advance();
        }
        if (total > 1) {
            issue_a(1);
            issue_b(1);
            advance();
            ST_WAIT_VMCNT(NA + NB);
        } else {
            ST_WAIT_VMCNT(0);
        }
        barrier();  // k-tile 0 is in LDS
        int kt = 0, j = 0;
        for (int f = 0; f < total; ++f) {
            const bool ahead = f + 2 < total;
            if (ahead) issue_a(f + 2);  // into the stage of k-tile f-1, which every wavefront has left
            if (ahead) ST_WAIT_VMCNT(NA); else ST_WAIT_VMCNT(0);  // k-tile f+1 has landed
            barrier();                  // the computing wavefronts have read k-tile f
            if (ahead) {
                issue_b(f + 2);         // into the B stage of k-tile f
                advance();
            }
            if (++kt == steps) {
                kt = 0;
                ++j;
                if (j < my_tiles) barrier();  // the epilogue's strips (in the A stage of k-tile f) are done with
            }
        }
        return;
    }

    // ---- the eight computing wavefronts ----
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, lh = lane >> 5;
    f32x16 acc[TM][TN];
    auto clear = [&]() {
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int b = 0; b < TN; ++b)
                acc[a][b] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    };
    clear();
    // Fragment addresses are recomputed at the start of every tile (from a copy of the lane index the compiler
    // cannot see through): kept across the epilogue they are spilled there, and a reload behind the epilogue's stores
    // waits for those stores — the very wait this kernel exists to avoid.
    unsigned a_frag[4], b_frag[4];
    auto fragment_addresses = [&]() {
        const int l = fresh_lane_index();
        const int li_ = l & 31, lh_ = l >> 5;
        const int sw0 = ((li_ >> 1) ^ (li_ >> 4)) & 7;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            a_frag[c] = (wm * WTM + li_) * 128 + ((lh_ ^ sw0 ^ ((wm * WTM / 16) & 7) ^ (2 * c)) & 7) * 16;
            b_frag[c] = B_REGION + (wn * WTN + li_) * 128 + ((lh_ ^ sw0 ^ ((wn * WTN / 16) & 7) ^ (2 * c)) & 7) * 16;
        }
    };
    fragment_addresses();
    bf16x8 fa[2][TM], fb[2][TN];
    auto read_a = [&](int buf, int a_stage, int kk, int t) {
        fa[buf][t] = *reinterpret_cast<const bf16x8 *>(lds_bytes + a_frag[kk ^ t] + a_stage * A_STAGE + t * 4096);
    };
    auto read_b = [&](int buf, int b_stage, int kk, int t) {
        fb[buf][t] = *reinterpret_cast<const bf16x8 *>(lds_bytes + b_frag[kk ^ t] + b_stage * B_STAGE + t * 4096);
    };
    // One sub-step: four MFMAs on fragment buffer `buf`, each followed by one fragment read of the sub-step after it.
    auto substep = [&](int buf, bool reads, int a_stage_r, int b_stage_r, int kk_r) {
#pragma unroll
        for (int slot = 0; slot < 4; ++slot) {
            acc[slot / TN][slot % TN] =
                __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][slot % TN], fa[buf][slot / TN], acc[slot / TN][slot % TN], 0, 0, 0);
            ST_SCHED_FENCE();
            if (reads) {
                if (slot == 0) read_a(buf ^ 1, a_stage_r, kk_r, 0);
                else if (slot <= TN) read_b(buf ^ 1, b_stage_r, kk_r, slot - 1);
                else read_a(buf ^ 1, a_stage_r, kk_r, slot - TN);
            }
            ST_SCHED_FENCE();
        }
    };
    auto barrier = [&]() {
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wavefront's LDS traffic is done
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    auto first_fragments = [&](int a_stage, int b_stage) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) read_a(0, a_stage, 0, tm);
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) read_b(0, b_stage, 0, tn);
    };

    barrier();  // k-tile 0 is in LDS
    first_fragments(0, 0);
    int a_stage = 0, f = 0;
    for (int j = 0; j < my_tiles; ++j) {
        int m0, n0;
        tile_of(j, m0, n0);
        for (int kt = 0; kt < steps; ++kt, ++f) {
            const int b_stage = f & 1;
            const int a_next = a_stage == 2 ? 0 : a_stage + 1;
            substep(0, true, a_stage, b_stage, 1);
            substep(1, true, a_stage, b_stage, 2);
            substep(0, true, a_stage, b_stage, 3);
            barrier();  // everyone has read k-tile f; k-tile f+1 has landed
            // The last sub-step is the same code for every k-tile, fragment reads of the following k-tile included (after
            // a tile's last k-tile they fetch the next tile's first fragments, which the epilogue path below fetches again:
            // an arm of the branch that ends in MFMAs of its own made the compiler carry both arms' fragment registers
            // through the epilogue, spill them there and reload them behind the tile's stores).
            substep(1, true, a_next, b_stage ^ 1, 0);
            if (kt + 1 == steps) {
                // Strips: wavefronts 0-3 in the A stage this tile finished in, 4-7 beside the stages.
                unsigned char *strips = wave < 4 ? lds_bytes + a_stage * A_STAGE : lds_bytes + SPARE - 4 * (TM * 32 * WTN * 2);
                const int row_first = m0 + wm * WTM, col_base = n0 + wn * WTN;
                // (The epilogue's per-lane addresses are recomputed for every tile: hoisted out of the tile loop they
                // would stay in registers through the main loop, which has none to spare with three wavefronts on every SIMD.)
                const int lane_now = fresh_lane_index();
                unsigned char *strip = strips + wave * (TM * 32 * WTN * 2);
                if constexpr (OUT32) {
                    if (p.activation == ST_HIP_ACT_GELU) persistent_epilogue_f32<ST_HIP_ACT_GELU>(p, acc, strip, row_first, col_base, lane_now);
                    else if (p.activation == ST_HIP_ACT_RELU) persistent_epilogue_f32<ST_HIP_ACT_RELU>(p, acc, strip, row_first, col_base, lane_now);
                    else persistent_epilogue_f32<ST_HIP_ACT_NONE>(p, acc, strip, row_first, col_base, lane_now);
                } else {
                    if (p.activation == ST_HIP_ACT_GELU) persistent_epilogue_bf16<ST_HIP_ACT_GELU>(p, acc, strip, row_first, col_base, lane_now);
                    else if (p.activation == ST_HIP_ACT_RELU) persistent_epilogue_bf16<ST_HIP_ACT_RELU>(p, acc, strip, row_first, col_base, lane_now);
                    else persistent_epilogue_bf16<ST_HIP_ACT_NONE>(p, acc, strip, row_first, col_base, lane_now);
                }
                clear();
                if (j + 1 < my_tiles) barrier();  // the strips are done with: the A stage may be refilled
                // (Unconditional — after the last tile they read a stage nobody uses any more — so that nothing of the
                // old fragments has to survive the epilogue.)
                fragment_addresses();
                first_fragments(a_next, b_stage ^ 1);
            }
            a_stage = a_next;
        }
    }
}

__global__ __launch_bounds__(768) void gemm_bf16_persistent_256x128_kernel(GemmBf16Args p) { gemm_bf16_persistent_body<false>(p); }
__global__ __launch_bounds__(768) void gemm_bf16_persistent_256x128_f32out_kernel(GemmBf16Args p) { gemm_bf16_persistent_body<true>(p); }

// -------------------------------------------------------------------------------------------------
// Skinny kernel (M <= 64, decode-like): HBM-bound on B, so the job is to keep many bytes of B in flight
// on every compute unit.  The grid is (N/128 column strips) × (k-splits); a workgroup streams its
// 64-row k-tiles of B straight into a four-deep LDS ring with buffer_load ... lds (three tiles are always
// in flight), reads them back with the LDS transpose load and feeds 32x32x16 MFMAs whose A operand comes
// from global memory (A is tiny and cache-resident).  Split-k partial sums go to a workspace and are
// added in a fixed order by a second kernel that also applies the epilogue, so results are reproducible.
//
// Ring layout: row k of a tile holds 128 columns = 16 chunks of 16 B; chunk c of row k is stored at chunk
// position c ^ (2 * (k & 3)), which spreads the four rows a transpose read touches over all banks.
// -------------------------------------------------------------------------------------------------
struct SkinnyArgs {
    const uint16_t *A;
    const uint16_t *B;
    float *partial;         // [k_splits][M][N]
    float *C32;
    uint16_t *C16;
    const float *bias;
    const float *residual;
    int M, N, K;
    int tiles_n, k_splits, tiles_per_split;
    float scale;
    int activation;
};

template <int MT, int RING>  // MT row blocks of 32; RING stages
__device__ __forceinline__ void gemm_bf16_skinny_body(const SkinnyArgs &p)
{
    constexpr int BK = 64, BN = 128;
    constexpr int B_BYTES = BK * BN * 2;       // 16 KB
    constexpr int A_BYTES = MT * 32 * BK * 2;  // 4 KB per row block
    constexpr int STAGE = B_BYTES + A_BYTES;
    // Each wavefront issues 4 + MT direct loads per k-tile (the vmcnt immediates below count them).
    extern __shared__ __attribute__((aligned(16))) unsigned char ring[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 31, lh = lane >> 5;
    const int strip = blockIdx.x % p.tiles_n;
    const int split = blockIdx.x / p.tiles_n;
    const int n0 = strip * BN;
    const int tile0 = split * p.tiles_per_split;
    const int tiles = min(p.tiles_per_split, p.K / BK - tile0);
    const int N = p.N, K = p.K;

    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(p.A), 0, static_cast<int>(static_cast<unsigned>(p.M) * static_cast<unsigned>(K) * 2u), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(p.B), 0, static_cast<int>(static_cast<unsigned>(K) * static_cast<unsigned>(N) * 2u), 0x00020000);

    // B: instruction r of wavefront w fills rows (r*4 + w)*4 .. +3 of the stage (16 lanes per row).
    unsigned b_off[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = (r * 4 + wave) * 4 + (lane >> 4);
        const int chunk = (lane & 15) ^ (2 * (row & 3));
        b_off[r] = (static_cast<unsigned>(tile0 * BK + row) * N + n0 + chunk * 8) * 2u;
    }
    // A: instruction mt of wavefront w fills rows mt*32 + w*8 .. +7 (8 lanes per row, 128 B = this tile's 64
    // k-values); chunk q of row r is stored at q ^ ((r >> 1) & 7).  Rows >= M read as zero.
    unsigned a_off[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int row = mt * 32 + wave * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ ((row >> 1) & 7);
        a_off[mt] = (static_cast<unsigned>(row) * K + tile0 * BK + chunk * 8) * 2u;
    }
    const unsigned b_tile_step = static_cast<unsigned>(BK) * N * 2u;
    auto load_tile = [&](int tile, int stage) {
        unsigned char *base = ring + stage * STAGE;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_ptr)(base + (r * 4 + wave) * 1024), 16,
                                                     b_off[r] + tile * b_tile_step, 0, 0, 0);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_ptr)(base + B_BYTES + (mt * 4 + wave) * 1024), 16,
                                                     a_off[mt] + tile * (BK * 2u), 0, 0, 0);
    };

    // Transpose-read addresses: this wavefront owns columns wave*32 .. +31.  Lane roles as in the tiled
    // kernel: i16 supplies row i16/4 and the 8-byte piece i16%4 of a 4×16 block.
    const int i16 = lane & 15, c16 = (lane >> 4) & 1;
    const int piece = wave * 8 + c16 * 4 + (i16 & 3);  // 8-byte piece index within the 128-column row
    unsigned b_read[2];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int row = lh * 8 + half * 4 + (i16 >> 2);
        b_read[half] = row * 256 + (((piece >> 1) ^ (2 * (row & 3))) * 16) + (piece & 1) * 8;
    }
    unsigned a_read[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) a_read[kk] = B_BYTES + li * 128 + (((2 * kk + lh) ^ ((li >> 1) & 7)) & 7) * 16;
    const unsigned ring_address = static_cast<unsigned>(reinterpret_cast<uintptr_t>((lds_void_ptr)ring));

    f32x16 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
        acc[mt] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // Prologue: RING-1 tiles in flight.
#pragma unroll
    for (int i = 0; i < RING - 1; ++i)
        if (i < tiles) load_tile(i, i);
    for (int t = 0; t < tiles; ++t) {
        // Tile t must have landed; the (up to RING-2) tiles requested after it may stay in flight.
        const int newer = min(tiles - 1 - t, RING - 2);
        if (newer >= 2) {
            if constexpr (MT == 1) ST_WAIT_VMCNT(10); else ST_WAIT_VMCNT(12);
        } else if (newer == 1) {
            if constexpr (MT == 1) ST_WAIT_VMCNT(5); else ST_WAIT_VMCNT(6);
        } else {
            ST_WAIT_VMCNT(0);
        }
        // Tile t visible to all; everyone is done with tile t-1, whose stage is refilled next.  A bare s_barrier:
        // __syncthreads() carries a release fence that makes the compiler wait for every load in flight — the ring.
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (t + RING - 1 < tiles) load_tile(t + RING - 1, (t + RING - 1) % RING);
        const unsigned char *stage = ring + (t % RING) * STAGE;
        // The tile's eight transposing reads and the wait for them as one assembly block: the compiler does not know
        // which memory such a read touches and would wait for the whole ring, the tile just requested included,
        // before the first of them.
        bf16x8 fb[4];
        {
            const unsigned a0 = ring_address + (t % RING) * STAGE + b_read[0], a1 = ring_address + (t % RING) * STAGE + b_read[1];
            u32x2 r0, r1, r2, r3, r4, r5, r6, r7;
            asm volatile("ds_read_b64_tr_b16 %0, %8\n"
                         "ds_read_b64_tr_b16 %1, %9\n"
                         "ds_read_b64_tr_b16 %2, %8 offset:4096\n"
                         "ds_read_b64_tr_b16 %3, %9 offset:4096\n"
                         "ds_read_b64_tr_b16 %4, %8 offset:8192\n"
                         "ds_read_b64_tr_b16 %5, %9 offset:8192\n"
                         "ds_read_b64_tr_b16 %6, %8 offset:12288\n"
                         "ds_read_b64_tr_b16 %7, %9 offset:12288\n"
                         "s_waitcnt lgkmcnt(0)"
                         : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3), "=&v"(r4), "=&v"(r5), "=&v"(r6), "=&v"(r7)
                         : "v"(a0), "v"(a1)
                         : "memory");
            auto join = [](u32x2 lo, u32x2 hi) {
                const u32x4 v = {lo[0], lo[1], hi[0], hi[1]};
                return __builtin_bit_cast(bf16x8, v);
            };
            fb[0] = join(r0, r1);
            fb[1] = join(r2, r3);
            fb[2] = join(r4, r5);
            fb[3] = join(r6, r7);
        }
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const bf16x8 fa = *reinterpret_cast<const bf16x8 *>(stage + a_read[kk] + mt * 4096);
                acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb[kk], acc[mt], 0, 0, 0);
            }
        }
    }

    float *dst = p.partial + static_cast<size_t>(split) * p.M * N;
    const int col = n0 + wave * 32 + li;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = mt * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
            if (row < p.M) dst[static_cast<size_t>(row) * N + col] = acc[mt][r];
        }
    // (Letting the workgroup that finishes a strip last add the strip's partial sums, instead of a second launch, was
    // measured and dropped: with device-wide fences around an arrival counter 33 µs, with device-scope stores and
    // loads of the partial sums and no fence 14.2 µs, against 10.8 µs for the two launches at 16×4096×4096 — the 32
    // last workgroups reduce serially what the second launch spreads over the whole chip.)
}

// Plain (non-template) kernel entry points: the host-side stub of a kernel template whose body calls the
// LDS-load builtins is not emitted by this compiler, so the template stays a device function.
__global__ __launch_bounds__(256) void gemm_bf16_skinny32_kernel(SkinnyArgs p) { gemm_bf16_skinny_body<1, 4>(p); }
__global__ __launch_bounds__(256) void gemm_bf16_skinny64_kernel(SkinnyArgs p) { gemm_bf16_skinny_body<2, 3>(p); }

// Adds the k-split partial sums in split order (so the result does not depend on scheduling) and applies
// the epilogue.  One thread per output element; the partials of eight splits are requested together so
// the loads overlap, then added one by one.
__global__ __launch_bounds__(256) void gemm_bf16_skinny_reduce_kernel(SkinnyArgs p)
{
    const size_t plane = static_cast<size_t>(p.M) * p.N;
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= plane) return;
    float value = 0.0f;
    for (int s0 = 0; s0 < p.k_splits; s0 += 8) {
        float part[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) part[j] = (s0 + j < p.k_splits) ? p.partial[(s0 + j) * plane + idx] : 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) value += part[j];
    }
    if (p.scale != 1.0f) value *= p.scale;
    if (p.bias) value += p.bias[idx % p.N];
    if (p.residual) value += p.residual[idx];
    value = apply_activation(value, p.activation);
    if (p.C32) p.C32[idx] = value;
    if (p.C16) p.C16[idx] = f32_to_bf16_rne(value);
}

// The same for many splits of a small plane (64×64×100000 on the general kernel is 195 slices of 4096 values): sixteen
// lanes per output value, lane j adding splits j, j + 16, ... in order, then a butterfly over the sixteen — a fixed
// tree, so still independent of scheduling.
__global__ __launch_bounds__(256) void gemm_bf16_reduce_wide_kernel(SkinnyArgs p)
{
    const size_t plane = static_cast<size_t>(p.M) * p.N;
    const int lane16 = threadIdx.x & 15;
    const size_t idx = static_cast<size_t>(blockIdx.x) * 16 + (threadIdx.x >> 4);
    const bool valid = idx < plane;
    float value = 0.0f;
    for (int s0 = lane16; s0 < p.k_splits; s0 += 128) {
        float part[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) part[j] = (valid && s0 + 16 * j < p.k_splits) ? p.partial[(s0 + 16 * j) * plane + idx] : 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) value += part[j];
    }
#pragma unroll
    for (int offset = 8; offset > 0; offset >>= 1) value += __shfl_xor(value, offset, 16);
    if (!valid || lane16 != 0) return;
    if (p.scale != 1.0f) value *= p.scale;
    if (p.bias) value += p.bias[idx % p.N];
    if (p.residual) value += p.residual[idx];
    value = apply_activation(value, p.activation);
    if (p.C32) p.C32[idx] = value;
    if (p.C16) p.C16[idx] = f32_to_bf16_rne(value);
}

// The split of a skinny problem over workgroups; fills the shape fields of `sk` and returns the bytes of partial sums.
size_t plan_skinny(const GemmBf16Args &args, SkinnyArgs &sk)
{
    sk.M = args.M;
    sk.N = args.N;
    sk.K = args.K;
    sk.tiles_n = args.N / 128;
    const int k_tiles = args.K / 64;
    // Aim for one workgroup per compute unit (16×4096×4096: 10.1 µs with 256 workgroups, 10.7 with 512, 12.1 with
    // 192), but keep at least four k-tiles per split so the partial-sum traffic stays a small fraction of B.
    int splits = (256 + sk.tiles_n - 1) / sk.tiles_n;
    splits = std::max(1, std::min(splits, k_tiles / 4 > 0 ? k_tiles / 4 : 1));
    sk.tiles_per_split = (k_tiles + splits - 1) / splits;
    sk.k_splits = (k_tiles + sk.tiles_per_split - 1) / sk.tiles_per_split;
    return static_cast<size_t>(sk.k_splits) * args.M * args.N * sizeof(float);
}

// `workspace_offset`: bytes at the front of the stream's workspace that the caller is using (an unpacked B).
hipError_t launch_skinny(const GemmBf16Args &args, hipStream_t stream, size_t workspace_offset)
{
    SkinnyArgs sk;
    sk.A = args.A;
    sk.B = args.B;
    const size_t bytes = plan_skinny(args, sk);
    void *workspace = nullptr;
    hipError_t rc = stream_workspace(stream, workspace_offset + bytes, &workspace);  // hipMallocAsync/hipFreeAsync per call cost more than the kernel
    if (rc != hipSuccess) return rc;
    sk.partial = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) + workspace_offset);
    sk.C32 = args.C32;
    sk.C16 = args.C16;
    sk.bias = args.bias;
    sk.residual = args.residual;
    sk.scale = args.scale;
    sk.activation = args.activation;
    const dim3 grid(static_cast<unsigned>(sk.tiles_n * sk.k_splits));
    if (args.M <= 32) {
        constexpr int lds = 4 * (16384 + 4096);
        auto kernel = gemm_bf16_skinny32_kernel;
        rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (rc == hipSuccess) hipLaunchKernelGGL(kernel, grid, dim3(256), lds, stream, sk);
    } else {
        constexpr int lds = 3 * (16384 + 8192);
        auto kernel = gemm_bf16_skinny64_kernel;
        rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (rc == hipSuccess) hipLaunchKernelGGL(kernel, grid, dim3(256), lds, stream, sk);
    }
    if (rc == hipSuccess) rc = hipGetLastError();
    if (rc != hipSuccess) return rc;
    const size_t plane = static_cast<size_t>(args.M) * args.N;
    hipLaunchKernelGGL(gemm_bf16_skinny_reduce_kernel, dim3(static_cast<unsigned>((plane + 255) / 256)), dim3(256), 0, stream,
                       sk);
    return hipGetLastError();
}

// -------------------------------------------------------------------------------------------------
// Skinny kernel for a prepacked B (n×k, k contiguous), M <= 32: one launch, no workspace.
// A workgroup owns 16 columns of C (16 rows of Bᵀ, one contiguous 16·K block of memory); its eight wavefronts split
// K into eight contiguous ranges and each streams its range of Bᵀ and of A through a two-stage ring of its own in
// LDS, so the main loop needs no workgroup barrier.  The 16x16x32 MFMA wants lane (j, g) to hold 8 k-values of row
// j — sixteen rows per quarter-wavefront, which the memory pipeline serves at a fifth of the rate of contiguous
// accesses (measured: 4.7 µs against 0.1 µs beyond the launch for the 32 MiB of a 4096² B) — so the rows go
// global -> LDS with buffer_load ... lds, every quarter-wavefront fetching whole 128-byte lines, and the fragments
// are 128-bit LDS reads.  Chunk c (16 bytes) of row j is stored at position c ^ f(j) of its row (the load applies it
// by choosing which 16 bytes a lane fetches), which spreads the sixteen rows of a fragment read over all banks.
// The eight partial tiles are added through LDS in wavefront order: results do not depend on scheduling.
// -------------------------------------------------------------------------------------------------
typedef float f32x4_acc __attribute__((ext_vector_type(4)));

template <int MT, int STAGE_K>  // MT row blocks of 16; STAGE_K k-values per ring stage (a multiple of 32)
__device__ __forceinline__ void gemm_bf16_skinny_packed_body(const GemmBf16Args &p)
{
    constexpr int WAVES = 8;
    constexpr int ROW_BYTES = STAGE_K * 2;            // bytes of one row in a stage
    constexpr int CPR = ROW_BYTES / 16;               // 16-byte chunks per row
    constexpr int RPI = 1024 / ROW_BYTES;             // rows one load instruction fills
    constexpr int B_LOADS = 16 / RPI;                 // load instructions per stage: Bᵀ rows ...
    constexpr int A_LOADS = MT * 16 / RPI;            // ... and A rows
    constexpr int STAGE_BYTES = (1 + MT) * 16 * ROW_BYTES;
    constexpr int STEPS = STAGE_K / 32;               // MFMA k-steps per stage
    static_assert(CPR == 8 || CPR == 16, "row swizzle is written for 128- and 256-byte rows");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_bytes[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lj = lane & 15, lg = lane >> 4;
    const int M = p.M, N = p.N, K = p.K;
    const int n0 = blockIdx.x * 16;
    unsigned char *ring = lds_bytes + wave * (2 * STAGE_BYTES);
    float *partial = reinterpret_cast<float *>(lds_bytes + WAVES * 2 * STAGE_BYTES);  // [WAVES][MT*16][17]

    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(p.A), 0, static_cast<int>(static_cast<unsigned>(M) * static_cast<unsigned>(K) * 2u), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(p.B), 0, static_cast<int>(static_cast<unsigned>(N) * static_cast<unsigned>(K) * 2u), 0x00020000);

    auto swz = [](int row) { return CPR == 16 ? (row & 15) : ((row ^ (row >> 3)) & 7); };
    // Load instruction i fills rows i*RPI .. +RPI-1 of a stage; lane l writes position l % CPR of row i*RPI + l / CPR.
    constexpr unsigned kOutside = 0x80000000u;  // past the end of any buffer this kernel accepts: the load writes zeros
    unsigned b_off[B_LOADS], a_off[A_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const int row = i * RPI + lane / CPR;
        const int chunk = (lane % CPR) ^ swz(row);
        if (i < B_LOADS) b_off[i] = (static_cast<unsigned>(n0 + row) * K) * 2u + chunk * 16u;
        a_off[i] = row < M ? (static_cast<unsigned>(row) * K) * 2u + chunk * 16u : kOutside;
    }
    auto load_stage = [&](int stage, int slot) {
        unsigned char *base = ring + slot * STAGE_BYTES;
        const unsigned soff = static_cast<unsigned>(stage) * ROW_BYTES;
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_ptr)(base + i * 1024), 16, b_off[i], soff, 0, 0);
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_ptr)(base + 16 * ROW_BYTES + i * 1024), 16, a_off[i], soff, 0, 0);
    };

    const int stages = K / STAGE_K;
    const int per_wave = (stages + WAVES - 1) / WAVES;
    const int first = wave * per_wave;
    const int count = max(0, min(stages, first + per_wave) - first);

    f32x4_acc acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4_acc{0.f, 0.f, 0.f, 0.f};

    if (count > 0) load_stage(first, 0);
    if (count > 1) load_stage(first + 1, 1);
    for (int c = 0; c < count; ++c) {
        // Stage c has landed once at most the B_LOADS + A_LOADS requests of stage c+1 are outstanding.
        if (c + 1 < count) ST_WAIT_VMCNT(B_LOADS + A_LOADS);
        else ST_WAIT_VMCNT(0);
        asm volatile("" ::: "memory");
        const unsigned char *stage = ring + (c & 1) * STAGE_BYTES;
        bf16x8 fb[STEPS], fa[MT][STEPS];
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const int chunk = s * 4 + lg;
            fb[s] = *reinterpret_cast<const bf16x8 *>(stage + lj * ROW_BYTES + ((chunk ^ swz(lj)) << 4));
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int row = mt * 16 + lj;
                fa[mt][s] = *reinterpret_cast<const bf16x8 *>(stage + (16 + row) * ROW_BYTES + ((chunk ^ swz(row)) << 4));
            }
        }
        // The fragments are in registers before the slot is filled again.
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
        asm volatile("" ::: "memory");
        if (c + 2 < count) load_stage(first + c + 2, c & 1);
#pragma unroll
        for (int s = 0; s < STEPS; ++s)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[mt][s], fb[s], acc[mt], 0, 0, 0);
    }

    // Accumulator register i of lane (lj, lg) is C[4·lg + i][lj] of the wavefront's 16×16 block.
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) partial[(wave * MT * 16 + mt * 16 + lg * 4 + i) * 17 + lj] = acc[mt][i];
    __syncthreads();
    with_epilogue_ops(p.activation, p.residual != nullptr, [&](auto &&act, auto has_residual) {
        for (int e = tid; e < MT * 256; e += WAVES * 64) {
            const int row = e >> 4, col = e & 15;
            if (row >= M) continue;
            float value = partial[row * 17 + col];
#pragma unroll
            for (int w = 1; w < WAVES; ++w) value += partial[(w * MT * 16 + row) * 17 + col];
            const size_t idx = static_cast<size_t>(row) * N + n0 + col;
            value = value * p.scale + (p.bias ? p.bias[n0 + col] : -0.0f);
            if constexpr (decltype(has_residual)::value) value += p.residual[idx];
            value = act(value);
            if (p.C32) p.C32[idx] = value;
            if (p.C16) p.C16[idx] = f32_to_bf16_rne(value);
        }
    });
}

__global__ __launch_bounds__(512) void gemm_bf16_skinny_packed16_kernel(GemmBf16Args p) { gemm_bf16_skinny_packed_body<1, 128>(p); }
__global__ __launch_bounds__(512) void gemm_bf16_skinny_packed32_kernel(GemmBf16Args p) { gemm_bf16_skinny_packed_body<2, 64>(p); }

constexpr size_t skinny_packed_lds(int mt, int stage_k) { return 8 * 2 * (1 + mt) * 16 * stage_k * 2 + 8 * mt * 16 * 17 * sizeof(float); }

hipError_t launch_skinny_packed(const GemmBf16Args &args, hipStream_t stream)
{
    const dim3 grid(static_cast<unsigned>(args.N / 16));
    const bool one = args.M <= 16;
    auto kernel = one ? gemm_bf16_skinny_packed16_kernel : gemm_bf16_skinny_packed32_kernel;
    const size_t lds = one ? skinny_packed_lds(1, 128) : skinny_packed_lds(2, 64);
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        static_cast<int>(lds));
    if (rc != hipSuccess) return rc;
    hipLaunchKernelGGL(kernel, grid, dim3(512), lds, stream, args);
    return hipGetLastError();
}

// out(cols×rows) = in(rows×cols)ᵀ for 16-bit elements, 64×64 tiles through LDS, 128-bit global accesses when the
// shape allows (PackedB::from_row_major, crates/st-tensor/src/pure.rs:1299-1316, for bf16 storage).
__global__ __launch_bounds__(256) void transpose_u16_kernel(int rows, int cols, int vec, const uint16_t *in, uint16_t *out)
{
    __shared__ uint16_t tile[64][66];
    const int t = threadIdx.x;
    const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = (t >> 3) + 32 * i, c8 = (t & 7) * 8;
        uint16_t e[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (r0 + r < rows) {
            const uint16_t *src = in + static_cast<size_t>(r0 + r) * cols + c0 + c8;
            if (vec && c0 + c8 + 8 <= cols) {
                *reinterpret_cast<uint4 *>(e) = *reinterpret_cast<const uint4 *>(src);
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (c0 + c8 + j < cols) e[j] = src[j];
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) tile[r][c8 + j] = e[j];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int c = (t >> 3) + 32 * i, r8 = (t & 7) * 8;
        if (c0 + c >= cols) continue;
        uint16_t e[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) e[j] = tile[r8 + j][c];
        uint16_t *dst = out + static_cast<size_t>(c0 + c) * rows + r0 + r8;
        if (vec && r0 + r8 + 8 <= rows) {
            *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(e);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (r0 + r8 + j < rows) dst[j] = e[j];
        }
    }
}

// Few tiles and a long k (a batch of a hundred rows against a 4096² weight is 32 tiles of 64 k-tiles each): split k
// over workgroups.  With few workgroups on the chip a k-tile costs its workgroup about half a microsecond of load
// latency whatever the tile count, so the loop's time is the k-tiles per split; against that stand the partial sums,
// written once and read once, and the reduction's launch.  The split count is the one with the least sum of the three
// (at least two k-tiles per split, at most one workgroup per compute unit).
struct SplitChoice {
    size_t splits;
    double cost_us;
};
// `most_groups`: workgroups the chip holds at a time for this tiling (256 for the 256-row kernels, 512 for 128×128
// tiles); `tile_us`: what a k-tile costs a workgroup of that tiling when few are resident.
SplitChoice estimate_k_splits(size_t m, size_t n, size_t k, size_t tiles, size_t most_groups, double tile_us)
{
    const size_t k_tiles = k / 64;
    const double plane_bytes = static_cast<double>(m) * static_cast<double>(n) * sizeof(float);
    auto cost_us = [&](size_t splits) {
        const double loop = tile_us * static_cast<double>((k_tiles + splits - 1) / splits);
        const double sums = splits > 1 ? 3.0 + static_cast<double>(splits) * plane_bytes * 2.0 / 4.0e6 : 0.0;  // 4 TB/s
        return loop + sums;
    };
    SplitChoice best{1, cost_us(1)};
    if (tiles * 2 > most_groups || k_tiles < 8) return best;
    const size_t most = std::min<size_t>(most_groups / tiles, k_tiles / 2);
    for (size_t splits = 2; splits <= most; ++splits)
        if (cost_us(splits) < best.cost_us) best = SplitChoice{splits, cost_us(splits)};
    // (Measured on m = 33 … 2048 against n, k = 512 … 4096, both layouts of B, against the earlier rule — split as far
    // as the partial sums stay below the operands' bytes, 256-row tiles only: 10 to 35 % faster on most mid-size shapes,
    // e.g. 1024×768×3072 24.5 → 17.7 µs prepacked and 33.1 → 20.3 µs row-major, 512×512×2048 15.3 → 10.2 µs; none
    // slower by more than 3 %.)
    return best;
}
size_t choose_k_splits(size_t m, size_t n, size_t k, size_t tiles) { return estimate_k_splits(m, n, k, tiles, 256, 0.5).splits; }

// The 256-row tiling of an m×n×k product (n a multiple of 128): tile width, tile count and k-splits.
// One workgroup per compute unit at a time: the launch runs in rounds of 256 tiles.  Halving the tile width costs
// about 15 % in the main loop (more LDS traffic per flop), so do it only when it fills rounds that the 256-wide
// tiling would leave partly empty (or when n is not a multiple of 256).
struct TilePlan {
    bool narrow;
    size_t tiles;
    size_t k_splits;
};
TilePlan plan_tiles(size_t m, size_t n, size_t k)
{
    auto fill = [](size_t tiles) { return static_cast<double>(tiles) / static_cast<double>((tiles + 255) / 256 * 256); };
    const size_t row_tiles = (m + 255) / 256;
    // An n that is not a multiple of 128 hangs over the last tile either way; 256-wide tiles then only cost more when
    // they add a whole empty 128-column block to a narrow matrix.
    const size_t cols128 = (n + 127) / 128, cols256 = (n + 255) / 256;
    const bool wide_fits = n % 256 == 0 || (n % 128 != 0 && (cols128 % 2 == 0 || cols128 >= 16));
    TilePlan plan;
    plan.narrow = !wide_fits || fill(row_tiles * cols128) > 1.15 * fill(row_tiles * cols256);
    plan.tiles = row_tiles * (plan.narrow ? cols128 : cols256);
    plan.k_splits = choose_k_splits(m, n, k, plan.tiles);
    return plan;
}

// The launch arithmetic of the tiled kernels whose workgroups decode their index into (k-split, tile), checked on the
// host before every launch: the grid is tiles × k-splits and fits the 32-bit ids the kernels compute with, the tiles
// cover the matrix without an empty row or column of tiles, every split has k-tiles to walk and together they cover K,
// and the XCD remap only runs on a grid it divides.  A plan that fails is an error code, not a launch.
bool tile_launch_consistent(const GemmBf16Args &a, size_t grid, int bm, int bn)
{
    if (a.M <= 0 || a.N <= 0 || a.K < 64 || a.K % 64 != 0 || a.tiles_m <= 0 || a.tiles_n <= 0) return false;
    const size_t tiles = static_cast<size_t>(a.tiles_m) * static_cast<size_t>(a.tiles_n), k_tiles = static_cast<size_t>(a.K) / 64;
    if (grid == 0 || grid > 0x7fffffffu || a.k_splits < 1 || grid != tiles * static_cast<size_t>(a.k_splits)) return false;
    if (static_cast<size_t>(a.tiles_m) * bm < static_cast<size_t>(a.M) || static_cast<size_t>(a.tiles_m - 1) * bm >= static_cast<size_t>(a.M)) return false;
    if (static_cast<size_t>(a.tiles_n) * bn < static_cast<size_t>(a.N) || static_cast<size_t>(a.tiles_n - 1) * bn >= static_cast<size_t>(a.N)) return false;
    if (a.k_splits > 1) {
        const size_t per = static_cast<size_t>(a.tiles_per_split);
        if (a.tiles_per_split < 1 || a.partial == nullptr) return false;
        if (static_cast<size_t>(a.k_splits - 1) * per >= k_tiles || static_cast<size_t>(a.k_splits) * per < k_tiles) return false;
    }
    return !a.swizzle || grid % 8 == 0;
}

// Tiles and k-splits of a 256-row launch (BN columns per tile) filled into `args`; returns the grid.
size_t plan_256(GemmBf16Args &args, int bn)
{
    args.tiles_m = (args.M + 255) / 256;
    args.tiles_n = (args.N + bn - 1) / bn;  // the packed kernels take a ragged N: rows of Bᵀ past it read as zero
    size_t tiles = static_cast<size_t>(args.tiles_m) * static_cast<size_t>(args.tiles_n);
    const size_t k_tiles = static_cast<size_t>(args.K) / 64;
    const size_t splits = choose_k_splits(args.M, args.N, args.K, tiles);
    args.k_splits = 1;
    if (splits > 1) {
        args.tiles_per_split = static_cast<int>((k_tiles + splits - 1) / splits);
        args.k_splits = static_cast<int>((k_tiles + args.tiles_per_split - 1) / args.tiles_per_split);
        tiles *= static_cast<size_t>(args.k_splits);
    }
    args.swizzle = (tiles % 8 == 0) ? 1 : 0;
    return tiles;
}

template <int BN>
hipError_t launch_256(GemmBf16Args args, bool packed, hipStream_t stream, size_t workspace_offset)
{
    const size_t tiles = plan_256(args, BN);
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    SkinnyArgs reduce{};
    if (args.k_splits > 1) {
        const size_t bytes = static_cast<size_t>(args.k_splits) * args.M * args.N * sizeof(float);
        void *workspace = nullptr;
        hipError_t rc = stream_workspace(stream, workspace_offset + bytes, &workspace);
        if (rc != hipSuccess) return rc;
        args.partial = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) + workspace_offset);
        reduce.partial = args.partial;
        reduce.C32 = args.C32;
        reduce.C16 = args.C16;
        reduce.bias = args.bias;
        reduce.residual = args.residual;
        reduce.M = args.M;
        reduce.N = args.N;
        reduce.K = args.K;
        reduce.k_splits = args.k_splits;
        reduce.scale = args.scale;
        reduce.activation = args.activation;
    }
    if (!tile_launch_consistent(args, tiles, 256, BN)) return hipErrorInvalidConfiguration;
    constexpr size_t lds_bytes = 5 * 32768;  // three A stages + two B stages
    static_assert(lds_bytes >= 8 * 32 * (128 + 4) * sizeof(float), "eight epilogue strips must fit in the stage buffers");
    auto kernel = BN == 256 ? (packed ? gemm_bf16_256w8_packed_kernel : gemm_bf16_256rm_kernel)
                            : (packed ? gemm_bf16_256x128w8_packed_kernel : gemm_bf16_256x128rm_kernel);
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(tiles)), dim3(512), lds_bytes, stream, args);
    rc = hipGetLastError();
    if (rc != hipSuccess || args.k_splits == 1) return rc;
    const size_t plane = static_cast<size_t>(args.M) * args.N;
    hipLaunchKernelGGL(gemm_bf16_skinny_reduce_kernel, dim3(static_cast<unsigned>((plane + 255) / 256)), dim3(256), 0, stream,
                       reduce);
    return hipGetLastError();
}

hipError_t launch_128(GemmBf16Args args, bool packed, hipStream_t stream, size_t splits = 1, size_t workspace_offset = 0)
{
    args.tiles_m = (args.M + 127) / 128;
    args.tiles_n = (args.N + 127) / 128;
    size_t tiles = static_cast<size_t>(args.tiles_m) * static_cast<size_t>(args.tiles_n);
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    SkinnyArgs reduce{};
    if (splits > 1) {
        const size_t k_tiles = static_cast<size_t>(args.K) / 64;
        args.tiles_per_split = static_cast<int>((k_tiles + splits - 1) / splits);
        args.k_splits = static_cast<int>((k_tiles + args.tiles_per_split - 1) / args.tiles_per_split);
        const size_t bytes = static_cast<size_t>(args.k_splits) * args.M * args.N * sizeof(float);
        void *workspace = nullptr;
        hipError_t ws = stream_workspace(stream, workspace_offset + bytes, &workspace);
        if (ws != hipSuccess) return ws;
        args.partial = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) + workspace_offset);
        reduce.partial = args.partial;
        reduce.C32 = args.C32;
        reduce.C16 = args.C16;
        reduce.bias = args.bias;
        reduce.residual = args.residual;
        reduce.M = args.M;
        reduce.N = args.N;
        reduce.K = args.K;
        reduce.k_splits = args.k_splits;
        reduce.scale = args.scale;
        reduce.activation = args.activation;
        tiles *= static_cast<size_t>(args.k_splits);
    }
    args.swizzle = (tiles % 8 == 0) ? 1 : 0;
    if (!tile_launch_consistent(args, tiles, 128, 128)) return hipErrorInvalidConfiguration;
    constexpr size_t lds_bytes = 5 * 16384;  // three A stages + two B stages of 128 rows
    static_assert(lds_bytes >= 4 * 32 * (64 + 4) * sizeof(float), "four epilogue strips must fit in the stage buffers");
    auto kernel = packed ? gemm_bf16_128x128w4_packed_kernel : gemm_bf16_128x128w4_rm_kernel;
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(tiles)), dim3(256), lds_bytes, stream, args);
    rc = hipGetLastError();
    if (rc != hipSuccess || args.k_splits == 1) return rc;
    const size_t plane = static_cast<size_t>(args.M) * args.N;
    hipLaunchKernelGGL(gemm_bf16_skinny_reduce_kernel, dim3(static_cast<unsigned>((plane + 255) / 256)), dim3(256), 0, stream,
                       reduce);
    return hipGetLastError();
}

// The persistent kernel: one workgroup per compute unit (fewer when there are fewer tiles), twelve wavefronts each.
hipError_t launch_persistent_256x128(GemmBf16Args args, hipStream_t stream)
{
    args.tiles_m = args.M / 256;
    args.tiles_n = args.N / 128;
    const size_t tiles = static_cast<size_t>(args.tiles_m) * static_cast<size_t>(args.tiles_n);
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    const unsigned grid = static_cast<unsigned>(std::min<size_t>(tiles, 256));
    args.swizzle = (tiles % 8 == 0 && grid % 8 == 0) ? 1 : 0;
    // whole tiles only (the epilogues store without row or column checks), no k-splits, and a walk every workgroup ends
    if (args.M % 256 != 0 || args.N % 128 != 0 || args.K < 64 || args.K % 64 != 0 || args.k_splits != 1 || grid == 0)
        return hipErrorInvalidConfiguration;
    constexpr size_t lds_bytes = 3 * 32768 + 2 * 16384 + 32768;  // three A stages, two B stages, strips of four wavefronts
    auto kernel = args.C32 ? gemm_bf16_persistent_256x128_f32out_kernel : gemm_bf16_persistent_256x128_kernel;
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(768), lds_bytes, stream, args);
    return hipGetLastError();
}

hipError_t launch_rowcomplete(const RowLnArgs &args, hipStream_t stream)
{
    constexpr size_t lds_bytes = 3 * 64 * 128 + 2 * 512 * 128;  // three A stages + two B stages
    static_assert(lds_bytes >= 8 * 32 * (128 + 4) * sizeof(float) + 64 * 4 * 2 * sizeof(float), "epilogue strips and row statistics");
    auto kernel = gemm_bf16_rowcomplete_kernel;
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    const size_t tiles = (static_cast<size_t>(args.g.M) + 63) / 64;
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(tiles)), dim3(512), lds_bytes, stream, args);
    return hipGetLastError();
}

// k-slices of the general tile kernel (128×128 tiles, 32-wide k-tiles): none while the tiles alone give every other
// compute unit a workgroup; otherwise enough for about two workgroups per compute unit, each slice keeping at least 16
// k-tiles, and the partial planes (written once, read once, f32) staying below the operands' bytes.
size_t general_k_slices(size_t m, size_t n, size_t k)
{
    const size_t tiles = ((m + 127) / 128) * ((n + 127) / 128), k_steps = (k + 31) / 32;
    if (tiles > 128 || k_steps < 32) return 1;
    size_t slices = std::min<size_t>(512 / tiles, k_steps / 16);
    while (slices > 1 && slices * m * n * 8 > (m * k + k * n) * 2) --slices;
    return std::max<size_t>(slices, 1);
}
size_t general_slice_bytes(size_t m, size_t n, size_t k)
{
    const size_t slices = general_k_slices(m, n, k);
    return slices > 1 ? slices * m * n * sizeof(float) : 0;
}

// `workspace_offset`: bytes at the front of the stream's workspace that the caller is using (an unpacked B).
template <int BM, int BN, int BK>
hipError_t launch_tile(GemmBf16Args args, bool vec, hipStream_t stream, size_t workspace_offset)
{
    static_assert(BM == 128 && BN == 128 && BK == 32, "general_k_slices plans for this tiling");
    args.tiles_m = (args.M + BM - 1) / BM;
    args.tiles_n = (args.N + BN - 1) / BN;
    const size_t tiles = static_cast<size_t>(args.tiles_m) * static_cast<size_t>(args.tiles_n);
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    args.swizzle = (tiles % 8 == 0) ? 1 : 0;
    constexpr size_t lds_bytes = 2 * (static_cast<size_t>(BM) * (BK + 8) + static_cast<size_t>(BK) * (BN + 32)) * 2;
    const size_t slices = general_k_slices(args.M, args.N, args.K);
    SkinnyArgs reduce{};
    if (slices > 1) {
        const size_t k_steps = (static_cast<size_t>(args.K) + BK - 1) / BK;
        args.tiles_per_split = static_cast<int>((k_steps + slices - 1) / slices);
        args.k_splits = static_cast<int>((k_steps + args.tiles_per_split - 1) / args.tiles_per_split);
        void *workspace = nullptr;
        hipError_t ws = stream_workspace(stream, workspace_offset + slices * args.M * static_cast<size_t>(args.N) * sizeof(float),
                                         &workspace);
        if (ws != hipSuccess) return ws;
        reduce.partial = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) + workspace_offset);
        reduce.C32 = args.C32;
        reduce.C16 = args.C16;
        reduce.bias = args.bias;
        reduce.residual = args.residual;
        reduce.M = args.M;
        reduce.N = args.N;
        reduce.K = args.K;
        reduce.k_splits = args.k_splits;
        reduce.scale = args.scale;
        reduce.activation = args.activation;
        args.C32 = reduce.partial;
        args.C16 = nullptr;
        args.bias = nullptr;
        args.residual = nullptr;
        args.scale = 1.0f;
        args.activation = ST_HIP_ACT_NONE;
    }
    const dim3 grid(static_cast<unsigned>(tiles), static_cast<unsigned>(args.k_splits));
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
    rc = hipGetLastError();
    if (rc != hipSuccess || args.k_splits == 1) return rc;
    const size_t plane = static_cast<size_t>(args.M) * args.N;
    if (args.k_splits >= 32 && plane <= 65536)
        hipLaunchKernelGGL(gemm_bf16_reduce_wide_kernel, dim3(static_cast<unsigned>((plane + 15) / 16)), dim3(256), 0, stream, reduce);
    else
        hipLaunchKernelGGL(gemm_bf16_skinny_reduce_kernel, dim3(static_cast<unsigned>((plane + 255) / 256)), dim3(256), 0, stream,
                           reduce);
    return hipGetLastError();
}

bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

// Copies rows × cols matrices of 16-bit values into rows_pad × cols_pad ones, zeros in the new rows and columns: two
// matrices (the operands of a product) in one launch, the first `first_blocks` workgroups on the first.  A thread
// moves eight adjacent values of one output row (16-byte accesses at any alignment).
struct PadJob {
    const uint16_t *in;
    uint16_t *out;
    unsigned rows, cols, rows_pad, cols_pad;
};

__global__ __launch_bounds__(256) void pad_u16_pair_kernel(PadJob first, PadJob second, unsigned first_blocks)
{
    typedef uint32_t pad_u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
    const bool is_first = blockIdx.x < first_blocks;
    const PadJob &job = is_first ? first : second;
    const unsigned chunks = (job.cols_pad + 7) / 8;
    const unsigned idx = (blockIdx.x - (is_first ? 0u : first_blocks)) * 256u + threadIdx.x;  // below 2^28: the copies are below 2 GiB
    const unsigned r = idx / chunks;
    const unsigned c0 = (idx - r * chunks) * 8;
    if (r >= job.rows_pad) return;
    uint16_t *dst = job.out + static_cast<size_t>(r) * job.cols_pad + c0;
    const uint16_t *src = job.in + static_cast<size_t>(r) * job.cols + c0;
    if (r < job.rows && c0 + 8 <= job.cols) {
        *reinterpret_cast<pad_u32x4_a2 *>(dst) = *reinterpret_cast<const pad_u32x4_a2 *>(src);
        return;
    }
#pragma unroll
    for (unsigned e = 0; e < 8; ++e) {
        const unsigned c = c0 + e;
        if (c < job.cols_pad) dst[e] = (r < job.rows && c < job.cols) ? src[e] : static_cast<uint16_t>(0);
    }
}

PadJob pad_job(size_t rows, size_t cols, size_t rows_pad, size_t cols_pad, const uint16_t *in, uint16_t *out)
{
    return PadJob{in, out, static_cast<unsigned>(rows), static_cast<unsigned>(cols), static_cast<unsigned>(rows_pad),
                  static_cast<unsigned>(cols_pad)};
}

hipError_t launch_pad_u16_pair(const PadJob &first, const PadJob &second, hipStream_t stream)
{
    auto blocks = [](const PadJob &job) {
        return static_cast<unsigned>((static_cast<size_t>(job.rows_pad) * ((job.cols_pad + 7) / 8) + 255) / 256);
    };
    const unsigned first_blocks = blocks(first), all = first_blocks + blocks(second);
    if (all == 0) return hipSuccess;
    hipLaunchKernelGGL(pad_u16_pair_kernel, dim3(all), dim3(256), 0, stream, first, second, first_blocks);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_transpose_u16(size_t rows, size_t cols, const uint16_t *in, uint16_t *out, hipStream_t stream)
{
    if (rows == 0 || cols == 0) return hipSuccess;
    const int vec = rows % 8 == 0 && cols % 8 == 0 && aligned16(in) && aligned16(out) ? 1 : 0;
    const dim3 grid(static_cast<unsigned>((cols + 63) / 64), static_cast<unsigned>((rows + 63) / 64));
    hipLaunchKernelGGL(transpose_u16_kernel, grid, dim3(256), 0, stream, static_cast<int>(rows), static_cast<int>(cols), vec,
                       in, out);
    return hipGetLastError();
}

hipError_t launch_gemm_bf16(size_t m, size_t n, size_t k, const uint16_t *lhs, const uint16_t *rhs,
                            float *out_f32, uint16_t *out_bf16, const GemmEpilogue &epilogue,
                            hipStream_t stream, bool rhs_packed)
{
    if (m == 0 || n == 0) return hipSuccess;
    if (gemv_bf16_applies(m, n, k, lhs, rhs))
        return launch_gemv_bf16(m, n, k, lhs, rhs, rhs_packed, out_f32, out_bf16, epilogue, stream);
    // An A of 2 GiB or more (the 256-row kernels address their operands through 32-bit byte offsets): row blocks of A
    // are independent products, so the launch is cut into blocks that fit and each takes the fast path.
    if (m * k * sizeof(uint16_t) >= (1ull << 31) && gemm_row_block(k, sizeof(uint16_t)) > 0) {
        const size_t block = gemm_row_block(k, sizeof(uint16_t));
        for (size_t row = 0; row < m; row += block) {
            const size_t rows = std::min(block, m - row);
            GemmEpilogue part = epilogue;
            if (part.residual) part.residual += row * n;
            const hipError_t rc = launch_gemm_bf16(rows, n, k, lhs + row * k, rhs, out_f32 ? out_f32 + row * n : nullptr,
                                                   out_bf16 ? out_bf16 + row * n : nullptr, part, stream, rhs_packed);
            if (rc != hipSuccess) return rc;
        }
        return hipSuccess;
    }
    // A k that is not a multiple of 64 (784 inputs, 1000 features): the direct-to-LDS kernels take whole 64-wide k-tiles
    // only, and the general kernel runs such a product at half their speed (8192×4096×1000: 141 µs against 65 µs at
    // k = 1024).  Where the product is large against its operands, zero-padded copies of A and B along k (exact: the
    // new terms are 0·0) go into the stream's second scratch buffer, one launch for both, and the product runs on them.
    if (k % 64 != 0 && k > 64 && m >= 128 && n >= 128 && 2.0 * m * n * k >= 2e9 && m * (k + 64) * sizeof(uint16_t) < (1ull << 31) &&
        (k + 64) * n * sizeof(uint16_t) < (1ull << 31)) {
        const size_t k_pad = (k + 63) / 64 * 64;
        const size_t a_bytes = (m * k_pad * sizeof(uint16_t) + 255) & ~static_cast<size_t>(255);
        void *copies = nullptr;
        hipError_t rc = stream_workspace_slot(stream, 1, a_bytes + k_pad * n * sizeof(uint16_t), &copies);
        if (rc != hipSuccess) return rc;
        uint16_t *a_pad = static_cast<uint16_t *>(copies);
        uint16_t *b_pad = reinterpret_cast<uint16_t *>(static_cast<unsigned char *>(copies) + a_bytes);
        rc = launch_pad_u16_pair(pad_job(m, k, m, k_pad, lhs, a_pad),
                                 rhs_packed ? pad_job(n, k, n, k_pad, rhs, b_pad) : pad_job(k, n, k_pad, n, rhs, b_pad), stream);
        if (rc != hipSuccess) return rc;
        return launch_gemm_bf16(m, n, k_pad, a_pad, b_pad, out_f32, out_bf16, epilogue, stream, rhs_packed);
    }
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
    // The 256-tile kernel addresses its operands through 32-bit buffer offsets and reads bias/residual/output
    // in 16-byte pieces.
    const bool fits_buffer = m * k * 2 < (1ull << 31) && k * n * 2 < (1ull << 31);
    const bool epilogue_aligned = aligned16(out_f32) && aligned16(epilogue.bias) && aligned16(epilogue.residual) &&
                                  (reinterpret_cast<uintptr_t>(out_bf16) & 7u) == 0;
    const bool fits_256 = vec && k >= 64 && k % 64 == 0 && n % 128 == 0 && fits_buffer && epilogue_aligned;
    // (A prepacked B the 256-row kernels take stays with them, split over k: unpacking it for the skinny kernel is a
    // pass over B per call — 33×4096×4096: 27.9 µs that way, 13.8 µs this way.)
    const bool skinny = m <= 64 && vec && k >= 256 && k % 64 == 0 && n % 128 == 0 && fits_buffer && !(rhs_packed && fits_256);
    // Decode-like shapes on a prepacked B with enough 16-column strips to occupy the chip: one launch, no workspace.
    if (rhs_packed && m <= 32 && k >= 128 && k % 128 == 0 && n % 16 == 0 && n / 16 >= 64 && aligned16(lhs) && aligned16(rhs) &&
        fits_buffer)
        return launch_skinny_packed(args, stream);
    size_t workspace_offset = 0;
    // An n that is not a multiple of 128 (a vocabulary of 50257, 1000 classes) with a k the 256-row kernels take: the
    // packed kernels run it as it is — rows of Bᵀ past n read as zero through the buffer range check, and the epilogue
    // for a ragged n stores at any alignment.  A row-major B is packed into the stream's workspace first (one pass
    // over B, a few per cent of such a product) — its rows start at odd addresses, which the direct-to-LDS loads do
    // not take.  (4096×50257×768: 3455 µs on the general kernel.)
    if (n % 128 != 0 && n > 128 && m > 64 && k >= 64 && k % 64 == 0 && aligned16(lhs) && fits_buffer &&
        (!rhs_packed || aligned16(rhs))) {
        const TilePlan plan = plan_tiles(m, n, k);
        if (!rhs_packed) {
            workspace_offset = (k * n * sizeof(uint16_t) + 255) & ~static_cast<size_t>(255);
            const size_t behind = plan.k_splits > 1 ? plan.k_splits * m * n * sizeof(float) : 0;
            void *workspace = nullptr;
            hipError_t rc = stream_workspace(stream, workspace_offset + behind, &workspace);
            if (rc != hipSuccess) return rc;
            rc = launch_transpose_u16(k, n, rhs, static_cast<uint16_t *>(workspace), stream);
            if (rc != hipSuccess) return rc;
            args.B = static_cast<const uint16_t *>(workspace);
        }
        const size_t tiles_128 = ((m + 127) / 128) * ((n + 127) / 128);
        if (plan.tiles < 192 && tiles_128 >= 2 * plan.tiles && plan.k_splits == 1) return launch_128(args, true, stream);
        if (plan.narrow) return launch_256<128>(args, true, stream, workspace_offset);
        return launch_256<256>(args, true, stream, workspace_offset);
    }
    if (rhs_packed && (!fits_256 || skinny) && k > 0) {
        // Shapes the packed 256-row kernels do not take: unpack B into the front of the stream's workspace (sized for
        // the skinny kernel's partial sums behind it as well, so that it does not move) and go on with B as k×n.
        workspace_offset = (k * n * sizeof(uint16_t) + 255) & ~static_cast<size_t>(255);
        SkinnyArgs probe;
        const size_t behind = skinny ? plan_skinny(args, probe) : fits_256 ? 0 : general_slice_bytes(m, n, k);
        void *workspace = nullptr;
        hipError_t rc = stream_workspace(stream, workspace_offset + behind, &workspace);
        if (rc != hipSuccess) return rc;
        rc = launch_transpose_u16(n, k, rhs, static_cast<uint16_t *>(workspace), stream);
        if (rc != hipSuccess) return rc;
        args.B = static_cast<const uint16_t *>(workspace);
        rhs_packed = false;
    }
    if (skinny) return launch_skinny(args, stream, workspace_offset);
    // The 256-row kernels serve every shape they can address: measured against the 128×128 tile kernel they win
    // from a single tile up (256×256×4096: 58 vs 74 µs; 1024³: 21 vs 30 µs; 16384×256×512: 17 vs 24 µs).
    if (fits_256) {
        const TilePlan plan = plan_tiles(m, n, k);
        const bool narrow = plan.narrow;
        // A 256-row tiling that would leave most compute units without a tile, and a k not worth splitting: 128×128
        // tiles, two workgroups per compute unit (1024³: 16 tiles of 256×256, 64 of 128×128).
        const size_t tiles_256 = plan.tiles;
        const size_t tiles_128 = ((m + 127) / 128) * (n / 128);
        if (tiles_256 < 192 && tiles_128 >= 2 * tiles_256) {
            // Either tiling may split k; the smaller tiles need fewer splits (less partial-sum traffic) for the same
            // number of workgroups, and two of their workgroups share a compute unit.
            const SplitChoice big = estimate_k_splits(m, n, k, tiles_256, 256, 0.5);
            const SplitChoice small = estimate_k_splits(m, n, k, tiles_128, 512, 0.42);
            if (small.cost_us <= big.cost_us) return launch_128(args, rhs_packed, stream, small.splits, workspace_offset);
        }
        // Several rounds of 256×128 tiles with bf16 as the only output (the QKV projection of a transformer block):
        // the persistent kernel, whose stores drain under the next tile's main loop (16384×1536×512: 34.1 µs against
        // 36.8).  Where the plan is 256×256 tiles they stay ahead (16384×2048×512: 48.2 µs against 51.8).
        if (narrow && rhs_packed && out_f32 == nullptr && out_bf16 != nullptr && aligned16(out_bf16) && epilogue.residual == nullptr &&
            m % 256 == 0 && (m / 256) * (n / 128) > 256 && m * n * 2 < (1ull << 31))
            return launch_persistent_256x128(args, stream);
        // f32 as the only output, a short k and at least four rounds of 256×128 tiles: the same kernel with an f32
        // epilogue — a tile's stores drain under the next tile's main loop (16384×4096×512: 89 µs against 95).  With a
        // long k the 256×256 tiles' main loop (a third less LDS traffic per flop) is worth more than the overlap: 4096³
        // as 512 tiles of 256×128, two per workgroup, measured 115.6 µs here against 110.0 µs, 8192×8192×4096 483 against
        // 433 µs, and 4096×4096×1024 42.8 against 38.5 µs.
        if (rhs_packed && out_f32 != nullptr && out_bf16 == nullptr && epilogue.residual == nullptr && m % 256 == 0 &&
            k <= 512 && (m / 256) * (n / 128) >= 1024 && m * n * 4 < (1ull << 32))
            return launch_persistent_256x128(args, stream);
        if (narrow) return launch_256<128>(args, rhs_packed, stream, workspace_offset);
        return launch_256<256>(args, rhs_packed, stream, workspace_offset);
    }
    return launch_tile<128, 128, 32>(args, vec, stream, workspace_offset);
}

// The 256-row tiling launch_gemm_bf16 would use for an m×n×k product (k a multiple of 64, n of 128, 16-byte aligned
// operands), with the launcher's own consistency check evaluated on it: what st_hip_gemm_bf16_tile_plan reports.
GemmTilePlanReport gemm_bf16_tile_plan_report(size_t m, size_t n, size_t k)
{
    GemmTilePlanReport report{};
    if (m == 0 || n == 0 || k < 64 || k % 64 != 0 || m > 0x7fffffffu || n > 0x7fffffffu || k > 0x7fffffffu) return report;
    const TilePlan plan = plan_tiles(m, n, k);
    GemmBf16Args args{};
    args.M = static_cast<int>(m);
    args.N = static_cast<int>(n);
    args.K = static_cast<int>(k);
    const int bn = plan.narrow ? 128 : 256;
    const size_t grid = plan_256(args, bn);
    static float placeholder;
    if (args.k_splits > 1) args.partial = &placeholder;  // the launcher points this at scratch memory
    report.tile_cols = bn;
    report.tiles_m = args.tiles_m;
    report.tiles_n = args.tiles_n;
    report.k_splits = args.k_splits;
    report.k_tiles_per_split = args.k_splits > 1 ? args.tiles_per_split : static_cast<int>(k / 64);
    report.workgroups = grid;
    report.consistent = tile_launch_consistent(args, grid, 256, bn) ? 1 : 0;
    // every (split, tile) a workgroup decodes to, walked the way the kernels decode it
    const size_t tiles = static_cast<size_t>(args.tiles_m) * args.tiles_n;
    if (grid <= (1u << 24)) {
        std::vector<unsigned char> seen(grid, 0);
        for (size_t block = 0; block < grid; ++block) {
            size_t logical = block;
            if (args.swizzle) logical = (block & 7) * (grid >> 3) + (block >> 3);
            const size_t split = logical / tiles, rest = logical - split * tiles;
            const size_t width = 4 * static_cast<size_t>(args.tiles_n), group = rest / width, first_m = group * 4;
            const size_t group_size = std::min<size_t>(args.tiles_m - first_m, 4);
            const size_t tile_m = first_m + (rest % width) % group_size, tile_n = (rest % width) / group_size;
            const size_t first_k = split * static_cast<size_t>(args.tiles_per_split);
            const bool inside = split < static_cast<size_t>(args.k_splits) && tile_m < static_cast<size_t>(args.tiles_m) &&
                                tile_n < static_cast<size_t>(args.tiles_n) && tile_m * 256 < m && tile_n * bn < n && first_k < k / 64;
            if (!inside) {
                ++report.out_of_range;
                continue;
            }
            unsigned char &cell = seen[(split * args.tiles_m + tile_m) * args.tiles_n + tile_n];
            if (cell) ++report.duplicates; else ++report.items;
            cell = 1;
        }
    }
    return report;
}

// bf16 convolution as an implicit GEMM on the packed kernels' machinery (crates/st-nn/src/layers/conv.rs:685-748,
// 2559-2599 on bf16 operands): the images are copied once into a zero-padded channels-last layout, in which the 64
// channels of one tap of one output pixel are 128 contiguous bytes — one row of a 64-wide k-tile, fetched straight into
// LDS like a row of a prepacked B — and the weights are re-laid to match (k ordered tap-major).  No patch matrix.
size_t conv2d_bf16_workspace_bytes(const ConvShape &c)
{
    const size_t c_pad = (static_cast<size_t>(c.c_in) + 63) / 64 * 64;
    const size_t hp = static_cast<size_t>(c.h) + 2 * c.pad_h, wp = static_cast<size_t>(c.w) + 2 * c.pad_w;
    const size_t image_bytes = (static_cast<size_t>(c.batch) * hp * wp * c_pad * 2 + 255) & ~static_cast<size_t>(255);
    return image_bytes + static_cast<size_t>(c.c_out) * c.kh * c.kw * c_pad * 2;
}

bool conv2d_bf16_supported(const ConvShape &c)
{
    if (c.batch <= 0 || c.c_out <= 0 || c.oh <= 0 || c.ow <= 0) return true;  // nothing to compute
    const size_t c_pad = (static_cast<size_t>(c.c_in) + 63) / 64 * 64;
    const size_t hp = static_cast<size_t>(c.h) + 2 * c.pad_h, wp = static_cast<size_t>(c.w) + 2 * c.pad_w;
    const size_t image_bytes = static_cast<size_t>(c.batch) * hp * wp * c_pad * 2;
    const size_t k = static_cast<size_t>(c.kh) * c.kw * c_pad;
    const size_t pixels = static_cast<size_t>(c.batch) * c.oh * c.ow;
    // 32-bit byte offsets into both operands, 32-bit pixel and tile counts
    return image_bytes < (1ull << 31) && static_cast<size_t>(c.c_out) * k * 2 < (1ull << 31) && pixels < (1ull << 31) &&
           k < (1ull << 31);
}

hipError_t launch_conv2d_bf16(const ConvShape &c, int activation, const uint16_t *input, const uint16_t *weight, const float *bias,
                              float *out_f32, uint16_t *out_bf16, hipStream_t stream)
{
    if (c.batch <= 0 || c.c_out <= 0 || c.oh <= 0 || c.ow <= 0) return hipSuccess;
    if (!conv2d_bf16_supported(c)) return hipErrorInvalidValue;
    const int c_pad = (c.c_in + 63) / 64 * 64;
    const int hp = c.h + 2 * c.pad_h, wp = c.w + 2 * c.pad_w;
    const int taps = c.kh * c.kw;
    const size_t image_bytes = (static_cast<size_t>(c.batch) * hp * wp * c_pad * 2 + 255) & ~static_cast<size_t>(255);
    void *workspace = nullptr;
    hipError_t rc = stream_workspace(stream, conv2d_bf16_workspace_bytes(c), &workspace);
    if (rc != hipSuccess) return rc;
    uint16_t *images = static_cast<uint16_t *>(workspace);
    uint16_t *weights = reinterpret_cast<uint16_t *>(static_cast<unsigned char *>(workspace) + image_bytes);
    ConvBf16Relayout relayout;
    relayout.in = input;
    relayout.out = images;
    relayout.weight_in = weight;
    relayout.weight_out = weights;
    relayout.batch = c.batch;
    relayout.c_in = c.c_in;
    relayout.h = c.h;
    relayout.w = c.w;
    relayout.c_pad = c_pad;
    relayout.hp = hp;
    relayout.wp = wp;
    relayout.pad_h = c.pad_h;
    relayout.pad_w = c.pad_w;
    relayout.c_out = c.c_out;
    relayout.taps = taps;
    // one launch: a workgroup per (channel block, padded row, image), then one per 1024 weight values
    const size_t image_blocks = static_cast<size_t>(c_pad / 64) * hp * c.batch;
    const size_t weight_blocks = (static_cast<size_t>(c.c_out) * taps * c_pad + 1023) / 1024;
    if (image_blocks + weight_blocks > 0x7fffffffu) return hipErrorInvalidConfiguration;
    relayout.image_blocks = static_cast<unsigned>(image_blocks);
    hipLaunchKernelGGL(conv_bf16_relayout_kernel, dim3(static_cast<unsigned>(image_blocks + weight_blocks)), dim3(256), 0, stream, relayout);
    rc = hipGetLastError();
    if (rc != hipSuccess) return rc;

    GemmBf16Args args;
    args.A = weights;
    args.B = images;
    args.C32 = out_f32;
    args.C16 = out_bf16;
    args.bias = bias;
    args.residual = nullptr;
    args.M = c.c_out;
    args.N = static_cast<int>(static_cast<size_t>(c.batch) * c.oh * c.ow);
    args.K = taps * c_pad;
    args.scale = 1.0f;
    args.activation = activation;
    args.conv.ohow = c.oh * c.ow;
    args.conv.ow = c.ow;
    args.conv.hp = hp;
    args.conv.wp = wp;
    args.conv.c_pad = c_pad;
    args.conv.stride_h = c.stride_h;
    args.conv.stride_w = c.stride_w;
    args.conv.dil_h = c.dil_h;
    args.conv.dil_w = c.dil_w;
    args.conv.kw = c.kw;
    args.conv.c_blocks = c_pad / 64;
    args.conv.c_out = c.c_out;
    args.conv.image_bytes = static_cast<unsigned>(static_cast<size_t>(c.batch) * hp * wp * c_pad * 2);
    // Tiles: 256 channels where the layer has them, 128 otherwise; 256 pixels wide only when that still gives every
    // compute unit a tile.
    const bool tall = c.c_out > 128;
    const size_t tiles_m = (static_cast<size_t>(c.c_out) + (tall ? 255 : 127)) / (tall ? 256 : 128);
    const bool wide = tall && tiles_m * ((static_cast<size_t>(args.N) + 255) / 256) >= 256;
    const size_t bn = wide ? 256 : 128;
    args.tiles_m = static_cast<int>(tiles_m);
    args.tiles_n = static_cast<int>((static_cast<size_t>(args.N) + bn - 1) / bn);
    const size_t tiles = static_cast<size_t>(args.tiles_m) * args.tiles_n;
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    args.swizzle = (tiles % 8 == 0) ? 1 : 0;
    if (!tile_launch_consistent(args, tiles, tall ? 256 : 128, static_cast<int>(bn))) return hipErrorInvalidConfiguration;
    auto kernel = !tall ? conv2d_bf16_128x128w4_kernel : wide ? conv2d_bf16_256x256w8_kernel : conv2d_bf16_256x128w8_kernel;
    const size_t lds_bytes = tall ? 5 * 32768 : 5 * 16384;
    rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(tiles)), dim3(tall ? 512 : 256), lds_bytes, stream, args);
    return hipGetLastError();
}

// out_f32 = (lhs·rhs + bias) + residual, out_ln = layer_norm(out_f32; gamma, beta, epsilon) rounded to bf16; rhs packed n×k.
// n = 512 with k a multiple of 64 up to 1024 and 16-byte aligned operands runs as ONE kernel (the row-complete GEMM above with the
// normalisation in its epilogue); every other shape as the GEMM followed by the layer-norm kernel.
hipError_t launch_gemm_bf16_residual_layer_norm(size_t m, size_t n, size_t k, const uint16_t *lhs, const uint16_t *packed_rhs,
                                                const float *bias, const float *residual, const float *gamma, const float *beta,
                                                float epsilon, float *out_f32, uint16_t *out_ln, hipStream_t stream)
{
    if (m == 0 || n == 0) return hipSuccess;
    const bool fits_buffer = m * k * 2 < (1ull << 31) && k * n * 2 < (1ull << 31);
    const bool aligned = aligned16(lhs) && aligned16(packed_rhs) && aligned16(bias) && aligned16(residual) && aligned16(gamma) &&
                         aligned16(beta) && aligned16(out_f32) && (reinterpret_cast<uintptr_t>(out_ln) & 7u) == 0;
    // Measured at m = 16384 (one 64-row workgroup per compute unit): 27.3 µs against 18.2 + 10.2 µs for the two kernels at
    // k = 512, 51.2 against 37.9 + 10.1 µs at k = 2048 — a 64-row tile streams the whole of B through every compute unit,
    // which costs more than the saved pass over the rows once k is long.
    // (m <= 64 stays with the GEMM dispatcher, which splits k over the chip for such shapes, and so does every shape of
    // few row tiles and a long k that the dispatcher would split: the split sums add up in another order.)
    if (n == 512 && m > 64 && k >= 64 && k % 64 == 0 && k <= 1024 && fits_buffer && aligned && plan_tiles(m, n, k).k_splits == 1) {
        RowLnArgs row;
        row.g.A = lhs;
        row.g.B = packed_rhs;
        row.g.C32 = out_f32;
        row.g.C16 = nullptr;
        row.g.bias = bias;
        row.g.residual = residual;
        row.g.M = static_cast<int>(m);
        row.g.N = static_cast<int>(n);
        row.g.K = static_cast<int>(k);
        row.g.tiles_m = row.g.tiles_n = 0;
        row.g.swizzle = 0;
        row.g.scale = 1.0f;
        row.g.activation = ST_HIP_ACT_NONE;
        row.gamma = gamma;
        row.beta = beta;
        row.epsilon = epsilon;
        row.ln_bf16 = out_ln;
        return launch_rowcomplete(row, stream);
    }
    GemmEpilogue epilogue;
    epilogue.bias = bias;
    epilogue.residual = residual;
    hipError_t rc = launch_gemm_bf16(m, n, k, lhs, packed_rhs, out_f32, nullptr, epilogue, stream, true);
    if (rc != hipSuccess) return rc;
    return launch_layer_norm_f32(m, n, out_f32, nullptr, gamma, beta, epsilon, nullptr, out_ln, stream);
}

}  // namespace sthip
