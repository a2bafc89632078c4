// Fused conv2d + bias + activation as an implicit GEMM on the f32 matrix cores of gfx950.
//
// Semantics follow Conv2d::forward_cpu, crates/st-nn/src/layers/conv.rs:2559-2599: zero-padded im2col
// with patch column s = (ic*KH + ky)*KW + kx (:702-748), contraction "ps,os->po" over s (:199-326),
// + bias[o] (:2594-2597), result stored as NCHW (:918-948).  Here the patch matrix is never built:
//
//   out[b][o][p] = act( Σ_s W[o][s] · X[b][ic(s)][oy(p)*sh + ky(s)*dh - ph][ox(p)*sw + kx(s)*dw - pw] + bias[o] )
//
// is computed as the GEMM  W(C_out × S) · P_b(S × OH·OW)  per image b, so that a tile's rows are output
// channels and its columns are consecutive output pixels — exactly the NCHW store order, which removes
// the reference's separate matrix→NCHW pass.  The weight tile is read as stored (OIHW = row-major,
// s contiguous).  The patch tile is gathered from the image on the way into LDS with an offset table
// lut[s] = {ic*H*W + ky*dh*W + kx*dw, ky*dh | kx*dw << 16} built once per workgroup in LDS, so the
// per-element cost is two adds, two range checks and one load.
//
// MFMA usage is the same as the f32 GEMM (32x32x2 f32, k issued as the pairs {s, s+4}).
#include "device_math.h"
#include "kernels.h"

#include <type_traits>

namespace sthip {

namespace {

struct ConvArgs {
    const float *input;
    const float *weight;
    const float *bias;
    float *out;
    ConvShape s;
    int K;        // c_in * kh * kw
    int spatial;  // oh * ow
    int tiles_px, tiles_oc;
    int xcd_swizzle;
    int activation;
    unsigned tap_bytes[32];  // ring kernel: byte offset of tap ky*kw + kx relative to a pixel's top-left tap
};


// FULLK: c_in*kh*kw is a multiple of the 16-wide k-tile and weight rows are 16-byte aligned, so the loop
// carries no k bounds checks; weight rows past c_out are clamped to the last row (what they contribute
// only reaches output channels that are never stored).
//
// TRANSPOSED turns the gather into that of the convolution's adjoint (gradient with respect to the input, the
// col2im of crates/st-nn/src/layers/conv.rs:860-916 written as a gather): the "image" is grad_output with
// s.c_in = C_out channels of s.h × s.w = OH × OW values, the output pixels (s.oh × s.ow = H × W) are input
// positions, and tap (ky, kx) of output pixel (y, x) reads grad_output at ((y + pad - ky·dil) / stride, ...) when
// that division is exact and in range.  The weight matrix is then W[ic][(oc, ky, kx)].
template <int BM, int BN, int BK, int WM, int WN, bool VEC, bool FULLK, bool TRANSPOSED>
__global__ __launch_bounds__(64 * WM * WN) void conv2d_f32_kernel(ConvArgs p)
{
    // WM×WN wavefronts, each owning (BM/WM) output channels × (BN/WN) pixels.  As in the f32 GEMM, many
    // wavefronts with 32×32 tiles keep the (slow) f32 matrix pipe busier than few wavefronts with big tiles.
    constexpr int T = 64 * WM * WN;
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(TM >= 1 && TN >= 1, "wavefront tile must be at least 32×32");
    static_assert(T % BN == 0 && (BK * BN) % T == 0 && (BM * BK / 4) % T == 0, "loader mapping");
    constexpr int A_STRIDE = BK + 4;
    constexpr int B_STRIDE = BN + 8;
    constexpr int A_ELEMS = BM * A_STRIDE;
    constexpr int B_ELEMS = BK * B_STRIDE;
    constexpr int B_PER_THREAD = BK * BN / T;
    constexpr int B_ROW_STEP = T / BN;
    constexpr int A_LOADS = BM * BK / 4 / T;

    extern __shared__ __attribute__((aligned(16))) unsigned char conv_lds[];
    const int K = p.K;
    const int k_padded = (K + 15) & ~15;
    int2 *lut = reinterpret_cast<int2 *>(conv_lds);
    float *As = reinterpret_cast<float *>(conv_lds + static_cast<size_t>(k_padded) * sizeof(int2));
    float *Bs = As + 2 * A_ELEMS;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int li = lane & 31, lh = lane >> 5;

    // Workgroup ids are dealt round-robin to the 8 XCDs (id & 7).  When the batch divides by 8 every XCD
    // keeps whole images, so an image (and its halo re-reads) is fetched into one L2 only.
    int bid = blockIdx.x;
    if (p.xcd_swizzle) bid = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int tile_oc = bid % p.tiles_oc;
    bid /= p.tiles_oc;
    const int tile_px = bid % p.tiles_px;
    const int image = bid / p.tiles_px;
    const int oc0 = tile_oc * BM, px0 = tile_px * BN;

    const ConvShape &s = p.s;
    const int H = s.h, W = s.w;
    const int khw = s.kh * s.kw;
    for (int k = tid; k < K; k += T) {
        const int ic = k / khw, rem = k - ic * khw;
        const int ky = rem / s.kw, kx = rem - ky * s.kw;
        const int dy = ky * s.dil_h, dx = kx * s.dil_w;
        lut[k] = make_int2(TRANSPOSED ? ic * H * W : ic * H * W + dy * W + dx, dy | (dx << 16));
    }

    // Every thread gathers one pixel column of the patch tile, rows (tid / BN) + B_ROW_STEP * r.
    const int px_local = tid % BN;
    const int krow0 = tid / BN;
    const int px = px0 + px_local;
    const bool px_valid = px < p.spatial;
    const int oy = px / s.ow, ox = px - oy * s.ow;
    const int iy0 = TRANSPOSED ? oy + s.pad_h : oy * s.stride_h - s.pad_h;
    const int ix0 = TRANSPOSED ? ox + s.pad_w : ox * s.stride_w - s.pad_w;
    const int base = iy0 * W + ix0;
    const float *img = p.input + static_cast<size_t>(image) * s.c_in * H * W;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    float4 ra[A_LOADS];
    float rb[B_PER_THREAD];

    const float *w_src[A_LOADS];
#pragma unroll
    for (int r = 0; r < A_LOADS; ++r) {
        const int f = tid + T * r;
        w_src[r] = p.weight + static_cast<size_t>(min(oc0 + (f >> 2), s.c_out - 1)) * K + (f & 3) * 4;
    }
    auto load_global = [&](int k0) {
#pragma unroll
        for (int r = 0; r < A_LOADS; ++r) {
            if (FULLK) {
                ra[r] = *reinterpret_cast<const float4 *>(w_src[r] + k0);
                continue;
            }
            const int f = tid + T * r;
            const int row = f >> 2, c4 = (f & 3) * 4;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (oc0 + row < s.c_out) {
                const float *src = p.weight + static_cast<size_t>(oc0 + row) * K + k0 + c4;
                if (VEC) {
                    if (k0 + c4 < K) v = *reinterpret_cast<const float4 *>(src);
                } else {
                    if (k0 + c4 + 0 < K) v.x = src[0];
                    if (k0 + c4 + 1 < K) v.y = src[1];
                    if (k0 + c4 + 2 < K) v.z = src[2];
                    if (k0 + c4 + 3 < K) v.w = src[3];
                }
            }
            ra[r] = v;
        }
#pragma unroll
        for (int r = 0; r < B_PER_THREAD; ++r) {
            const int k = k0 + krow0 + B_ROW_STEP * r;
            float v = 0.0f;
            if (px_valid && (FULLK || k < K)) {
                const int2 e = lut[k];
                if (TRANSPOSED) {
                    const int ty = iy0 - (e.y & 0xffff), tx = ix0 - (e.y >> 16);
                    if (ty >= 0 && tx >= 0) {
                        const int sy = ty / s.stride_h, sx = tx / s.stride_w;
                        if (sy * s.stride_h == ty && sx * s.stride_w == tx && sy < H && sx < W) v = img[e.x + sy * W + sx];
                    }
                } else {
                    const int iy = iy0 + (e.y & 0xffff);
                    const int ix = ix0 + (e.y >> 16);
                    if (static_cast<unsigned>(iy) < static_cast<unsigned>(H) &&
                        static_cast<unsigned>(ix) < static_cast<unsigned>(W))
                        v = img[base + e.x];
                }
            }
            rb[r] = v;
        }
    };
    auto store_lds = [&](int stage) {
        float *as = As + stage * A_ELEMS;
        float *bs = Bs + stage * B_ELEMS;
#pragma unroll
        for (int r = 0; r < A_LOADS; ++r) {
            const int f = tid + T * r;
            const int row = f >> 2, c4 = (f & 3) * 4;
            *reinterpret_cast<float4 *>(&as[row * A_STRIDE + c4]) = ra[r];
        }
#pragma unroll
        for (int r = 0; r < B_PER_THREAD; ++r) bs[(krow0 + B_ROW_STEP * r) * B_STRIDE + px_local] = rb[r];
    };
    auto compute = [&](int stage) {
        const float *as = As + stage * A_ELEMS;
        const float *bs = Bs + stage * B_ELEMS;
#pragma unroll
        for (int kk = 0; kk < BK / 8; ++kk) {
            float a[TM][4], b[TN][4];
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                const int row = wm * WTM + tm * 32 + li;
                const float4 v = *reinterpret_cast<const float4 *>(&as[row * A_STRIDE + kk * 8 + lh * 4]);
                a[tm][0] = v.x; a[tm][1] = v.y; a[tm][2] = v.z; a[tm][3] = v.w;
            }
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
                const int col = wn * WTN + tn * 32 + li;
#pragma unroll
                for (int t = 0; t < 4; ++t) b[tn][t] = bs[(kk * 8 + lh * 4 + t) * B_STRIDE + col];
            }
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn)
                        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[tm][t], b[tn][t], acc[tm][tn], 0, 0, 0);
        }
    };

    __syncthreads();  // offset table complete
    const int steps = (K + BK - 1) / BK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int t = 0; t < steps; ++t) {
        const bool more = t + 1 < steps;
        if (more) load_global((t + 1) * BK);
        compute(t & 1);
        if (more) store_lds((t + 1) & 1);
        __syncthreads();
    }

    float *out_image = p.out + static_cast<size_t>(image) * s.c_out * p.spatial;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        const int col = px0 + wn * WTN + tn * 32 + li;
        if (col >= p.spatial) continue;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int oc = oc0 + wm * WTM + tm * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                if (oc >= s.c_out) continue;
                float value = acc[tm][tn][r];
                if (p.bias) value += p.bias[oc];
                out_image[static_cast<size_t>(oc) * p.spatial + col] = apply_activation(value, p.activation);
            }
        }
    }
}

// -------------------------------------------------------------------------------------------------
// Ring kernel: the same implicit GEMM, but both operands travel global memory -> LDS without passing
// through registers (buffer_load ... lds) into a three-deep ring of 16-wide k-tiles, so two k-tiles of
// loads are in flight while the matrix cores work on the third.  Per k-tile a wavefront issues one
// 16-byte-per-lane load of weights and 16/WAVES one-pixel-per-lane gathers; a tap that falls into the padding
// is given an out-of-range offset, for which the buffer load writes zero into LDS.  Whether tap (ky, kx) of
// this lane's pixel is inside the image is a bit of a per-lane mask computed once, and which (channel, tap) a
// gathered row belongs to is wavefront-uniform and tracked in scalar registers, so the loop's vector address
// arithmetic is a shift, an add and a shift-add per gathered row.
//
// Needs: c_in*kh*kw a multiple of 16 with 16-byte aligned weight rows, kh*kw <= 32, one image smaller than
// 1 GiB and the weights smaller than 2 GiB (32-bit buffer offsets).  Everything else takes the register-staged kernel above.
//
// LDS per stage: weights BM rows × 64 B, 16-byte chunk c of row r stored at position c ^ ((r >> 2) & 3)
// (the swizzle is applied by choosing which chunk each lane fetches), then 16 patch rows of 64 pixels with a
// 288-byte row pitch; both make the fragment reads conflict-free.  Three stages of the 128-row tile are
// 38 KB, so four workgroups share a compute unit.
// -------------------------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void *lds_void_ptr;

#define ST_CONV_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (7 << 4) | (15 << 8) | ((((n) >> 4) & 3) << 14))

constexpr int kRingStages = 3;

template <int BM, int WM, int WN>
__device__ __forceinline__ void conv2d_f32_ring_body(const ConvArgs &p)
{
    constexpr int BN = 64, BK = 16, RING = kRingStages;
    constexpr int WAVES = WM * WN;
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(TM >= 1 && TN >= 1, "wavefront tile must be at least 32×32");
    static_assert(BM == 16 * WAVES, "one 16-row weight load per wavefront and k-tile");
    static_assert(BK % WAVES == 0, "patch rows divide over the wavefronts");
    constexpr int B_ROWS = BK / WAVES;           // gathered rows per wavefront and k-tile
    constexpr int LOADS = 1 + B_ROWS;            // load instructions per wavefront and k-tile
    constexpr int B_PITCH = (BN + 8) * 4;        // bytes
    constexpr int A_BYTES = BM * BK * 4;
    constexpr int STAGE = A_BYTES + BK * B_PITCH;

    extern __shared__ __attribute__((aligned(16))) unsigned char conv_lds[];
    const int K = p.K;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: the per-row tap bookkeeping stays on the SALU
    const int wm = wave / WN, wn = wave % WN;
    const int li = lane & 31, lh = lane >> 5;

    int bid = blockIdx.x;
    if (p.xcd_swizzle) bid = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int tile_oc = bid % p.tiles_oc;
    bid /= p.tiles_oc;
    const int tile_px = bid % p.tiles_px;
    const int image = bid / p.tiles_px;
    const int oc0 = tile_oc * BM, px0 = tile_px * BN;

    const ConvShape &s = p.s;
    const int H = s.h, W = s.w;
    const int khw = s.kh * s.kw;
    const unsigned channel_bytes = static_cast<unsigned>(H) * W * 4u;

    // This lane's pixel (the same in every wavefront) and the validity of each of its kh*kw taps.
    const int px = px0 + lane;
    const bool px_valid = px < p.spatial;
    const int oy = px / s.ow, ox = px - oy * s.ow;
    const int iy0 = oy * s.stride_h - s.pad_h;
    const int ix0 = ox * s.stride_w - s.pad_w;
    const unsigned base_bytes = static_cast<unsigned>(iy0 * W + ix0) * 4u;  // may wrap; valid taps unwrap it
    unsigned tap_mask = 0;
    for (int j = 0; j < khw; ++j) {
        const int ky = j / s.kw, kx = j - ky * s.kw;
        const bool ok = px_valid && static_cast<unsigned>(iy0 + ky * s.dil_h) < static_cast<unsigned>(H) &&
                        static_cast<unsigned>(ix0 + kx * s.dil_w) < static_cast<unsigned>(W);
        tap_mask |= (ok ? 1u : 0u) << j;
    }
    const unsigned tap_outside = ~tap_mask;  // bit j set: tap j of this pixel reads padding (or the pixel is past the end)

    const size_t image_elems = static_cast<size_t>(s.c_in) * H * W;
    const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(p.input + static_cast<size_t>(image) * image_elems), 0, static_cast<int>(image_elems * 4), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(p.weight), 0, static_cast<int>(static_cast<size_t>(s.c_out) * K * 4), 0x00020000);

    // Weights: wavefront w fills rows 16w .. 16w+15 of the stage; lane L lands at row L/4, chunk position L%4.
    const int a_row = wave * 16 + (lane >> 2);
    const int a_chunk = (lane & 3) ^ ((a_row >> 2) & 3);
    const unsigned a_off = (static_cast<unsigned>(min(oc0 + a_row, s.c_out - 1)) * K + a_chunk * 4) * 4u;

    // Patch row `wave*B_ROWS + r` of k-tile t is reduction index k = 16t + row = ic*kh*kw + tap.  issue() is called
    // for t = 0, 1, 2, ... in order, so (ic, tap) of each of this wavefront's rows is advanced by 16 per call.
    int row_ic[B_ROWS], row_tap[B_ROWS];
#pragma unroll
    for (int r = 0; r < B_ROWS; ++r) {
        const int row = wave * B_ROWS + r;
        row_ic[r] = row / khw;
        row_tap[r] = row - row_ic[r] * khw;
    }
    const int step_ic = BK / khw, step_tap = BK - step_ic * khw;

    // Every vector instruction of the loop costs matrix-pipe time (the f32 MFMAs and the ordinary VALU do not
    // overlap on a SIMD), so the gather address is three of them: the tap's outside-bit is shifted to bit 31 and
    // added to the in-image offset, which pushes the offset of a padding tap past the buffer's range.  (Needs the
    // image and its top/left padding to stay below 2^30 bytes so that no wrapped offset lands back in range.)
    auto issue = [&](auto slot_tag, int t) {  // requests k-tile t into ring slot SLOT
        constexpr int SLOT = decltype(slot_tag)::value;
        unsigned char *stage = conv_lds + SLOT * STAGE;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_void_ptr)(stage + wave * 1024), 16, a_off, t * (BK * 4), 0, 0);
#pragma unroll
        for (int r = 0; r < B_ROWS; ++r) {
            const int row = wave * B_ROWS + r;
            const unsigned tap_bytes = p.tap_bytes[row_tap[r]] + static_cast<unsigned>(row_ic[r]) * channel_bytes;
            const unsigned off = ((tap_outside >> row_tap[r]) << 31) + (base_bytes + tap_bytes);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (lds_void_ptr)(stage + A_BYTES + row * B_PITCH), 4, off, 0, 0, 0);
            row_tap[r] += step_tap;
            row_ic[r] += step_ic;
            if (row_tap[r] >= khw) {
                row_tap[r] -= khw;
                ++row_ic[r];
            }
        }
    };

    // Per-lane fragment addresses within a stage; the stage offset is a compile-time constant in the unrolled loop,
    // so the reads need no address arithmetic.
    unsigned a_lane[BK / 8][TM], b_lane[TN];
#pragma unroll
    for (int kk = 0; kk < BK / 8; ++kk)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const int row = wm * WTM + tm * 32 + li;
            a_lane[kk][tm] = row * 64 + (((kk * 2 + lh) ^ ((row >> 2) & 3)) * 16);
        }
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) b_lane[tn] = A_BYTES + lh * 4 * B_PITCH + (wn * WTN + tn * 32 + li) * 4;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    // All fragments of the k-tile are read first and the MFMAs then run back to back at raised priority: the
    // wavefront holds the matrix pipe for one uninterrupted run instead of stalling on LDS between pairs.
    auto compute = [&](auto slot_tag) {
        constexpr int SLOT = decltype(slot_tag)::value;
        const unsigned char *stage = conv_lds + SLOT * STAGE;
        float a[BK / 8][TM][4], b[BK / 8][TN][4];
#pragma unroll
        for (int kk = 0; kk < BK / 8; ++kk) {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                const f32x4 v = *reinterpret_cast<const f32x4 *>(stage + a_lane[kk][tm]);
                a[kk][tm][0] = v[0]; a[kk][tm][1] = v[1]; a[kk][tm][2] = v[2]; a[kk][tm][3] = v[3];
            }
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    b[kk][tn][t] = *reinterpret_cast<const float *>(stage + b_lane[tn] + (kk * 8 + t) * B_PITCH);
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

    static_assert(RING == 3, "the loop below is unrolled for three ring slots");
    const int steps = K / BK;
    if (steps > 0) issue(std::integral_constant<int, 0>{}, 0);
    if (steps > 1) issue(std::integral_constant<int, 1>{}, 1);
    // Drain the prologue once.  (With prologue loads still counted as outstanding at the loop header the
    // compiler's wait-count insertion falls back to a full vmcnt(0) inside the loop.)
    ST_CONV_WAIT_VMCNT(0);
    auto step = [&](auto slot_tag, int t) {
        constexpr int SLOT = decltype(slot_tag)::value;
        // This wavefront's loads of k-tile t have landed once only the loads of k-tile t+1 are outstanding; the
        // barrier then extends that to every wavefront and also says that everyone is done reading the slot
        // k-tile t+2 is about to overwrite.
        //
        // A bare s_barrier, not __syncthreads(): the latter's workgroup release fence makes the compiler wait for
        // every outstanding load, including the k-tile that was just requested.  Nothing in the loop writes LDS
        // with ordinary stores, the loads into LDS are ordered by the vmcnt wait above, and a wavefront's LDS
        // reads of a slot have returned (its MFMAs consumed them) before it arrives at the next barrier.
        if (t + 1 < steps) ST_CONV_WAIT_VMCNT(LOADS);
        else ST_CONV_WAIT_VMCNT(0);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (t + 2 < steps) issue(std::integral_constant<int, (SLOT + 2) % RING>{}, t + 2);
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

    float *out_image = p.out + static_cast<size_t>(image) * s.c_out * p.spatial;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        const int col = px0 + wn * WTN + tn * 32 + li;
        if (col >= p.spatial) continue;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int oc = oc0 + wm * WTM + tm * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                if (oc >= s.c_out) continue;
                float value = acc[tm][tn][r];
                if (p.bias) value += p.bias[oc];
                out_image[static_cast<size_t>(oc) * p.spatial + col] = apply_activation(value, p.activation);
            }
        }
    }
}

// (A kernel template whose body uses the LDS-load builtins loses its host-side launch stub with this
// compiler, hence plain kernels around the templated body.)
__global__ __launch_bounds__(512) void conv2d_f32_ring128_kernel(ConvArgs p) { conv2d_f32_ring_body<128, 4, 2>(p); }
__global__ __launch_bounds__(256) void conv2d_f32_ring64_kernel(ConvArgs p) { conv2d_f32_ring_body<64, 2, 2>(p); }

template <int BM>
hipError_t launch_ring(ConvArgs args, hipStream_t stream)
{
    args.tiles_oc = (args.s.c_out + BM - 1) / BM;
    args.tiles_px = (args.spatial + 63) / 64;
    const size_t tiles = static_cast<size_t>(args.tiles_oc) * args.tiles_px * static_cast<size_t>(args.s.batch);
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    args.xcd_swizzle = (args.s.batch % 8 == 0) ? 1 : 0;
    for (int j = 0; j < 32; ++j) {
        const int ky = j / args.s.kw, kx = j % args.s.kw;
        args.tap_bytes[j] = j < args.s.kh * args.s.kw
                                ? static_cast<unsigned>(ky * args.s.dil_h * args.s.w + kx * args.s.dil_w) * 4u : 0u;
    }
    const size_t lds_bytes = kRingStages * (static_cast<size_t>(BM) * 64 + 16 * 288);
    auto kernel = BM == 128 ? conv2d_f32_ring128_kernel : conv2d_f32_ring64_kernel;
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(tiles)), dim3(BM == 128 ? 512 : 256), lds_bytes, stream, args);
    return hipGetLastError();
}

template <int BM, int BN, int BK, int WM, int WN, bool TRANSPOSED = false>
hipError_t launch_tile(ConvArgs args, bool vec, hipStream_t stream)
{
    args.tiles_oc = (args.s.c_out + BM - 1) / BM;
    args.tiles_px = (args.spatial + BN - 1) / BN;
    const size_t tiles = static_cast<size_t>(args.tiles_oc) * args.tiles_px * static_cast<size_t>(args.s.batch);
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    args.xcd_swizzle = (args.s.batch % 8 == 0) ? 1 : 0;
    const size_t k_padded = (static_cast<size_t>(args.K) + 15) & ~static_cast<size_t>(15);
    const size_t lds_bytes = k_padded * sizeof(int2) +
                             2 * (static_cast<size_t>(BM) * (BK + 4) + static_cast<size_t>(BK) * (BN + 8)) * sizeof(float);
    const dim3 grid(static_cast<unsigned>(tiles));
    const dim3 block(64 * WM * WN);
    hipError_t rc;
    auto launch = [&](auto kernel) -> hipError_t {
        hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
        if (status != hipSuccess) return status;
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, args);
        return hipSuccess;
    };
    if (vec && args.K % BK == 0)
        rc = launch(conv2d_f32_kernel<BM, BN, BK, WM, WN, true, true, TRANSPOSED>);
    else if (vec)
        rc = launch(conv2d_f32_kernel<BM, BN, BK, WM, WN, true, false, TRANSPOSED>);
    else
        rc = launch(conv2d_f32_kernel<BM, BN, BK, WM, WN, false, false, TRANSPOSED>);
    if (rc != hipSuccess) return rc;
    return hipGetLastError();
}

}  // namespace

hipError_t launch_conv2d_f32(const ConvShape &shape, int activation, const float *input, const float *weight,
                             const float *bias, float *out, hipStream_t stream)
{
    if (shape.batch == 0 || shape.c_out == 0 || shape.oh == 0 || shape.ow == 0) return hipSuccess;
    ConvArgs args;
    args.input = input;
    args.weight = weight;
    args.bias = bias;
    args.out = out;
    args.s = shape;
    args.K = shape.c_in * shape.kh * shape.kw;
    args.spatial = shape.oh * shape.ow;
    args.tiles_px = args.tiles_oc = 0;
    args.xcd_swizzle = 0;
    args.activation = activation;
    // The offset table packs ky*dh and kx*dw into 16 bits each.
    if ((shape.kh - 1) * static_cast<long long>(shape.dil_h) > 0x7fff ||
        (shape.kw - 1) * static_cast<long long>(shape.dil_w) > 0x7fff || args.K > kConvMaxReduction)
        return hipErrorInvalidValue;
    const bool vec = (args.K % 4 == 0) && ((reinterpret_cast<uintptr_t>(weight) & 15u) == 0);
    // 8 wavefronts of 32×32 per 128×64 tile measured best for wide layers (128×128 tiles, 32-deep k-tiles and
    // 4-wavefront layouts were all 10-20 % slower on the 64->128 channel 56×56 case).
    const bool ring_ok = vec && args.K % 16 == 0 && shape.kh * shape.kw <= 32 &&
                         static_cast<size_t>(shape.c_in) * shape.h * shape.w * 4 < (1ull << 30) &&
                         (static_cast<size_t>(shape.pad_h) * shape.w + shape.pad_w) * 4 < (1ull << 30) &&
                         (static_cast<size_t>(shape.oh + 64) * shape.stride_h * shape.w + static_cast<size_t>(shape.ow) * shape.stride_w) * 4 < (1ull << 30) &&
                         static_cast<size_t>(shape.c_out) * args.K * 4 < (1ull << 31);
    if (ring_ok) return shape.c_out > 64 ? launch_ring<128>(args, stream) : launch_ring<64>(args, stream);
    if (shape.c_out > 64) return launch_tile<128, 64, 16, 4, 2>(args, vec, stream);
    return launch_tile<64, 64, 16, 2, 2>(args, vec, stream);
}

// Adjoint gather for strides other than 1: `shape` describes the virtual forward problem (see TRANSPOSED above).
hipError_t launch_conv2d_adjoint_f32(const ConvShape &shape, const float *grad_output, const float *weight_ic_major,
                                     float *grad_input, hipStream_t stream)
{
    if (shape.batch == 0 || shape.c_out == 0 || shape.oh == 0 || shape.ow == 0) return hipSuccess;
    ConvArgs args;
    args.input = grad_output;
    args.weight = weight_ic_major;
    args.bias = nullptr;
    args.out = grad_input;
    args.s = shape;
    args.K = shape.c_in * shape.kh * shape.kw;
    args.spatial = shape.oh * shape.ow;
    args.tiles_px = args.tiles_oc = 0;
    args.xcd_swizzle = 0;
    args.activation = ST_HIP_ACT_NONE;
    if ((shape.kh - 1) * static_cast<long long>(shape.dil_h) > 0x7fff ||
        (shape.kw - 1) * static_cast<long long>(shape.dil_w) > 0x7fff || args.K > kConvMaxReduction)
        return hipErrorInvalidValue;
    const bool vec = (args.K % 4 == 0) && ((reinterpret_cast<uintptr_t>(weight_ic_major) & 15u) == 0);
    if (shape.c_out > 64) return launch_tile<128, 64, 16, 4, 2, true>(args, vec, stream);
    return launch_tile<64, 64, 16, 2, 2, true>(args, vec, stream);
}

}  // namespace sthip
