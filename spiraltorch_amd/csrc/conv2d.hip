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
//
// Three kernel families share this formulation, chosen by shape in launch_conv2d_f32: the general tile kernel
// described above (any shape), the ring kernel (weights and patch rows go memory -> LDS directly; the better steady
// state for layers that give the chip several rounds of tiles) and the strip kernel (weights resident in LDS, image
// values loaded straight into the MFMA operand registers, blocks claimed dynamically; the better balance when the
// tiles of a layer quantise badly over the chip, and for narrow layers).
#include "device_math.h"
#include "kernels.h"

#include <atomic>
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
    unsigned tap_bytes[64];  // ring kernel: byte offset of tap ky*kw + kx relative to a pixel's top-left tap
    // General kernel, k-sliced form (few tiles, long reduction): workgroup (tile, blockIdx.y) sums reduction terms
    // [y·k_slice, (y+1)·k_slice) and writes them, raw, to plane y of `out` (the launch passes the partial planes as
    // `out`, no bias and no activation); conv_slice_reduce_kernel adds the planes in order and finishes.
    int k_slice = 0;  // 0: the whole reduction; else a multiple of the 16-wide k-tile
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
    // This workgroup's part of the reduction, [k_lo, K): K below is its END; p.K stays the row stride of the weights.
    const int k_lo = p.k_slice ? static_cast<int>(blockIdx.y) * p.k_slice : 0;
    const int K = p.k_slice ? min(p.K, k_lo + p.k_slice) : p.K;
    // The offset table holds one segment of the reduction (kConvTableEntries entries) at a time.
    const int k_padded = (min(p.K, kConvTableEntries) + 15) & ~15;
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
    int seg0 = k_lo;  // first reduction index of the segment the table describes
    auto fill_table = [&]() {
        const int seg_end = min(K, seg0 + kConvTableEntries);
        for (int k = seg0 + tid; k < seg_end; k += T) {
            const int ic = k / khw, rem = k - ic * khw;
            const int ky = rem / s.kw, kx = rem - ky * s.kw;
            const int dy = ky * s.dil_h, dx = kx * s.dil_w;
            lut[k - seg0] = make_int2(TRANSPOSED ? ic * H * W : ic * H * W + dy * W + dx, dy | (dx << 16));
        }
    };

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
        w_src[r] = p.weight + static_cast<size_t>(min(oc0 + (f >> 2), s.c_out - 1)) * p.K + (f & 3) * 4;
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
                const float *src = p.weight + static_cast<size_t>(oc0 + row) * p.K + k0 + c4;
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
                const int2 e = lut[k - seg0];
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

    // Segment by segment (one for every layer up to kConvTableEntries reduction terms): table, then its k-tiles
    // through the two-stage pipeline; the accumulators run on across segments, in reduction order.
    static_assert(kConvTableEntries % BK == 0, "segments hold whole k-tiles");
    for (; seg0 < K; seg0 += kConvTableEntries) {
        fill_table();
        __syncthreads();  // offset table complete (and the previous segment's last tile has been consumed)
        const int steps = (min(K - seg0, kConvTableEntries) + BK - 1) / BK;
        load_global(seg0);
        store_lds(0);
        __syncthreads();
        for (int t = 0; t < steps; ++t) {
            const bool more = t + 1 < steps;
            if (more) load_global(seg0 + (t + 1) * BK);
            compute(t & 1);
            if (more) store_lds((t + 1) & 1);
            __syncthreads();
        }
    }

    float *out_image = p.out + (static_cast<size_t>(blockIdx.y) * s.batch + image) * s.c_out * p.spatial;
    with_epilogue_ops(p.activation, false, [&](auto &&act, auto) {
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
                    const float value = acc[tm][tn][r] + (p.bias ? p.bias[oc] : -0.0f);  // x + -0.0f == x
                    out_image[static_cast<size_t>(oc) * p.spatial + col] = act(value);
                }
            }
        }
    });
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
// Needs: c_in*kh*kw a multiple of 16 with 16-byte aligned weight rows, kh*kw <= 64, one image smaller than
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
    unsigned long long tap_mask = 0;  // up to 64 taps (7×7 kernels have 49)
    for (int j = 0; j < khw; ++j) {
        const int ky = j / s.kw, kx = j - ky * s.kw;
        const bool ok = px_valid && static_cast<unsigned>(iy0 + ky * s.dil_h) < static_cast<unsigned>(H) &&
                        static_cast<unsigned>(ix0 + kx * s.dil_w) < static_cast<unsigned>(W);
        tap_mask |= (ok ? 1ull : 0ull) << j;
    }
    const unsigned long long tap_outside = ~tap_mask;  // bit j set: tap j of this pixel reads padding (or the pixel is past the end)

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
            const unsigned off = (static_cast<unsigned>(tap_outside >> row_tap[r]) << 31) + (base_bytes + tap_bytes);
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
    with_epilogue_ops(p.activation, false, [&](auto &&act, auto) {
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
                    const float value = acc[tm][tn][r] + (p.bias ? p.bias[oc] : -0.0f);  // x + -0.0f == x
                    out_image[static_cast<size_t>(oc) * p.spatial + col] = act(value);
                }
            }
        }
    });
}

// (A kernel template whose body uses the LDS-load builtins loses its host-side launch stub with this
// compiler, hence plain kernels around the templated body.)
__global__ __launch_bounds__(512) void conv2d_f32_ring128_kernel(ConvArgs p) { conv2d_f32_ring_body<128, 4, 2>(p); }
__global__ __launch_bounds__(256) void conv2d_f32_ring64_kernel(ConvArgs p) { conv2d_f32_ring_body<64, 2, 2>(p); }

// ---- strip kernel: 32 output channels × a long run of pixels per workgroup, no LDS traffic for the image --------
//
// A workgroup of 16 wavefronts owns 32 output channels and a run of 32-pixel blocks of one image.  Its weights
// (32 rows × c_in × 9 taps) are staged into LDS once and stay there; after that single barrier the wavefronts
// never synchronise again: each takes the next unclaimed block from a counter in LDS, runs the whole reduction
// for that 32×32 block, stores it and takes another.  With only 32 output channels per workgroup every gathered
// image value feeds exactly one MFMA, so it is loaded from global memory (L1/L2) straight into the B operand
// register: one buffer load per MFMA, all nine taps of the next channel pair requested before the MFMAs of the
// current pair (measured: f32 MFMAs interleaved one-to-one with independent buffer loads still run at the
// matrix pipe's full rate).  The nine per-lane byte offsets of a block are computed once, with bit 31 set for
// padding taps, which the buffer range check turns into 0.0.  Because blocks finish at different times, the
// output stores of one block overlap the arithmetic of the others, and the unit of load balancing is a single
// block on a single SIMD.  Where the LDS has room beside the weights (and the output plane is a multiple of four
// pixels, 16-byte aligned) a block leaves through a per-wavefront LDS tile as 128-bit stores, four instead of
// sixteen store instructions per block (config 2: 162 -> 157 µs).
//
// k runs in the pairs {(ic, tap), (ic+1, tap)}: lanes 0-31 supply channel 2j, lanes 32-63 channel 2j+1.
struct StripArgs {
    const float *input;
    const float *weight;
    const float *bias;
    float *out;
    ConvShape s;
    int spatial;           // oh * ow
    int blocks_per_image;  // ceil(spatial / 32)
    int chunks;            // workgroups per image and channel strip
    int blocks_per_chunk;
    int oc_strips;         // ceil(c_out / 32)
    int total;             // workgroups
    int xcd_swizzle;
    int activation;
};

constexpr int kStripTaps = 9, kStripThreads = 1024;
// 32 rows × c_in channels × 9 taps of f32 weights + the counter must fit 160 KiB of LDS: up to 104 channels with the
// taps of a channel padded to 12 words (128-bit reads), up to 142 channels packed.
constexpr int kStripMaxChannelsPadded = 104, kStripMaxChannels = 142;

inline int strip_pitch(int c_in) { return c_in <= kStripMaxChannelsPadded ? 12 : 9; }
inline size_t strip_lds_bytes(int c_in) { return static_cast<size_t>(c_in) * 32 * strip_pitch(c_in) * 4 + 16; }
// Epilogue tiles for 128-bit stores: per wavefront 16 channels × 32 pixels, rows 36 words apart.
constexpr int kStripStagePitch = 36;
constexpr size_t kStripStageBytes = static_cast<size_t>(kStripThreads / 64) * 16 * kStripStagePitch * 4;

template <int PITCH, bool WIDE>
__device__ __forceinline__ void conv2d_f32_strip_body(const StripArgs &p)
{
    extern __shared__ __align__(16) unsigned char strip_lds[];
    float *lds_w = reinterpret_cast<float *>(strip_lds);
    const ConvShape &s = p.s;
    const int K = s.c_in * kStripTaps;
    unsigned *counter = reinterpret_cast<unsigned *>(strip_lds + static_cast<size_t>(s.c_in) * 32 * PITCH * 4);
    const int tid = threadIdx.x, lane = tid & 63, lh = lane >> 5, li = lane & 31;
    int bid = blockIdx.x;
    if (p.xcd_swizzle) bid = (bid & 7) * (p.total >> 3) + (bid >> 3);  // the workgroups of an image share an XCD's L2
    const int per_image = p.chunks * p.oc_strips;
    const int image = bid / per_image;
    const int sub = bid - image * per_image;
    const int chunk = sub / p.oc_strips, strip = sub - chunk * p.oc_strips;
    const int oc0 = strip * 32;
    const int first = chunk * p.blocks_per_chunk;
    const int nblocks = min(p.blocks_per_chunk, p.blocks_per_image - first);

    // Weights of the strip: LDS index of (oc, ic, tap) is (ic*32 + oc)*PITCH + tap, so that a lane's nine taps of a
    // channel are consecutive and the 32 lanes of a half-wavefront sit PITCH words apart (no bank conflicts for 9 or 12).
    if (K % 4 == 0 && (reinterpret_cast<uintptr_t>(p.weight) & 15u) == 0) {
        constexpr int BATCH = 5;  // 128-bit reads in flight per lane before the first is scattered into LDS
        const int per_row = K >> 2, total = 32 * per_row;
        for (int base = 0; base < total; base += kStripThreads * BATCH) {
            float4 held[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const int v = base + j * kStripThreads + tid;
                const int oc = v / per_row, q = v - oc * per_row;
                held[j] = (v < total && oc0 + oc < s.c_out)
                              ? *reinterpret_cast<const float4 *>(p.weight + static_cast<size_t>(oc0 + oc) * K + 4 * q)
                              : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            }
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const int v = base + j * kStripThreads + tid;
                if (v >= total) continue;
                const int oc = v / per_row, q = v - oc * per_row;
                const float values[4] = {held[j].x, held[j].y, held[j].z, held[j].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int r = 4 * q + e;
                    const int ic = r / kStripTaps, tap = r - ic * kStripTaps;
                    lds_w[(ic * 32 + oc) * PITCH + tap] = values[e];
                }
            }
        }
    } else {
        for (int e = tid; e < 32 * K; e += kStripThreads) {
            const int oc = e / K, r = e - oc * K;
            const int ic = r / kStripTaps, tap = r - ic * kStripTaps;
            lds_w[(ic * 32 + oc) * PITCH + tap] = oc0 + oc < s.c_out ? p.weight[static_cast<size_t>(oc0 + oc) * K + r] : 0.0f;
        }
    }
    if (tid == 0) *counter = 0;
    __syncthreads();

    const unsigned channel_bytes = static_cast<unsigned>(s.h) * s.w * 4u;
    const unsigned pair_bytes = 2 * channel_bytes;
    const int pairs = s.c_in >> 1;
    const size_t image_elems = static_cast<size_t>(s.c_in) * s.h * s.w;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(p.input + static_cast<size_t>(image) * image_elems), 0, static_cast<int>(image_elems * 4), 0x00020000);
    const float *a_lane = lds_w + (lh * 32 + li) * PITCH;
    float *out_image = p.out + static_cast<size_t>(image) * s.c_out * p.spatial;
    // 128-bit store path (WIDE): the wavefront's 32 × 32 results go through an LDS tile of its own, 16 channels at a time,
    // and leave as rows of four pixels per lane (lane -> channel row lane/8 (+8), pixels 4·(lane%8) .. +3).
    float *stage = reinterpret_cast<float *>(strip_lds + static_cast<size_t>(s.c_in) * 32 * PITCH * 4 + 16) +
                   (tid >> 6) * (16 * kStripStagePitch);
    float bias_wide[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}};
    if constexpr (WIDE) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int oc = oc0 + h * 16 + q * 8 + (lane >> 3);
                bias_wide[h][q] = (p.bias && oc < s.c_out) ? p.bias[oc] : 0.0f;
            }
    }

    // (An earlier form delayed the wavefronts sharing a SIMD by a quarter of a block each at start-up, reading their slot
    // from the hardware-id register; with operands requested two channel pairs ahead it no longer gains anything —
    // config 2 forward: 130.1 µs with it, 129.8 µs without; grad_input 137.2 against 138.7 µs — and is gone.)
    for (;;) {
        unsigned claimed = 0;
        if (lane == 0) claimed = atomicAdd(counter, 1u);
        const int blk = __builtin_amdgcn_readfirstlane(claimed);
        if (blk >= nblocks) break;

        const int px = (first + blk) * 32 + li;
        const bool valid = px < p.spatial;
        unsigned off[kStripTaps];
        {
            const int oy = px / s.ow, ox = px - oy * s.ow;
            const int iy0 = oy * s.stride_h - s.pad_h, ix0 = ox * s.stride_w - s.pad_w;
#pragma unroll
            for (int tap = 0; tap < kStripTaps; ++tap) {
                const int ky = tap / s.kw, kx = tap - ky * s.kw;
                const int iy = iy0 + ky * s.dil_h, ix = ix0 + kx * s.dil_w;
                const bool inside = valid && static_cast<unsigned>(iy) < static_cast<unsigned>(s.h) &&
                                    static_cast<unsigned>(ix) < static_cast<unsigned>(s.w);
                off[tap] = inside ? lh * channel_bytes + static_cast<unsigned>(iy * s.w + ix) * 4u : 0x80000000u;
            }
        }
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

        auto load_b = [&](float (&dst)[kStripTaps], int pair) {
            // (readfirstlane keeps the scalar offset in an SGPR; left to itself the compiler may move the
            // loop-carried value to a VGPR and wrap every buffer load in a uniformity loop.)
            const unsigned soff = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(pair) * pair_bytes);
#pragma unroll
            for (int tap = 0; tap < kStripTaps; ++tap)
                dst[tap] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, off[tap], soff, 0));
        };
        auto load_a = [&](float (&dst)[kStripTaps], int pair) {
            const float *src = a_lane + pair * (64 * PITCH);
            if constexpr (PITCH == 12) {  // 16-byte aligned rows: three 128-bit reads
#pragma unroll
                for (int q = 0; q < 3; ++q) {
                    const f32x4 v = *reinterpret_cast<const f32x4 *>(src + 4 * q);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (4 * q + e < kStripTaps) dst[4 * q + e] = v[e];
                }
            } else {
#pragma unroll
                for (int tap = 0; tap < kStripTaps; ++tap) dst[tap] = src[tap];
            }
        };
        // One channel pair: the operands of the pair after next are requested, then nine MFMAs run on this pair's;
        // three register sets in rotation (one pair ahead leaves the loads too little time: 157 -> 149 µs at
        // config 2; a fourth set spills).  Scheduling fences: without them the compiler sinks each load to just
        // before its use to save registers, which leaves the loads no time to complete.
        auto pair_body = [&](const float (&a_use)[kStripTaps], const float (&b_use)[kStripTaps], float (&a_next)[kStripTaps],
                             float (&b_next)[kStripTaps], int pair) {
            const int following = pair + 2 < pairs ? pair + 2 : pairs - 1;  // past the end: a re-read (unused)
            load_b(b_next, following);
            load_a(a_next, following);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int tap = 0; tap < kStripTaps; ++tap)
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_use[tap], b_use[tap], acc, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        };
        float a0[kStripTaps], a1[kStripTaps], a2[kStripTaps], b0[kStripTaps], b1[kStripTaps], b2[kStripTaps];
        load_b(b0, 0);
        load_a(a0, 0);
        load_b(b1, pairs > 1 ? 1 : 0);
        load_a(a1, pairs > 1 ? 1 : 0);
        int pair = 0;
        for (; pair + 3 <= pairs; pair += 3) {
            pair_body(a0, b0, a2, b2, pair);
            pair_body(a1, b1, a0, b0, pair + 1);
            pair_body(a2, b2, a1, b1, pair + 2);
        }
        if (pair < pairs) pair_body(a0, b0, a2, b2, pair);
        if (pair + 1 < pairs) pair_body(a1, b1, a0, b0, pair + 1);

        // The activation is wavefront-uniform: GELU takes a copy of the store code of its own, ReLU and none share a
        // branch-free one (decided per element, the stores of a block were cut into a dozen basic blocks).
        auto store_block = [&](auto &&act) {
            if constexpr (WIDE) {
                const int px4 = (first + blk) * 32 + (lane & 7) * 4;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
#pragma unroll
                    for (int rr = 0; rr < 8; ++rr) {
                        const int r = h * 8 + rr;
                        stage[(((r >> 2) & 1) * 8 + lh * 4 + (r & 3)) * kStripStagePitch + li] = acc[r];
                    }
#pragma unroll
                    for (int q = 0; q < 2; ++q) {
                        const int row = q * 8 + (lane >> 3);
                        const f32x4 v = *reinterpret_cast<const f32x4 *>(stage + row * kStripStagePitch + (lane & 7) * 4);
                        const int oc = oc0 + h * 16 + row;
                        f32x4 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) o[e] = act(v[e] + bias_wide[h][q]);
                        if (oc < s.c_out && px4 < p.spatial)
                            *reinterpret_cast<f32x4 *>(out_image + static_cast<size_t>(oc) * p.spatial + px4) = o;
                    }
                }
            } else if (valid) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int oc = oc0 + (r >> 2) * 8 + lh * 4 + (r & 3);
                    if (oc < s.c_out)  // (the bias is re-read per block: sixteen registers are worth more in the main loop)
                        out_image[static_cast<size_t>(oc) * p.spatial + px] = act(acc[r] + (p.bias ? p.bias[oc] : 0.0f));
                }
            }
        };
        if (p.activation == ST_HIP_ACT_GELU) store_block([](float v) { return gelu_tanh(v); });
        else store_block([relu = p.activation == ST_HIP_ACT_RELU](float v) { return relu_or_identity(v, relu); });
    }
}

// (A kernel template loses its host-side launch stub with this compiler when its body uses some builtins, hence
// plain kernels around the templated body.)
__global__ __launch_bounds__(kStripThreads) void conv2d_f32_strip12_kernel(StripArgs p) { conv2d_f32_strip_body<12, false>(p); }
__global__ __launch_bounds__(kStripThreads) void conv2d_f32_strip12_wide_kernel(StripArgs p) { conv2d_f32_strip_body<12, true>(p); }
__global__ __launch_bounds__(kStripThreads) void conv2d_f32_strip9_kernel(StripArgs p) { conv2d_f32_strip_body<9, false>(p); }

// Splits `shape` into strip workgroups.  False when the shape does not fit the kernel, or (unless `forced`) when
// the split would leave more than a fifth of the chip's SIMD time idle.
bool plan_strip(const ConvShape &shape, bool forced, StripArgs &args)
{
    if (shape.kh * shape.kw != kStripTaps || shape.c_in % 2 != 0 || shape.c_in > kStripMaxChannels) return false;
    const long long spatial = static_cast<long long>(shape.oh) * shape.ow;
    const long long blocks = (spatial + 31) / 32;
    const long long strips = (shape.c_out + 31) / 32;
    long long chunks = 1;
    while (shape.batch * strips * chunks < 256 && blocks / (chunks + 1) >= 16) ++chunks;
    const long long per_chunk = (blocks + chunks - 1) / chunks;
    chunks = (blocks + per_chunk - 1) / per_chunk;
    const long long total = shape.batch * strips * chunks;
    if (total > 0x7fffffff) return false;
    // Cost in 32×32 blocks per SIMD: one workgroup per compute unit at a time, its blocks spread over four SIMDs.
    const long long rounds = (total + 255) / 256;
    const double cost = static_cast<double>(rounds) * static_cast<double>((per_chunk + 3) / 4);
    const double ideal = static_cast<double>(shape.batch) * strips * blocks / 1024.0;
    if (!forced && ideal < 0.8 * cost) return false;
    args.spatial = static_cast<int>(spatial);
    args.blocks_per_image = static_cast<int>(blocks);
    args.chunks = static_cast<int>(chunks);
    args.blocks_per_chunk = static_cast<int>(per_chunk);
    args.oc_strips = static_cast<int>(strips);
    args.total = static_cast<int>(total);
    args.xcd_swizzle = total % 8 == 0 ? 1 : 0;
    return true;
}

hipError_t launch_strip(StripArgs args, int which, hipStream_t stream)
{
    size_t lds_bytes = strip_lds_bytes(args.s.c_in);
    if (which == ST_HIP_CONV_KERNEL_STRIP12_WIDE) lds_bytes += kStripStageBytes;
    auto kernel = which == ST_HIP_CONV_KERNEL_STRIP12_WIDE ? conv2d_f32_strip12_wide_kernel
                  : which == ST_HIP_CONV_KERNEL_STRIP12    ? conv2d_f32_strip12_kernel
                                                           : conv2d_f32_strip9_kernel;
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(args.total)), dim3(kStripThreads), lds_bytes, stream, args);
    return hipGetLastError();
}

template <int BM>
hipError_t launch_ring(ConvArgs args, hipStream_t stream)
{
    args.tiles_oc = (args.s.c_out + BM - 1) / BM;
    args.tiles_px = (args.spatial + 63) / 64;
    const size_t tiles = static_cast<size_t>(args.tiles_oc) * args.tiles_px * static_cast<size_t>(args.s.batch);
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    args.xcd_swizzle = (args.s.batch % 8 == 0) ? 1 : 0;
    for (int j = 0; j < 64; ++j) {
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

// Adds the partial planes of a k-sliced launch in slice order (so the result does not depend on scheduling), then bias
// and activation.  One thread per output value; eight planes are requested together so the loads overlap.
__global__ __launch_bounds__(256) void conv_slice_reduce_kernel(size_t count, int slices, int c_out, int spatial, int activation,
                                                                const float *partial, const float *bias, float *out)
{
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= count) return;
    float value = 0.0f;
    for (int s0 = 0; s0 < slices; s0 += 8) {
        float part[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) part[j] = (s0 + j < slices) ? partial[(s0 + j) * count + idx] : 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) value += part[j];
    }
    if (bias) value += bias[(idx / spatial) % c_out];
    out[idx] = apply_activation(value, activation);
}

// How many slices the reduction of `shape` is cut into: none unless the general kernel's tiles would leave half of the
// compute units idle while each walks at least 48 k-tiles (a k-tile costs a workgroup 0.5 to 1 µs of load latency
// whatever the tile count, so 48 of them are 25 to 50 µs); then enough for about four workgroups per compute unit,
// at least 8 k-tiles per slice, and at most 64 MB of partial planes.
int conv_k_slices(const ConvShape &shape)
{
    const size_t K = static_cast<size_t>(shape.c_in) * shape.kh * shape.kw, k_steps = (K + 15) / 16;
    const size_t spatial = static_cast<size_t>(shape.oh) * shape.ow;
    const size_t tiles = static_cast<size_t>(shape.batch) * ((spatial + 63) / 64) * ((shape.c_out + (shape.c_out > 64 ? 127 : 63)) / (shape.c_out > 64 ? 128 : 64));
    if (tiles > 128 || k_steps < 48) return 1;
    size_t slices = std::min<size_t>(1024 / tiles, k_steps / 8);
    const size_t plane_bytes = static_cast<size_t>(shape.batch) * shape.c_out * spatial * sizeof(float);
    while (slices > 1 && slices * plane_bytes > (64u << 20)) --slices;
    return static_cast<int>(std::max<size_t>(slices, 1));
}

template <int BM, int BN, int BK, int WM, int WN, bool TRANSPOSED = false>
hipError_t launch_tile(ConvArgs args, bool vec, hipStream_t stream, unsigned slices = 1)
{
    args.tiles_oc = (args.s.c_out + BM - 1) / BM;
    args.tiles_px = (args.spatial + BN - 1) / BN;
    const size_t tiles = static_cast<size_t>(args.tiles_oc) * args.tiles_px * static_cast<size_t>(args.s.batch);
    if (tiles > 0x7fffffffu) return hipErrorInvalidConfiguration;
    args.xcd_swizzle = (args.s.batch % 8 == 0) ? 1 : 0;
    const size_t k_padded = (static_cast<size_t>(std::min(args.K, kConvTableEntries)) + 15) & ~static_cast<size_t>(15);
    const size_t lds_bytes = k_padded * sizeof(int2) +
                             2 * (static_cast<size_t>(BM) * (BK + 4) + static_cast<size_t>(BK) * (BN + 8)) * sizeof(float);
    const dim3 grid(static_cast<unsigned>(tiles), slices);
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

// Kernel family forced by st_hip_conv2d_force_family (a diagnostic hook: the parity tests use it to run every family
// on small shapes); ST_HIP_CONV_FAMILY_AUTO in normal use.
std::atomic<int> g_forced_family{ST_HIP_CONV_FAMILY_AUTO};

// One to four output channels over many pixels (the last layer of an image generator, a regression head): an MFMA tile
// of 64 output channels would be padding from the fourth row on, and the layer is a stream over the input.  Here a
// thread owns one output pixel and all CO channels; the weights are the same for the whole wavefront and come through
// the scalar cache, the input through the vector cache, neighbouring pixels sharing most of their taps.
template <int CO>
__global__ __launch_bounds__(256) void conv2d_f32_direct_kernel(ConvArgs p)
{
    const ConvShape &s = p.s;
    const int px = static_cast<int>(blockIdx.x) * 256 + static_cast<int>(threadIdx.x);
    const int image = static_cast<int>(blockIdx.y);
    if (px >= p.spatial) return;
    const int oy = px / s.ow, ox = px - oy * s.ow;
    const int iy0 = oy * s.stride_h - s.pad_h, ix0 = ox * s.stride_w - s.pad_w;
    const size_t plane_elems = static_cast<size_t>(s.h) * s.w;
    const float *in = p.input + static_cast<size_t>(image) * s.c_in * plane_elems;
    const int K = p.K;
    float acc[CO];
#pragma unroll
    for (int co = 0; co < CO; ++co) acc[co] = 0.0f;
    for (int ci = 0; ci < s.c_in; ++ci) {
        const float *plane = in + static_cast<size_t>(ci) * plane_elems;
        const float *w_ci = p.weight + static_cast<size_t>(ci) * s.kh * s.kw;
        for (int ky = 0; ky < s.kh; ++ky) {
            const int iy = iy0 + ky * s.dil_h;
            const bool row_ok = iy >= 0 && iy < s.h;
            const float *row = plane + static_cast<size_t>(row_ok ? iy : 0) * s.w;
            for (int kx = 0; kx < s.kw; ++kx) {
                const int ix = ix0 + kx * s.dil_w;
                const float v = (row_ok && ix >= 0 && ix < s.w) ? row[ix] : 0.0f;
                const float *w_tap = w_ci + ky * s.kw + kx;
#pragma unroll
                for (int co = 0; co < CO; ++co) acc[co] = fmaf(v, w_tap[static_cast<size_t>(co) * K], acc[co]);
            }
        }
    }
#pragma unroll
    for (int co = 0; co < CO; ++co) {
        const float value = acc[co] + (p.bias ? p.bias[co] : -0.0f);
        p.out[(static_cast<size_t>(image) * CO + co) * p.spatial + px] = apply_activation(value, p.activation);
    }
}

// The same for unit stride and dilation along x and a kernel width known at compile time: a thread owns four adjacent
// pixels of an output row, so that a row segment of KW + 3 input values (one 16-byte load at any alignment plus KW - 1
// single ones) feeds 4·KW·CO multiply-adds, and the weights (at most 64 KB) are read from LDS, every lane the same word.
// KH: the kernel height when it equals KW and is at most 5 (the loop over its rows is then unrolled, so that the loads of all rows of
// a channel are in flight together: a thread's chain of load → multiply-add steps is what bounds this kernel), else 0.
template <int CO, int KW, int KH>
__global__ __launch_bounds__(256) void conv2d_f32_direct_rows_kernel(ConvArgs p)
{
    typedef float direct_f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
    extern __shared__ float direct_weights[];  // CO × K, as stored
    const ConvShape &s = p.s;
    const int K = p.K;
    for (int i = static_cast<int>(threadIdx.x); i < CO * K; i += 256) direct_weights[i] = p.weight[i];
    __syncthreads();
    const int quads = (s.ow + 3) / 4;  // threads per output row
    const int item = static_cast<int>(blockIdx.x) * 256 + static_cast<int>(threadIdx.x);
    if (item >= s.oh * quads) return;
    const int oy = item / quads, ox0 = (item - oy * quads) * 4;
    const int image = static_cast<int>(blockIdx.y);
    const int iy0 = oy * s.stride_h - s.pad_h, ix0 = ox0 - s.pad_w;
    constexpr int SEG = KW + 3;
    const bool inside_x = ix0 >= 0 && ix0 + SEG <= s.w;
    const size_t plane_elems = static_cast<size_t>(s.h) * s.w;
    const float *in = p.input + static_cast<size_t>(image) * s.c_in * plane_elems;
    float acc[CO][4];
#pragma unroll
    for (int co = 0; co < CO; ++co)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[co][j] = 0.0f;
    const int kh = KH > 0 ? KH : s.kh;
#pragma unroll 2
    for (int ci = 0; ci < s.c_in; ++ci) {
        const float *plane = in + static_cast<size_t>(ci) * plane_elems;
#pragma unroll
        for (int ky = 0; ky < kh; ++ky) {
            const int iy = iy0 + ky * s.dil_h;
            const bool row_ok = iy >= 0 && iy < s.h;  // a row of padding reads row 0 and counts as zeros
            const float *row = plane + static_cast<size_t>(row_ok ? iy : 0) * s.w;
            float v[SEG];
            if (inside_x) {
                const direct_f32x4_a4 t = *reinterpret_cast<const direct_f32x4_a4 *>(row + ix0);
                v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3];
#pragma unroll
                for (int i = 4; i < SEG; ++i) v[i] = row[ix0 + i];
            } else {
#pragma unroll
                for (int i = 0; i < SEG; ++i) {
                    const int ix = ix0 + i;
                    v[i] = (ix >= 0 && ix < s.w) ? row[ix] : 0.0f;
                }
            }
#pragma unroll
            for (int i = 0; i < SEG; ++i) v[i] = row_ok ? v[i] : 0.0f;
            const float *taps = direct_weights + (ci * kh + ky) * KW;
#pragma unroll
            for (int kx = 0; kx < KW; ++kx)
#pragma unroll
                for (int co = 0; co < CO; ++co) {
                    const float weight = taps[co * K + kx];
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[co][j] = fmaf(v[j + kx], weight, acc[co][j]);
                }
        }
    }
#pragma unroll
    for (int co = 0; co < CO; ++co) {
        const float b = p.bias ? p.bias[co] : -0.0f;
        float *dst = p.out + (static_cast<size_t>(image) * CO + co) * p.spatial + static_cast<size_t>(oy) * s.ow + ox0;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (ox0 + j < s.ow) dst[j] = apply_activation(acc[co][j] + b, p.activation);
    }
}

template <int CO, int KW>
hipError_t launch_direct_rows(const ConvArgs &args, hipStream_t stream)
{
    const size_t items = static_cast<size_t>(args.s.oh) * ((args.s.ow + 3) / 4);
    const dim3 grid(static_cast<unsigned>((items + 255) / 256), static_cast<unsigned>(args.s.batch));
    const size_t lds_bytes = static_cast<size_t>(CO) * args.K * sizeof(float);
    if (args.s.kh == KW && KW <= 5) hipLaunchKernelGGL((conv2d_f32_direct_rows_kernel<CO, KW, KW>), grid, dim3(256), lds_bytes, stream, args);
    else hipLaunchKernelGGL((conv2d_f32_direct_rows_kernel<CO, KW, 0>), grid, dim3(256), lds_bytes, stream, args);
    return hipGetLastError();
}

template <int CO>
hipError_t launch_direct_rows_for(const ConvArgs &args, hipStream_t stream)
{
    switch (args.s.kw) {
    case 1: return launch_direct_rows<CO, 1>(args, stream);
    case 3: return launch_direct_rows<CO, 3>(args, stream);
    case 5: return launch_direct_rows<CO, 5>(args, stream);
    default: return launch_direct_rows<CO, 7>(args, stream);
    }
}

template <int CO>
hipError_t launch_direct(const ConvArgs &args, hipStream_t stream)
{
    const ConvShape &s = args.s;
    if (s.stride_w == 1 && s.dil_w == 1 && (s.kw == 1 || s.kw == 3 || s.kw == 5 || s.kw == 7) &&
        static_cast<size_t>(CO) * args.K * sizeof(float) <= 64 * 1024)
        return launch_direct_rows_for<CO>(args, stream);
    const dim3 grid(static_cast<unsigned>((args.spatial + 255) / 256), static_cast<unsigned>(args.s.batch));
    hipLaunchKernelGGL(conv2d_f32_direct_kernel<CO>, grid, dim3(256), 0, stream, args);
    return hipGetLastError();
}

// At most four output channels over at least 65536 output pixels in all, kernels of more than one tap (8 × 64 × 256 × 256
// → 3, 3×3: 440 → 104 µs; 7×7: 2751 → 433 µs; 16 × 32 × 128 × 128 → 1: 118 → 35 µs.  With 16384 pixels there are too few
// threads for their serial walk over c_in·kh: 4 × 128 × 64 × 64 → 4 takes 64 µs on the tile kernel, 127 µs here).
bool conv_direct_applies(const ConvShape &shape)
{
    return shape.c_out <= 4 && shape.kh * shape.kw > 1 && shape.batch <= 65535 &&
           static_cast<long long>(shape.batch) * shape.oh * shape.ow >= 65536;
}

// The dispatcher's decision for `shape`: one of ST_HIP_CONV_KERNEL_*, or 0 when a forced family cannot serve the
// shape.  `strip` is filled when a strip kernel is chosen.
int choose_conv_kernel(const ConvShape &shape, bool weight_aligned, bool out_aligned, int forced, StripArgs &strip,
                       bool allow_slices = true)
{
    const int K = shape.c_in * shape.kh * shape.kw;
    const int spatial = shape.oh * shape.ow;
    const bool vec = (K % 4 == 0) && weight_aligned;
    // Both direct-load kernels address one image through 32-bit byte offsets with the top bits spare.
    const bool image_ok = static_cast<size_t>(shape.c_in) * shape.h * shape.w * 4 < (1ull << 30);
    // 8 wavefronts of 32×32 per 128×64 tile measured best for wide layers (128×128 tiles, 32-deep k-tiles and
    // 4-wavefront layouts were all 10-20 % slower on the 64->128 channel 56×56 case).
    const bool ring_ok = vec && K % 16 == 0 && shape.kh * shape.kw <= 64 && image_ok &&
                         (static_cast<size_t>(shape.pad_h) * shape.w + shape.pad_w) * 4 < (1ull << 30) &&
                         (static_cast<size_t>(shape.oh + 64) * shape.stride_h * shape.w + static_cast<size_t>(shape.ow) * shape.stride_w) * 4 < (1ull << 30) &&
                         static_cast<size_t>(shape.c_out) * K * 4 < (1ull << 31);
    auto strip_kernel = [&]() {
        if (strip_pitch(shape.c_in) != 12) return ST_HIP_CONV_KERNEL_STRIP9;
        const bool wide = spatial % 4 == 0 && out_aligned &&
                          strip_lds_bytes(shape.c_in) + kStripStageBytes <= 160 * 1024;
        return wide ? ST_HIP_CONV_KERNEL_STRIP12_WIDE : ST_HIP_CONV_KERNEL_STRIP12;
    };
    switch (forced) {
    case ST_HIP_CONV_FAMILY_TILE: return ST_HIP_CONV_KERNEL_TILE;
    case ST_HIP_CONV_FAMILY_RING: return ring_ok ? ST_HIP_CONV_KERNEL_RING : 0;
    case ST_HIP_CONV_FAMILY_STRIP: return image_ok && plan_strip(shape, true, strip) ? strip_kernel() : 0;
    default: break;
    }
    // Few tiles with a long reduction (deep layers on tiny planes at small batch, one or a few output channels): every
    // kernel here walks the reduction serially inside a workgroup, so the chip is filled by cutting the reduction.
    if (conv_direct_applies(shape)) return ST_HIP_CONV_KERNEL_DIRECT;
    if (allow_slices && conv_k_slices(shape) > 1) return ST_HIP_CONV_KERNEL_TILE_KSLICED;
    if (!ring_ok) return ST_HIP_CONV_KERNEL_TILE;
    // The ring kernel has the better steady state (several rounds of 128×64 tiles per compute unit); the strip
    // kernel, balanced to the single SIMD, wins when the ring kernel's tiles would fill the chip fewer than
    // 1.75 times (1024 resident tiles) and for 64 or fewer output channels.
    const long long ring_tiles = static_cast<long long>(shape.batch) * ((spatial + 63) / 64) * ((shape.c_out + 127) / 128);
    const bool prefer_strip = shape.c_out <= 64 || ring_tiles < 1792;
    if (prefer_strip && plan_strip(shape, false, strip)) return strip_kernel();
    return ST_HIP_CONV_KERNEL_RING;
}

}  // namespace

void set_conv_forced_family(int family) { g_forced_family.store(family, std::memory_order_relaxed); }

int planned_conv_kernel(const ConvShape &shape, bool weight_aligned, bool out_aligned)
{
    StripArgs strip;
    return choose_conv_kernel(shape, weight_aligned, out_aligned, g_forced_family.load(std::memory_order_relaxed), strip);
}

size_t conv2d_scratch_bytes(const ConvShape &shape, bool weight_aligned, bool out_aligned)
{
    StripArgs strip;
    if (choose_conv_kernel(shape, weight_aligned, out_aligned, g_forced_family.load(std::memory_order_relaxed), strip) !=
        ST_HIP_CONV_KERNEL_TILE_KSLICED)
        return 0;
    return static_cast<size_t>(conv_k_slices(shape)) * shape.batch * shape.c_out * shape.oh * shape.ow * sizeof(float);
}

hipError_t launch_conv2d_f32(const ConvShape &shape, int activation, const float *input, const float *weight,
                             const float *bias, float *out, hipStream_t stream, int scratch, size_t scratch_offset)
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
        (shape.kw - 1) * static_cast<long long>(shape.dil_w) > 0x7fff)
        return hipErrorInvalidValue;
    const bool weight_aligned = (reinterpret_cast<uintptr_t>(weight) & 15u) == 0;
    const bool out_aligned = (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    StripArgs strip;
    const int kernel = choose_conv_kernel(shape, weight_aligned, out_aligned,
                                          g_forced_family.load(std::memory_order_relaxed), strip, scratch == kConvScratchStream);
    switch (kernel) {
    case ST_HIP_CONV_KERNEL_TILE_KSLICED: {
        const size_t slices = static_cast<size_t>(conv_k_slices(shape));
        const size_t k_steps = (static_cast<size_t>(args.K) + 15) / 16, steps_per_slice = (k_steps + slices - 1) / slices;
        const size_t used = (k_steps + steps_per_slice - 1) / steps_per_slice;
        const size_t count = static_cast<size_t>(shape.batch) * shape.c_out * args.spatial;
        // The kernel's workgroup (tile, y) walks k-tiles [y·steps_per_slice, (y+1)·steps_per_slice) and writes plane y:
        // every launched slice has k-tiles, together they cover the reduction, and their planes fit the scratch asked for.
        if (used == 0 || used > slices || used > 65535 || (used - 1) * steps_per_slice >= k_steps || used * steps_per_slice < k_steps)
            return hipErrorInvalidConfiguration;
        void *workspace = nullptr;
        hipError_t rc = stream_workspace(stream, scratch_offset + slices * count * sizeof(float), &workspace);
        if (rc != hipSuccess) return rc;
        float *partial = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) + scratch_offset);
        args.out = partial;
        args.bias = nullptr;
        args.activation = ST_HIP_ACT_NONE;
        args.k_slice = static_cast<int>(steps_per_slice * 16);
        const bool vec = (args.K % 4 == 0) && weight_aligned;
        rc = shape.c_out > 64 ? launch_tile<128, 64, 16, 4, 2>(args, vec, stream, static_cast<unsigned>(used))
                              : launch_tile<64, 64, 16, 2, 2>(args, vec, stream, static_cast<unsigned>(used));
        if (rc != hipSuccess) return rc;
        hipLaunchKernelGGL(conv_slice_reduce_kernel, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, stream, count,
                           static_cast<int>(used), shape.c_out, args.spatial, activation, partial, bias, out);
        return hipGetLastError();
    }
    case ST_HIP_CONV_KERNEL_DIRECT:
        switch (shape.c_out) {
        case 1: return launch_direct<1>(args, stream);
        case 2: return launch_direct<2>(args, stream);
        case 3: return launch_direct<3>(args, stream);
        default: return launch_direct<4>(args, stream);
        }
    case ST_HIP_CONV_KERNEL_STRIP12:
    case ST_HIP_CONV_KERNEL_STRIP12_WIDE:
    case ST_HIP_CONV_KERNEL_STRIP9:
        strip.input = input;
        strip.weight = weight;
        strip.bias = bias;
        strip.out = out;
        strip.s = shape;
        strip.activation = activation;
        return launch_strip(strip, kernel, stream);
    case ST_HIP_CONV_KERNEL_RING: {
        // 128 output channels per tile unless that leaves half of the compute units without a tile (deep layers on
        // small planes: 512 channels on 7×7 are 32 × 1 × 4 tiles); 64-channel tiles then double the workgroups and
        // still run in one round (512→512 on 7×7: 196 → 151 µs; with 192 tiles of 128 channels, 768→768 7×7 with a
        // 7×7 kernel, the 384 tiles of 64 are slower: 1539 → 1837 µs).
        const long long tiles128 = static_cast<long long>(shape.batch) * ((args.spatial + 63) / 64) * ((shape.c_out + 127) / 128);
        return shape.c_out > 64 && tiles128 > 128 ? launch_ring<128>(args, stream) : launch_ring<64>(args, stream);
    }
    case ST_HIP_CONV_KERNEL_TILE: {
        const bool vec = (args.K % 4 == 0) && weight_aligned;
        if (shape.c_out > 64) return launch_tile<128, 64, 16, 4, 2>(args, vec, stream);
        return launch_tile<64, 64, 16, 2, 2>(args, vec, stream);
    }
    default:
        return hipErrorInvalidConfiguration;  // a forced family that cannot serve the shape (entry points check first)
    }
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
        (shape.kw - 1) * static_cast<long long>(shape.dil_w) > 0x7fff)
        return hipErrorInvalidValue;
    const bool vec = (args.K % 4 == 0) && ((reinterpret_cast<uintptr_t>(weight_ic_major) & 15u) == 0);
    if (shape.c_out > 64) return launch_tile<128, 64, 16, 4, 2, true>(args, vec, stream);
    return launch_tile<64, 64, 16, 2, 2, true>(args, vec, stream);
}

}  // namespace sthip
