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
};


// FULLK: c_in*kh*kw is a multiple of the 16-wide k-tile and weight rows are 16-byte aligned, so the loop
// carries no k bounds checks; weight rows past c_out are clamped to the last row (what they contribute
// only reaches output channels that are never stored).
template <int BM, int BN, int BK, int WM, int WN, bool VEC, bool FULLK>
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
        lut[k] = make_int2(ic * H * W + dy * W + dx, dy | (dx << 16));
    }

    // Every thread gathers one pixel column of the patch tile, rows (tid / BN) + B_ROW_STEP * r.
    const int px_local = tid % BN;
    const int krow0 = tid / BN;
    const int px = px0 + px_local;
    const bool px_valid = px < p.spatial;
    const int oy = px / s.ow, ox = px - oy * s.ow;
    const int iy0 = oy * s.stride_h - s.pad_h;
    const int ix0 = ox * s.stride_w - s.pad_w;
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
                const int iy = iy0 + (e.y & 0xffff);
                const int ix = ix0 + (e.y >> 16);
                if (static_cast<unsigned>(iy) < static_cast<unsigned>(H) &&
                    static_cast<unsigned>(ix) < static_cast<unsigned>(W))
                    v = img[base + e.x];
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

template <int BM, int BN, int BK, int WM, int WN>
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
        rc = launch(conv2d_f32_kernel<BM, BN, BK, WM, WN, true, true>);
    else if (vec)
        rc = launch(conv2d_f32_kernel<BM, BN, BK, WM, WN, true, false>);
    else
        rc = launch(conv2d_f32_kernel<BM, BN, BK, WM, WN, false, false>);
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
    if (shape.c_out > 64) return launch_tile<128, 64, 16, 4, 2>(args, vec, stream);
    return launch_tile<64, 64, 16, 2, 2>(args, vec, stream);
}

}  // namespace sthip
