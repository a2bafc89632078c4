// Conv2d backward on gfx950: gradients with respect to the input, the weight and the bias.
//
// Reference: Conv2d::backward → accumulate_from_grad_matrix, crates/st-nn/src/layers/conv.rs:780-813, with
// G = grad_output re-laid as (batch·OH·OW, C_out) (:750-778):
//   grad_weight = (Gᵀ · patches) · scale        (matmul_lhs_transpose_scaled, :791-795; scale = 1/batch)
//   grad_bias   = column sums of G · scale       (:796-799)
//   grad_input  = col2im(G · W)                  (:803-809, col2im :860-916)
// Neither the patch matrix, nor G, nor the (pixels × C_in·KH·KW) product is materialised here:
//   * grad_input is the adjoint convolution.  For stride 1 it IS a forward convolution of grad_output with the
//     taps flipped and the channel roles swapped (padding dil·(k−1) − pad), so it runs on the forward kernels;
//     other strides take the same implicit GEMM with the adjoint gather.
//   * grad_weight is an implicit GEMM  G_b(C_out × pixels) · patches_b(pixels × C_in·KH·KW)  summed over images:
//     C_out × C_in·KH·KW is small and the reduction long, so the images are split over workgroups, partial tiles
//     go to the stream's workspace and a second kernel adds them in a fixed order (reproducible) and scales.
//   * grad_bias is a per-channel sum over NCHW planes.
#include "device_math.h"
#include "kernels.h"

#include <algorithm>
#include <cmath>
#include <mutex>

namespace sthip {

// Scratch of the allocation-free grad_input entry point: the flipped, channel-swapped weights live here instead of
// in memory from hipMalloc.  Each GPU the library runs on holds its own copy of the array until the process ends.
// In host code the array's name is only a stand-in for the symbol: its device address on the current GPU comes from
// hipGetSymbolAddress (noalloc_scratch below), and only that pointer is ever passed to a kernel.
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void *scratch_ptr[kMaxDevices] = {};

}  // namespace

// Device address of `scratch` on the current GPU, resolved once per device.
hipError_t noalloc_scratch(void **out)
{
    int device = 0;
    hipError_t rc = hipGetDevice(&device);
    if (rc != hipSuccess) return rc;
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (scratch_ptr[device] == nullptr) {
        void *ptr = nullptr;
        rc = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (rc != hipSuccess) return rc;
        scratch_ptr[device] = ptr;
    }
    *out = scratch_ptr[device];
    return hipSuccess;
}

namespace {

// dst[ic][oc][ky][kx] = src[oc][ic][flip ? KH-1-ky : ky][flip ? KW-1-kx : kx]
__global__ __launch_bounds__(256) void conv_weight_to_adjoint_kernel(int c_out, int c_in, int kh, int kw, int flip,
                                                                     const float *src, float *dst)
{
    const size_t total = static_cast<size_t>(c_out) * c_in * kh * kw;  // (may exceed 2^31 values)
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    const int kx = static_cast<int>(i % kw);
    size_t rest = i / kw;
    const int ky = static_cast<int>(rest % kh);
    rest /= kh;
    const int oc = static_cast<int>(rest % c_out);
    const int ic = static_cast<int>(rest / c_out);
    const int sy = flip ? kh - 1 - ky : ky, sx = flip ? kw - 1 - kx : kx;
    dst[i] = src[((static_cast<size_t>(oc) * c_in + ic) * kh + sy) * kw + sx];
}

// col2im as a gather (crates/st-nn/src/layers/conv.rs:860-916 adds patch gradients into the input gradient patch by
// patch; here every input position collects the entries that land on it, in the same order: output rows ascending,
// then output columns ascending).  cols: [images][OH·OW][C_in·KH·KW], the product grad_outputᵀ · W of each image.
// One thread per input value.
__global__ __launch_bounds__(256) void conv_col2im_gather_kernel(ConvShape s, int images, const float *cols, float *grad_input)
{
    const size_t total = static_cast<size_t>(images) * s.c_in * s.h * s.w;
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    const int x = static_cast<int>(idx % s.w);
    size_t rest = idx / s.w;
    const int y = static_cast<int>(rest % s.h);
    rest /= s.h;
    const int ic = static_cast<int>(rest % s.c_in);
    const int image = static_cast<int>(rest / s.c_in);
    const int S = s.c_in * s.kh * s.kw;
    const float *image_cols = cols + static_cast<size_t>(image) * s.oh * s.ow * S + static_cast<size_t>(ic) * s.kh * s.kw;
    // Taps that can reach this position: (y + pad − ky·dil) a non-negative multiple of the stride below OH·stride.
    // Without dilation they are every stride-th ky, so the loop steps over the others (a 16×16 kernel at stride 16 has
    // one candidate per axis, not sixteen).
    const int step_y = s.dil_h == 1 ? s.stride_h : 1, step_x = s.dil_w == 1 ? s.stride_w : 1;
    int ky_last = s.kh - 1, kx_last = s.kw - 1;
    if (s.dil_h == 1) ky_last -= ((ky_last - (y + s.pad_h)) % step_y + step_y) % step_y;
    if (s.dil_w == 1) kx_last -= ((kx_last - (x + s.pad_w)) % step_x + step_x) % step_x;
    float sum = 0.0f;
    for (int ky = ky_last; ky >= 0; ky -= step_y) {  // descending ky = ascending output row
        const int ty = y + s.pad_h - ky * s.dil_h;
        if (ty < 0 || ty % s.stride_h != 0) continue;
        const int oy = ty / s.stride_h;
        if (oy >= s.oh) continue;
        for (int kx = kx_last; kx >= 0; kx -= step_x) {
            const int tx = x + s.pad_w - kx * s.dil_w;
            if (tx < 0 || tx % s.stride_w != 0) continue;
            const int ox = tx / s.stride_w;
            if (ox >= s.ow) continue;
            sum += image_cols[(static_cast<size_t>(oy) * s.ow + ox) * S + ky * s.kw + kx];
        }
    }
    grad_input[idx] = sum;
}

__device__ __forceinline__ float wave_sum64(float v)
{
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset);
    return v;
}

// partial[b][oc] = Σ_pixels grad_output[b][oc][pixel]; one wavefront per (b, oc) plane.
__global__ __launch_bounds__(256) void conv_grad_bias_partial_kernel(int planes, int spatial, const float *grad_output,
                                                                     float *partial)
{
    const int lane = threadIdx.x & 63;
    const int plane = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (plane >= planes) return;
    const float *src = grad_output + static_cast<size_t>(plane) * spatial;
    float sum = 0.0f;
    for (int i = lane; i < spatial; i += 64) sum += src[i];
    sum = wave_sum64(sum);
    if (lane == 0) partial[plane] = sum;
}

// out[i] = scale · Σ_c partial[c][i] in a fixed order: 16 outputs per workgroup, sixteen groups of lanes take every
// sixteenth chunk (four loads in flight each) and their partial sums are added through LDS.
__global__ __launch_bounds__(256) void conv_reduce_chunks_kernel(int chunks, size_t count, const float *partial, float scale,
                                                                 float *out)
{
    __shared__ float stage[16][17];
    const int col = threadIdx.x & 15, sub = threadIdx.x >> 4;
    const size_t i = static_cast<size_t>(blockIdx.x) * 16 + col;
    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (i < count) {
        int c = sub;
        for (; c + 48 < chunks; c += 64) {
            float t[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) t[u] = partial[static_cast<size_t>(c + 16 * u) * count + i];
#pragma unroll
            for (int u = 0; u < 4; ++u) sum[u] += t[u];
        }
        for (; c < chunks; c += 16) sum[0] += partial[static_cast<size_t>(c) * count + i];
    }
    stage[sub][col] = (sum[0] + sum[1]) + (sum[2] + sum[3]);
    __syncthreads();
    if (sub == 0 && i < count) {
        float total = stage[0][col];
#pragma unroll
        for (int k = 1; k < 16; ++k) total += stage[k][col];
        out[i] = total * scale;
    }
}

// The same sum, 128 bits per lane (count a multiple of 4, 16-byte aligned buffers): 128 outputs per workgroup, 32
// lanes side by side read 512 contiguous bytes of a chunk, eight groups of lanes take every eighth chunk (four loads
// in flight each), and the eight partial sums are added through LDS in a fixed order.
__global__ __launch_bounds__(256) void conv_reduce_chunks_vec_kernel(int chunks, size_t count4, const float4 *partial,
                                                                     float scale, float4 *out)
{
    __shared__ float4 stage[8][33];
    const int col = threadIdx.x & 31, sub = threadIdx.x >> 5;
    const size_t i = static_cast<size_t>(blockIdx.x) * 32 + col;
    float4 sum[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) sum[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    auto add = [](float4 &a, const float4 &b) { a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w; };
    if (i < count4) {
        int c = sub;
        for (; c + 24 < chunks; c += 32) {
            float4 t[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) t[u] = partial[static_cast<size_t>(c + 8 * u) * count4 + i];
#pragma unroll
            for (int u = 0; u < 4; ++u) add(sum[u], t[u]);
        }
        for (; c < chunks; c += 8) add(sum[0], partial[static_cast<size_t>(c) * count4 + i]);
    }
    add(sum[0], sum[1]);
    add(sum[2], sum[3]);
    add(sum[0], sum[2]);
    stage[sub][col] = sum[0];
    __syncthreads();
    if (sub == 0 && i < count4) {
        float4 total = stage[0][col];
#pragma unroll
        for (int k = 1; k < 8; ++k) add(total, stage[k][col]);
        out[i] = make_float4(total.x * scale, total.y * scale, total.z * scale, total.w * scale);
    }
}

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

struct GradWeightArgs {
    const float *input;        // (N, C_in, H, W)
    const float *grad_output;  // (N, C_out, OH, OW)
    float *partial;            // (chunks, C_out, S)
    ConvShape s;
    int S;                     // c_in * kh * kw
    int spatial;               // oh * ow
    int tiles_s;
    int steps_per_chunk;       // 16-pixel steps (numbered image by image) per workgroup
    int workgroups;            // tiles × chunks; the launch grid is this rounded up to a multiple of 8
};

// One workgroup: a (64·TM output channels) × (64·TN reduction columns s) tile of grad_weight, summed over the pixels
// of its images; four wavefronts in a 2×2 arrangement, each owning TM×TN 32×32 accumulators.  Per 16-pixel step the G
// tile (pixel-contiguous in NCHW) and the patch tile (gathered: a thread owns TN columns s, whose channel/tap offsets
// are fixed for the whole kernel) are fetched into registers while the MFMAs of the previous step run, then written to
// the other LDS stage.  The big tile (TM = 2, TN = 3: 128 × 192, three of which span a 3×3 layer's 576 columns exactly
// for 64 input channels) reads 5 fragments per 24 MFMAs instead of 2 per 4.
//
// SETS > 1: the workgroup is SETS such groups of four wavefronts working on the same tile.  Each takes its own run of
// steps (chunk·SETS + set) through LDS stages of its own; at the end the sets' accumulators are added through LDS in
// the order ((0 + 1) + 2) and set 0 stores the one partial tile — a third of the partial tiles, of the bytes the
// chunk reduction reads back, and of the store burst at the end of the launch, for the same wavefronts per SIMD.
template <bool VEC, int TM, int TN, int SETS = 1>
__device__ __forceinline__ void conv_grad_weight_body(const GradWeightArgs &p, float *As, float *Bs)
{
    constexpr int BM = 64 * TM, BN = 64 * TN, BK = 16;
    // Both tiles are kept pixel-contiguous (row = channel or patch column, 16 pixels + 4 words of padding), so that a
    // lane's four k-values of either operand are one conflict-free 128-bit LDS read.
    constexpr int A_STRIDE = BK + 4, B_STRIDE = BK + 4;
    constexpr int A_STAGE = BM * A_STRIDE, B_STAGE = BN * B_STRIDE;

    const int set = SETS > 1 ? __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 8)) : 0;
    float *const lds_all = As;  // (SETS > 1: As is the start of the workgroup's LDS, [set][A stages | B stages])
    if constexpr (SETS > 1) {
        As = lds_all + set * (2 * A_STAGE + 2 * B_STAGE);
        Bs = As + 2 * A_STAGE;
    }
    const int tid = threadIdx.x & 255;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: the pixel bookkeeping below stays off the VALU
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, lh = lane >> 5;
    const ConvShape &s = p.s;
    const int H = s.h, W = s.w;

    // Workgroup ids go round-robin over the 8 XCDs; give each XCD a contiguous run of (chunk, tile) pairs so that
    // the tiles that share a chunk's pixels find them in the same L2.
    // (The grid is padded to a multiple of 8; the padding workgroups leave at once.)
    int bid = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    if (bid >= p.workgroups) return;
    const int tile_s = bid % p.tiles_s;
    bid /= p.tiles_s;
    const int tiles_oc = (s.c_out + BM - 1) / BM;
    const int tile_oc = bid % tiles_oc;
    const int chunk = (bid / tiles_oc) * SETS + set;
    const int oc0 = tile_oc * BM, s0 = tile_s * BN;

    // This thread's patch columns (lane + 64·j) and their fixed taps.
    const int khw = s.kh * s.kw;
    bool col_valid[TN];
    int dy[TN], dx[TN], tap_offset[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int col = s0 + j * 64 + lane;
        col_valid[j] = col < p.S;
        const int ic = col_valid[j] ? col / khw : 0;
        const int rem = col_valid[j] ? col - ic * khw : 0;
        const int ky = rem / s.kw, kx = rem - ky * s.kw;
        dy[j] = ky * s.dil_h - s.pad_h;
        dx[j] = kx * s.dil_w - s.pad_w;
        tap_offset[j] = ic * H * W;
    }
    const int prow0 = wave * 4;  // patch rows prow0 .. prow0+3 of a step: four consecutive pixels, the same for all lanes

    // G tile: a thread loads 4 consecutive pixels of the channel rows a_row + 64·i.
    const int a_row = tid >> 2, a_c4 = (tid & 3) * 4;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const int steps_per_image = (p.spatial + BK - 1) / BK;
    const int first_step = chunk * p.steps_per_chunk;
    const int total_steps = max(0, min(s.batch * steps_per_image, first_step + p.steps_per_chunk) - first_step);

    // (oy, ox) of this wavefront's first pixel of the step being loaded, advanced by 16 pixels per step without
    // divisions.  Memory is addressed through per-image buffer descriptors with 32-bit offsets; anything outside
    // (padding, pixels past the end, channels past C_out) gets an out-of-range offset and reads as zero.
    int load_image = first_step / steps_per_image, load_step = first_step - load_image * steps_per_image;
    int oy, ox;
    {
        const int first_pixel = load_step * BK + prow0;
        oy = first_pixel / s.ow;
        ox = first_pixel - oy * s.ow;
    }
    const unsigned image_bytes = static_cast<unsigned>(s.c_in) * H * W * 4u;
    const unsigned grad_bytes = static_cast<unsigned>(s.c_out) * p.spatial * 4u;
    constexpr unsigned kOutside = 0x80000000u;
    unsigned a_base[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i)
        a_base[i] = oc0 + a_row + 64 * i < s.c_out ? (static_cast<unsigned>(oc0 + a_row + 64 * i) * p.spatial + a_c4) * 4u : kOutside;

    u32x4_t ra[TM];
    float rb[TN][4];
    auto load_global = [&]() {
        const int p0 = load_step * BK;
        const __amdgpu_buffer_rsrc_t rsrc_g = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float *>(p.grad_output + static_cast<size_t>(load_image) * s.c_out * p.spatial), 0,
            static_cast<int>(grad_bytes), 0x00020000);
        const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float *>(p.input + static_cast<size_t>(load_image) * s.c_in * H * W), 0, static_cast<int>(image_bytes),
            0x00020000);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            if (VEC) {  // spatial % 4 == 0: a 16-byte chunk is entirely inside its channel row or entirely past it
                const unsigned off = (p0 + a_c4 < p.spatial) ? a_base[i] + static_cast<unsigned>(p0) * 4u : kOutside;
                ra[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_g, off, 0, 0);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const unsigned off = (p0 + a_c4 + e < p.spatial) ? a_base[i] + static_cast<unsigned>(p0 + e) * 4u : kOutside;
                    ra[i][e] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_g, off, 0, 0);
                }
            }
        }
        // The four pixels are the same for every lane of the wavefront (lanes differ in their taps), so whether they
        // sit in one image row is a scalar question.  If they do, and no lane's tap straddles the left or right
        // border, the four values are one 128-bit load (dword-aligned is enough for buffer loads).
        const bool one_row = s.stride_w == 1 && ox + 3 < s.ow && p0 + prow0 + 3 < p.spatial;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            bool vector_done = false;
            if (one_row) {
                const int iy = oy * s.stride_h + dy[j], ix0 = ox + dx[j];
                const bool row_ok = col_valid[j] && static_cast<unsigned>(iy) < static_cast<unsigned>(H);
                const bool full = row_ok && ix0 >= 0 && ix0 + 3 < W;
                if (__builtin_amdgcn_ballot_w64(row_ok && !full) == 0) {
                    const unsigned off = full ? static_cast<unsigned>(tap_offset[j] + iy * W + ix0) * 4u : kOutside;
                    const u32x4_t raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, off, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; ++r) rb[j][r] = __uint_as_float(raw[r]);
                    vector_done = true;
                }
            }
            if (!vector_done) {
                int py = oy, px = ox;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int iy = py * s.stride_h + dy[j], ix = px * s.stride_w + dx[j];
                    const bool inside = col_valid[j] && p0 + prow0 + r < p.spatial &&
                                        static_cast<unsigned>(iy) < static_cast<unsigned>(H) &&
                                        static_cast<unsigned>(ix) < static_cast<unsigned>(W);
                    const unsigned off = inside ? static_cast<unsigned>(tap_offset[j] + iy * W + ix) * 4u : kOutside;
                    rb[j][r] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc_x, off, 0, 0));
                    if (++px == s.ow) {
                        px = 0;
                        ++py;
                    }
                }
            }
        }
        // advance to the next step (possibly the next image)
        if (++load_step == steps_per_image) {
            load_step = 0;
            ++load_image;
            oy = prow0 / s.ow;
            ox = prow0 - oy * s.ow;
        } else {
            ox += BK;
            while (ox >= s.ow) {
                ox -= s.ow;
                ++oy;
            }
        }
    };
    auto store_lds = [&](int stage) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
            *reinterpret_cast<u32x4_t *>(&As[stage * A_STAGE + (a_row + 64 * i) * A_STRIDE + a_c4]) = ra[i];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            f32x4 packed;
            packed[0] = rb[j][0]; packed[1] = rb[j][1]; packed[2] = rb[j][2]; packed[3] = rb[j][3];
            *reinterpret_cast<f32x4 *>(&Bs[stage * B_STAGE + (j * 64 + lane) * B_STRIDE + prow0]) = packed;
        }
    };
    auto compute = [&](int stage) {
        const float *as = As + stage * A_STAGE;
        const float *bs = Bs + stage * B_STAGE;
#pragma unroll
        for (int kk = 0; kk < BK / 8; ++kk) {
            f32x4 av[TM], bv[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                av[i] = *reinterpret_cast<const f32x4 *>(&as[(wm * 32 * TM + i * 32 + li) * A_STRIDE + kk * 8 + lh * 4]);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                bv[j] = *reinterpret_cast<const f32x4 *>(&bs[(wn * 32 * TN + j * 32 + li) * B_STRIDE + kk * 8 + lh * 4]);
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i][t], bv[j][t], acc[i][j], 0, 0, 0);
        }
    };

    if (total_steps > 0) {
        load_global();
        store_lds(0);
    }
    __syncthreads();
    // (SETS > 1: every set goes through the barriers of the longest run; a set whose run is shorter idles.)
    const int barrier_steps = SETS > 1 ? p.steps_per_chunk : total_steps;
    for (int t = 0; t < barrier_steps; ++t) {
        const bool more = t + 1 < total_steps;
        if (more) load_global();
        if (t < total_steps) compute(t & 1);
        if (more) store_lds((t + 1) & 1);
        __syncthreads();
    }

    if constexpr (SETS > 1) {
        // Thread t's 16·TM·TN accumulator values as 128-bit pieces e at (e·256 + t)·16 bytes: conflict-free both ways.
        static_assert(TM * TN * 16 * 256 * 4 <= SETS * (2 * A_STAGE + 2 * B_STAGE) * 4, "the tile fits the workgroup's LDS");
        f32x4 *exchange = reinterpret_cast<f32x4 *>(lds_all);
#pragma unroll
        for (int other = 1; other < SETS; ++other) {
            if (set == other) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            exchange[((i * TN + j) * 4 + q) * 256 + tid] =
                                f32x4{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
            }
            __syncthreads();
            if (set == 0) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const f32x4 v = exchange[((i * TN + j) * 4 + q) * 256 + tid];
                            acc[i][j][4 * q] += v[0];
                            acc[i][j][4 * q + 1] += v[1];
                            acc[i][j][4 * q + 2] += v[2];
                            acc[i][j][4 * q + 3] += v[3];
                        }
            }
            __syncthreads();
        }
        if (set != 0) return;
    }

    float *dst = p.partial + static_cast<size_t>(SETS > 1 ? chunk / SETS : chunk) * s.c_out * p.S;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int out_col = s0 + wn * 32 * TN + j * 32 + li;
        if (out_col >= p.S) continue;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int oc = oc0 + wm * 32 * TM + i * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                if (oc < s.c_out) dst[static_cast<size_t>(oc) * p.S + out_col] = acc[i][j][r];
            }
    }
}

template <bool VEC>
__global__ __launch_bounds__(256) void conv_grad_weight_kernel(GradWeightArgs p)
{
    __shared__ __attribute__((aligned(16))) float As[2 * 64 * 20];
    __shared__ __attribute__((aligned(16))) float Bs[2 * 64 * 20];
    conv_grad_weight_body<VEC, 1, 1>(p, As, Bs);
}

// Three workgroups per compute unit (3 × 51,200 B of LDS, three wavefronts per SIMD): the occupancy attribute makes
// the compiler fit 170 registers (it does, 160 without spilling) instead of spreading the accumulators over the
// accumulation registers at two wavefronts per SIMD.
template <bool VEC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void conv_grad_weight_big_kernel(GradWeightArgs p)
{
    __shared__ __attribute__((aligned(16))) float As[2 * 128 * 20];
    __shared__ __attribute__((aligned(16))) float Bs[2 * 192 * 20];
    conv_grad_weight_body<VEC, 2, 3>(p, As, Bs);
}

// The same tile with three sets of four wavefronts in one workgroup (one workgroup per compute unit, 153,600 B of LDS).
template <bool VEC>
__global__ __launch_bounds__(768) __attribute__((amdgpu_waves_per_eu(3, 3))) void conv_grad_weight_big3_kernel(GradWeightArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float grad_weight_lds[];
    conv_grad_weight_body<VEC, 2, 3, 3>(p, grad_weight_lds, nullptr);
}

}  // namespace

namespace {
// grad_input as a forward problem: grad_output is the image, input positions are the output pixels.  True when the
// forward kernels can run it (stride 1 and a non-negative adjoint padding); `t` is that problem either way, with
// the original stride/padding when the adjoint gather has to run instead.
bool grad_input_as_forward(const ConvShape &shape, ConvShape &t)
{
    const int adj_pad_h = shape.dil_h * (shape.kh - 1) - shape.pad_h;
    const int adj_pad_w = shape.dil_w * (shape.kw - 1) - shape.pad_w;
    const bool as_forward = shape.stride_h == 1 && shape.stride_w == 1 && adj_pad_h >= 0 && adj_pad_w >= 0;
    t = shape;
    t.c_in = shape.c_out;
    t.h = shape.oh;
    t.w = shape.ow;
    t.c_out = shape.c_in;
    t.oh = shape.h;
    t.ow = shape.w;
    if (as_forward) {
        t.pad_h = adj_pad_h;
        t.pad_w = adj_pad_w;
    }
    return as_forward;
}
}  // namespace

namespace {
// Strided (or over-padded) layers: the adjoint gather kernel tests every (channel, tap) for every input position,
// although only one tap in stride_h·stride_w can contribute, and its output-channel tiles hold 64 or 128 input
// channels — the ViT patch embedding (3 channels, 16×16 at stride 16) took 1.3 s that way.  The reference's own route,
// the product grad_outputᵀ·W followed by col2im, does the forward's flops once: per image an f32 GEMM with the
// transposed-A kernel (grad_output of an image is C_out × OH·OW, i.e. k × m), its result gathered into grad_input.
// Images are processed in groups whose products fit kCol2imWorkspaceBytes.  Chosen when the gather's wasted work
// (stride product × channel-tile padding) exceeds a factor of three; the allocation-free entry point keeps the gather.
constexpr size_t kCol2imWorkspaceBytes = 256u << 20;
bool grad_input_by_col2im(const ConvShape &shape)
{
    const double tile = shape.c_in > 64 ? 128.0 : 64.0;
    const double padded = std::ceil(shape.c_in / tile) * tile / shape.c_in;
    const size_t image_cols = static_cast<size_t>(shape.oh) * shape.ow * shape.c_in * shape.kh * shape.kw * sizeof(float);
    return static_cast<double>(shape.stride_h) * shape.stride_w * padded > 3.0 && image_cols <= kCol2imWorkspaceBytes &&
           image_cols > 0;
}
}  // namespace

int planned_conv_grad_input_kernel(const ConvShape &shape)
{
    ConvShape t;
    if (!grad_input_as_forward(shape, t)) return grad_input_by_col2im(shape) ? ST_HIP_CONV_KERNEL_COL2IM : ST_HIP_CONV_KERNEL_ADJOINT;
    return planned_conv_kernel(t, true, true);
}

hipError_t launch_conv2d_grad_input_f32(const ConvShape &shape, const float *grad_output, const float *weight,
                                        float *grad_input, hipStream_t stream, float *weight_scratch)
{
    if (shape.batch == 0 || shape.c_in == 0 || shape.h == 0 || shape.w == 0) return hipSuccess;
    const size_t weight_count = static_cast<size_t>(shape.c_out) * shape.c_in * shape.kh * shape.kw;
    ConvShape t;
    const bool as_forward = grad_input_as_forward(shape, t);
    hipError_t rc;
    if (!as_forward && weight_scratch == nullptr && grad_input_by_col2im(shape)) {
        const size_t m = static_cast<size_t>(shape.oh) * shape.ow, S = static_cast<size_t>(shape.c_in) * shape.kh * shape.kw;
        const size_t image_cols = m * S;
        const size_t group = std::max<size_t>(1, std::min<size_t>(shape.batch, kCol2imWorkspaceBytes / (image_cols * sizeof(float))));
        void *workspace = nullptr;
        rc = stream_workspace(stream, group * image_cols * sizeof(float), &workspace);
        if (rc != hipSuccess) return rc;
        float *cols = static_cast<float *>(workspace);
        const size_t image_in = static_cast<size_t>(shape.c_in) * shape.h * shape.w;
        for (size_t first = 0; first < static_cast<size_t>(shape.batch); first += group) {
            const size_t images = std::min(group, static_cast<size_t>(shape.batch) - first);
            // cols_i (OH·OW × S) = G_iᵀ · W with G_i = grad_output of image i, C_out × OH·OW (k × m), W = C_out × S: one
            // launch for the group's images (a launch per image cost 5 µs each whatever its size).
            rc = launch_gemm_f32_batched(images, m, S, static_cast<size_t>(shape.c_out), true,
                                         grad_output + first * shape.c_out * m, static_cast<size_t>(shape.c_out) * m, weight, cols,
                                         image_cols, stream);
            if (rc != hipSuccess) return rc;
            const size_t total = images * image_in;
            hipLaunchKernelGGL(conv_col2im_gather_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, stream,
                               shape, static_cast<int>(images), cols, grad_input + first * image_in);
            rc = hipGetLastError();
            if (rc != hipSuccess) return rc;
        }
        return hipSuccess;
    }
    float *adjoint_weight = weight_scratch;  // room for weight_count values, owned by the caller
    // The re-laid weights sit at the front of the stream's scratch buffer; a forward launch that cuts its reduction
    // into slices keeps its partial sums behind them (sized here, so the buffer does not move in between).
    const size_t weight_bytes = (weight_count * sizeof(float) + 255) & ~static_cast<size_t>(255);
    if (adjoint_weight == nullptr) {
        void *workspace = nullptr;
        const size_t behind = as_forward ? conv2d_scratch_bytes(t, true, (reinterpret_cast<uintptr_t>(grad_input) & 15u) == 0) : 0;
        rc = stream_workspace(stream, weight_bytes + behind, &workspace);
        if (rc != hipSuccess) return rc;
        adjoint_weight = static_cast<float *>(workspace);
    }
    hipLaunchKernelGGL(conv_weight_to_adjoint_kernel, dim3(static_cast<unsigned>((weight_count + 255) / 256)), dim3(256), 0,
                       stream, shape.c_out, shape.c_in, shape.kh, shape.kw, as_forward ? 1 : 0, weight, adjoint_weight);
    rc = hipGetLastError();
    if (rc != hipSuccess) return rc;
    if (as_forward)
        return launch_conv2d_f32(t, ST_HIP_ACT_NONE, grad_output, adjoint_weight, nullptr, grad_input, stream,
                                 weight_scratch ? kConvScratchNone : kConvScratchStream, weight_bytes);
    return launch_conv2d_adjoint_f32(t, grad_output, adjoint_weight, grad_input, stream);
}

hipError_t launch_conv2d_grad_bias_f32(const ConvShape &shape, const float *grad_output, float scale, float *grad_bias,
                                       hipStream_t stream)
{
    if (shape.c_out == 0) return hipSuccess;
    const size_t planes = static_cast<size_t>(shape.batch) * shape.c_out;
    const int spatial = shape.oh * shape.ow;
    void *workspace = nullptr;
    hipError_t rc = stream_workspace(stream, (planes ? planes : 1) * sizeof(float), &workspace);
    if (rc != hipSuccess) return rc;
    float *partial = static_cast<float *>(workspace);
    if (planes > 0) {
        hipLaunchKernelGGL(conv_grad_bias_partial_kernel, dim3(static_cast<unsigned>((planes + 3) / 4)), dim3(256), 0, stream,
                           static_cast<int>(planes), spatial, grad_output, partial);
        rc = hipGetLastError();
        if (rc != hipSuccess) return rc;
    }
    hipLaunchKernelGGL(conv_reduce_chunks_kernel, dim3(static_cast<unsigned>((shape.c_out + 15) / 16)), dim3(256), 0, stream,
                       shape.batch, static_cast<size_t>(shape.c_out), partial, scale, grad_bias);
    return hipGetLastError();
}

hipError_t launch_conv2d_grad_weight_f32(const ConvShape &shape, const float *input, const float *grad_output, float scale,
                                         float *grad_weight, hipStream_t stream)
{
    const int S = shape.c_in * shape.kh * shape.kw;
    const size_t count = static_cast<size_t>(shape.c_out) * S;
    if (count == 0) return hipSuccess;
    // One image of the input and of grad_output is addressed through 32-bit byte offsets.
    if (static_cast<size_t>(shape.c_in) * shape.h * shape.w * 4 >= (1ull << 31) ||
        static_cast<size_t>(shape.c_out) * shape.oh * shape.ow * 4 >= (1ull << 31))
        return hipErrorInvalidValue;
    GradWeightArgs args;
    args.input = input;
    args.grad_output = grad_output;
    args.s = shape;
    args.S = S;
    args.spatial = shape.oh * shape.ow;
    // 128 × 192 tiles when they waste little (every output channel and column a tile covers beyond the matrix is
    // arithmetic thrown away), 64 × 64 tiles otherwise.
    const long long big_cover = static_cast<long long>((shape.c_out + 127) / 128 * 128) * ((S + 191) / 192 * 192);
    const bool big = big_cover * 10 <= static_cast<long long>(count) * 12;
    const int bm = big ? 128 : 64, bn = big ? 192 : 64;
    args.tiles_s = (S + bn - 1) / bn;
    const int tiles = args.tiles_s * ((shape.c_out + bm - 1) / bm);
    // The reduction (all 16-pixel steps of all images, numbered image by image) is cut into chunks so that the
    // launch is about one round of resident workgroups (8 small or 3 big tiles per compute unit).
    const long long steps_per_image = (args.spatial + 15) / 16;
    const long long total_steps = steps_per_image * shape.batch;
    const long long slots = big ? 768 : 2048;
    long long chunks = slots / tiles;  // rounded down: one workgroup too many would run as a round of its own
    if (chunks > total_steps) chunks = total_steps;
    if (chunks < 1) chunks = 1;
    args.steps_per_chunk = static_cast<int>(total_steps > 0 ? (total_steps + chunks - 1) / chunks : 1);
    chunks = total_steps > 0 ? (total_steps + args.steps_per_chunk - 1) / args.steps_per_chunk : 1;
    // Big tiles with at least three runs of steps per tile: three runs share a workgroup (and a partial tile).
    const bool three_sets = big && chunks >= 3;
    if (three_sets) chunks = (chunks + 2) / 3;
    void *workspace = nullptr;
    hipError_t rc = stream_workspace(stream, static_cast<size_t>(chunks) * count * sizeof(float), &workspace);
    if (rc != hipSuccess) return rc;
    args.partial = static_cast<float *>(workspace);
    const bool vec = args.spatial % 4 == 0 && (reinterpret_cast<uintptr_t>(grad_output) & 15u) == 0;
    const size_t workgroups = static_cast<size_t>(tiles) * static_cast<size_t>(chunks);
    if (workgroups > 0x7ffffff0u) return hipErrorInvalidConfiguration;
    args.workgroups = static_cast<int>(workgroups);
    const dim3 grid(static_cast<unsigned>((workgroups + 7) / 8 * 8));
    if (three_sets) {
        constexpr size_t lds_bytes = 3 * (2 * 128 * 20 + 2 * 192 * 20) * sizeof(float);
        auto kernel = vec ? conv_grad_weight_big3_kernel<true> : conv_grad_weight_big3_kernel<false>;
        rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                 static_cast<int>(lds_bytes));
        if (rc != hipSuccess) return rc;
        hipLaunchKernelGGL(kernel, grid, dim3(768), lds_bytes, stream, args);
    } else if (big && vec)
        hipLaunchKernelGGL(conv_grad_weight_big_kernel<true>, grid, dim3(256), 0, stream, args);
    else if (big)
        hipLaunchKernelGGL(conv_grad_weight_big_kernel<false>, grid, dim3(256), 0, stream, args);
    else if (vec)
        hipLaunchKernelGGL(conv_grad_weight_kernel<true>, grid, dim3(256), 0, stream, args);
    else
        hipLaunchKernelGGL(conv_grad_weight_kernel<false>, grid, dim3(256), 0, stream, args);
    rc = hipGetLastError();
    if (rc != hipSuccess) return rc;
    if (count % 4 == 0 && ((reinterpret_cast<uintptr_t>(args.partial) | reinterpret_cast<uintptr_t>(grad_weight)) & 15u) == 0)
        hipLaunchKernelGGL(conv_reduce_chunks_vec_kernel, dim3(static_cast<unsigned>((count / 4 + 31) / 32)), dim3(256), 0, stream,
                           static_cast<int>(chunks), count / 4, reinterpret_cast<const float4 *>(args.partial), scale,
                           reinterpret_cast<float4 *>(grad_weight));
    else
        hipLaunchKernelGGL(conv_reduce_chunks_kernel, dim3(static_cast<unsigned>((count + 15) / 16)), dim3(256), 0, stream,
                           static_cast<int>(chunks), count, args.partial, scale, grad_weight);
    return hipGetLastError();
}

}  // namespace sthip
