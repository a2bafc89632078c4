// Scaled-dot-product attention with online softmax on bf16 operands (gfx950), used by the decoder stack.
//
// Same mathematics as crates/st-tensor/src/pure.rs:11845-11919 (per query: softmax over keys of
// q·k·scale, weighted sum of value rows, optional causal key range 0..=query), with the two matrix
// products taking bf16 inputs and accumulating in f32 on v_mfma_f32_32x32x16_bf16; the softmax itself
// (maximum, exponentials, sums, final division) stays in f32.  Heads are read in place from row-major
// (batch·sequence, width) matrices — context (b, h) owns columns h·D .. h·D+D-1 of rows b·S .. b·S+S-1,
// the layout crates/st-vision/src/models/vit.rs:151-180 indexes — so a fused [Q | K | V] projection output is
// consumed without a split pass and the result lands directly in the (tokens, heads·D) matrix the
// output projection reads.
//
// The kernel computes the transposed problem, Sᵀ = K·Qᵀ and Oᵀ += Vᵀ·Pᵀ: every lane then owns one query
// column, so the running maximum and sum are per-lane scalars and the probabilities leave the first
// product's accumulators already in the register layout the second product's B operand needs (no
// shuffle, no LDS round trip).  The accumulator of a 32x32 tile hands lane half h the keys
// {8a + 4h + c}; the second product wants eight k-indices per lane, so its Vᵀ operand takes keys
// 16j + 4h + {0..3} and 16j + 8 + 4h + {0..3}: V is staged exactly as it is stored (rows = keys, one 128-bit
// LDS write per 128-bit load) and those two groups of four keys are fetched with the transposing LDS read
// (ds_read_b64_tr_b16).  (Transposing while staging — eight 16-bit scattered writes per load — spent two thirds
// of the LDS cycles on bank conflicts.)
#include "device_math.h"
#include "kernels.h"

#include <type_traits>

namespace sthip {

namespace {

struct AttnBf16Args {
    const uint16_t *q;
    const uint16_t *k;
    const uint16_t *v;
    uint16_t *out;
    int batch, heads, S;
    int ld_in, ld_out;  // row strides in elements
    int q_tiles;
    int swizzle;
    float scale;
};

constexpr int kBQ16 = 128;
constexpr float kLog2e16 = 1.4426950408889634f;

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef s16x4 __attribute__((address_space(3))) *lds_s16x4_ptr;

__device__ __forceinline__ unsigned pack_bf16x2(float lo, float hi)
{
    const bf16x2_t v = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};  // round-to-nearest-even
    return __builtin_bit_cast(unsigned, v);
}

template <int D, bool CAUSAL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D == 64 ? (CAUSAL ? 4 : 3) : 2, D == 64 ? (CAUSAL ? 4 : 3) : 2))) void attention_bf16_kernel(AttnBf16Args p)
{
    constexpr int BKV = 64;
    constexpr int KS = D + 8;      // K row stride (elements): 16 bytes of padding keep 128-bit reads conflict-free
    constexpr int VS = D + 8;      // V row stride: V is staged as it is stored (rows = keys) and read transposed
    constexpr int K_ELEMS = BKV * KS, V_ELEMS = BKV * VS;
    constexpr int KC = D / 16;     // k-blocks of K·Qᵀ
    constexpr int DT = D / 32;     // 32-row tiles of Oᵀ
    constexpr int LOADS = BKV * D / 8 / 256;
    extern __shared__ __attribute__((aligned(16))) uint16_t attn16_lds[];
    uint16_t *Ks = attn16_lds;                // [2][K_ELEMS]
    uint16_t *Vs = attn16_lds + 2 * K_ELEMS;  // [2][V_ELEMS]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 31, lh = lane >> 5;
    const int S = p.S;
    const int contexts = p.batch * p.heads;

    // Workgroup -> (context, query tile): each XCD (workgroup id mod 8) keeps whole contexts so their K/V
    // stay in its L2; causal tiles run longest-first across all contexts of the XCD.
    int ctx, q_tile;
    if (p.swizzle) {
        const int per_xcd = contexts >> 3;
        const int xcd = blockIdx.x & 7, i = blockIdx.x >> 3;
        if (CAUSAL) {
            q_tile = p.q_tiles - 1 - i / per_xcd;
            ctx = xcd * per_xcd + i % per_xcd;
        } else {
            ctx = xcd * per_xcd + i / p.q_tiles;
            q_tile = i % p.q_tiles;
        }
    } else {
        if (CAUSAL) {
            q_tile = p.q_tiles - 1 - blockIdx.x / contexts;
            ctx = blockIdx.x % contexts;
        } else {
            ctx = blockIdx.x / p.q_tiles;
            q_tile = blockIdx.x % p.q_tiles;
        }
    }
    const int q0 = q_tile * kBQ16;
    const int wq0 = q0 + wave * 32;
    const int my_q = wq0 + li;
    const int b = ctx / p.heads, h = ctx % p.heads;
    const size_t in_base = static_cast<size_t>(b) * S * p.ld_in + static_cast<size_t>(h) * D;
    // One descriptor per operand covering exactly this context's rows: rows past the end read as zero.
    const unsigned in_bytes = (static_cast<unsigned>(S - 1) * static_cast<unsigned>(p.ld_in) + D) * 2u;
    const __amdgpu_buffer_rsrc_t rsrc_q =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(p.q + in_base), 0, static_cast<int>(in_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_k =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(p.k + in_base), 0, static_cast<int>(in_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_v =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(p.v + in_base), 0, static_cast<int>(in_bytes), 0x00020000);

    auto fetch8 = [&](const __amdgpu_buffer_rsrc_t &rsrc, int row, int d) -> u32x4_t {
        return __builtin_amdgcn_raw_buffer_load_b128(
            rsrc, (static_cast<unsigned>(row) * static_cast<unsigned>(p.ld_in) + d) * 2u, 0, 0);
    };

    // Qᵀ fragments (B operand): lane (li, lh) holds Q[my_q][16c + 8·lh .. +7].
    bf16x8 qf[KC];
#pragma unroll
    for (int c = 0; c < KC; ++c) {
        // A negative scale is moved into Q (sign bits flipped) so that the scale applied below is never negative
        // and the running maximum can be taken over the raw dot products.
        u32x4_t raw = fetch8(rsrc_q, my_q, c * 16 + lh * 8);
        if (p.scale < 0.0f) raw ^= 0x80008000u;
        qf[c] = __builtin_bit_cast(bf16x8, raw);
    }

    f32x16 oacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
        oacc[t] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float run_max = -INFINITY;
    float run_sum = 0.0f;

    const int key_end = CAUSAL ? min(S, q0 + kBQ16) : S;
    const int stages = (key_end + BKV - 1) / BKV;

    u32x4_t rk[LOADS], rv[LOADS];
    auto load_global = [&](int key0) {
#pragma unroll
        for (int r = 0; r < LOADS; ++r) {
            const int f = tid + 256 * r;
            const int row = f / (D / 8), c8 = (f % (D / 8)) * 8;
            rk[r] = fetch8(rsrc_k, key0 + row, c8);
            rv[r] = fetch8(rsrc_v, key0 + row, c8);
        }
    };
    auto store_lds = [&](int stage) {
        uint16_t *ks = Ks + stage * K_ELEMS;
        uint16_t *vs = Vs + stage * V_ELEMS;
#pragma unroll
        for (int r = 0; r < LOADS; ++r) {
            const int f = tid + 256 * r;
            const int row = f / (D / 8), c8 = (f % (D / 8)) * 8;
            *reinterpret_cast<u32x4_t *>(&ks[row * KS + c8]) = rk[r];
            *reinterpret_cast<u32x4_t *>(&vs[row * VS + c8]) = rv[r];
        }
    };
    // Transpose-read lane roles (ds_read_b64_tr_b16): within each 16-lane group lane i16 supplies the address of
    // row i16/4 and 4-column chunk i16%4 of a 4×16 block and receives column i16 of it (4 rows).
    const int i16 = lane & 15, c16 = (lane >> 4) & 1;
    const int v_read = (lh * 4 + (i16 >> 2)) * VS + c16 * 16 + (i16 & 3) * 4;

    // (Floored at a tiny positive value so that a zero scale still turns masked (-inf) logits into weight 0
    // instead of -inf·0.)
    const float scale_log2e = fmaxf(fabsf(p.scale) * kLog2e16, 1e-30f);
    const float lag = 8.0f / scale_log2e;  // 2^8 in units of the raw dot product
    // NT = number of 32-key tiles of this stage this wavefront works on (1 or 2).
    // MAY_MASK = false: the caller knows that every key of the stage exists and (causal) lies at or below every query
    // row of this wavefront.
    auto compute = [&](auto nt_tag, auto may_mask_tag, int stage, int key0) {
        constexpr int NT = decltype(nt_tag)::value;
        constexpr bool MAY_MASK = decltype(may_mask_tag)::value;
        const uint16_t *ks = Ks + stage * K_ELEMS;
        const uint16_t *vs = Vs + stage * V_ELEMS;
        f32x16 sacc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t)
            sacc[t] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            bf16x8 kf[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t)
                kf[t] = *reinterpret_cast<const bf16x8 *>(&ks[(t * 32 + li) * KS + c * 16 + lh * 8]);
#pragma unroll
            for (int t = 0; t < NT; ++t) sacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[t], qf[c], sacc[t], 0, 0, 0);
        }
        // The running maximum is kept in units of the raw dot product (scale >= 0 here), so the scale costs no pass
        // of its own: p = exp2(dot·scale·log2e − max·scale·log2e) is one fused multiply-add and one exp2.  Masking
        // only where a tile crosses the sequence end or the diagonal.
        const bool need_mask = MAY_MASK && ((key0 + NT * 32 > S) || (CAUSAL && key0 + NT * 32 - 1 > wq0));
        float tile_max = -INFINITY;
        // the last key this lane's query sees: one comparison per score (a causal row never looks past the sequence end)
        const int last_key = CAUSAL ? min(my_q, S - 1) : S - 1;
        if (need_mask) {
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = key0 + t * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                    float v = sacc[t][r];
                    if (key > last_key) v = -INFINITY;
                    sacc[t][r] = v;
                    tile_max = fmaxf(tile_max, v);
                }
        } else {
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) tile_max = fmaxf(tile_max, sacc[t][r]);
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32));
        // The reference maximum in the exponent is allowed to lag the true running maximum by up to 2^8 (weights then
        // reach 256 instead of 1, harmless in f32 and bf16); the accumulators are rescaled only when some query's
        // maximum has moved by more than that, which after the first key tiles is rare.
        if (__any(tile_max > run_max + lag)) {  // wavefront-uniform
            const float new_max = fmaxf(run_max, tile_max);
            const float new_safe = new_max == -INFINITY ? 0.0f : new_max;
            const float alpha = __builtin_amdgcn_exp2f((run_max - new_safe) * scale_log2e);  // run_max = -inf -> 0
            run_sum *= alpha;
#pragma unroll
            for (int t = 0; t < DT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[t][r] *= alpha;
            run_max = new_max;
        }
        const float safe_max = run_max == -INFINITY ? 0.0f : run_max;
        const float shift = -safe_max * scale_log2e;
        float tile_sum = 0.0f;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float pr = __builtin_amdgcn_exp2f(fmaf(sacc[t][r], scale_log2e, shift));
                sacc[t][r] = pr;
                tile_sum += pr;
            }
        run_sum += tile_sum;
        // Oᵀ += Vᵀ·Pᵀ, 16 keys per MFMA: accumulator registers 8j .. 8j+7 are this lane's k-indices 8·lh .. 8·lh+7,
        // which are keys 16j + 4·lh + {0..3} and 16j + 8 + 4·lh + {0..3}; the Vᵀ operand is gathered to match with
        // two transposing reads (4 keys × 16 head-dim columns per 16-lane group each).
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                u32x4_t packed;
#pragma unroll
                for (int e = 0; e < 4; ++e) packed[e] = pack_bf16x2(sacc[t][8 * j + 2 * e], sacc[t][8 * j + 2 * e + 1]);
                const bf16x8 pf = __builtin_bit_cast(bf16x8, packed);
                bf16x8 vf[DT];
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const uint16_t *src = &vs[(t * 32 + j * 16) * VS + v_read + dt * 32];
                    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(src));
                    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(src + 8 * VS));
                    vf[dt] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                }
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[dt], pf, oacc[dt], 0, 0, 0);
            }
    };

    if (stages > 0) {
        load_global(0);
        store_lds(0);
    }
    __syncthreads();
    // The stages whose 64 keys all exist and need no causal mask for any row of this wavefront come first, in a loop
    // with one path through it: a loop body that branches between the one-tile, the two-tile and the skipped form has
    // the output accumulators merged after the branch, and the compiler then copies all of their registers twice per
    // stage — behind the stage's last matrix instructions, whose latency the copies wait out.  The stages on and beyond
    // the diagonal (two per workgroup at most) and a ragged last stage take the branching loop after it.
    const int limit = CAUSAL ? min(S, wq0 + 32) : S;
    const int plain_stages = min(stages, (CAUSAL ? min(S, wq0 + 1) : S) / BKV);
    int t = 0;
    for (; t < plain_stages; ++t) {
        const bool more = t + 1 < stages;
        if (more) load_global((t + 1) * BKV);
        compute(std::integral_constant<int, 2>{}, std::false_type{}, t & 1, t * BKV);
        if (more) store_lds((t + 1) & 1);
        __syncthreads();
    }
    for (; t < stages; ++t) {
        const bool more = t + 1 < stages;
        if (more) load_global((t + 1) * BKV);
        const int key0 = t * BKV;
        // Tiles entirely past the sequence end or (causal) entirely above this wavefront's rows are skipped.
        if (key0 + 32 < limit) compute(std::integral_constant<int, 2>{}, std::true_type{}, t & 1, key0);
        else if (key0 < limit) compute(std::integral_constant<int, 1>{}, std::true_type{}, t & 1, key0);
        if (more) store_lds((t + 1) & 1);
        __syncthreads();
    }

    const float total = run_sum + __shfl_xor(run_sum, 32);
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    if (my_q < S) {
        uint16_t *orow = p.out + (static_cast<size_t>(b) * S + my_q) * p.ld_out + static_cast<size_t>(h) * D;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = t * 32 + g * 8 + lh * 4;
                u32x2_t packed;
                packed[0] = pack_bf16x2(oacc[t][g * 4 + 0] * inv, oacc[t][g * 4 + 1] * inv);
                packed[1] = pack_bf16x2(oacc[t][g * 4 + 2] * inv, oacc[t][g * 4 + 3] * inv);
                *reinterpret_cast<u32x2_t *>(orow + d) = packed;
            }
    }
}

// -------------------------------------------------------------------------------------------------
// head_dim 64: the same arithmetic in the same order as the kernel above (bit for bit the same output), with K and V
// going straight from global memory into LDS (buffer_load ... lds: no staging registers, no LDS write instructions).
// A stage is 64 rows of 128 bytes with the 16-byte chunks XOR-swizzled: chunk q of K row r sits at q ^ ((r >> 1) & 7):
// a 128-bit fragment read serves sixteen lanes — sixteen consecutive rows — per cycle from 64 banks, a row is 32 banks
// long, so rows 2i and 2i+1 lie on different bank halves and need the same shift, and the eight pairs eight different
// ones (with q ^ (r & 7), rows r and r + 8 met on the same banks: 32 % of the LDS cycles were bank conflicts).  Chunk q
// of V row r sits at q ^ 4·((r >> 1) & 1) (the four rows × 64 bytes one pass of a transposing read touches then cover
// all banks).
// -------------------------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void *lds_void_ptr16;

template <bool CAUSAL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void attention_bf16_d64_kernel(AttnBf16Args p)
{
    constexpr int D = 64, BKV = 64, KC = 4, DT = 2;
    constexpr int STAGE = BKV * D * 2;  // 8 KB: 64 rows of 128 bytes
    extern __shared__ __attribute__((aligned(16))) unsigned char lds16[];  // [K0][K1][V0][V1]
    unsigned char *const k_lds = lds16;
    unsigned char *const v_lds = lds16 + 2 * STAGE;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int S = p.S;
    const int contexts = p.batch * p.heads;

    // Workgroup -> (context, query tile) as in the kernel above.
    int ctx, q_tile;
    if (p.swizzle) {
        const int per_xcd = contexts >> 3;
        const int xcd = blockIdx.x & 7, i = blockIdx.x >> 3;
        if (CAUSAL) {
            q_tile = p.q_tiles - 1 - i / per_xcd;
            ctx = xcd * per_xcd + i % per_xcd;
        } else {
            ctx = xcd * per_xcd + i / p.q_tiles;
            q_tile = i % p.q_tiles;
        }
    } else {
        if (CAUSAL) {
            q_tile = p.q_tiles - 1 - blockIdx.x / contexts;
            ctx = blockIdx.x % contexts;
        } else {
            ctx = blockIdx.x / p.q_tiles;
            q_tile = blockIdx.x % p.q_tiles;
        }
    }
    const int q0 = q_tile * kBQ16;
    const int wq0 = q0 + wave * 32;
    const int my_q = wq0 + li;
    const int b = ctx / p.heads, h = ctx % p.heads;
    const size_t in_base = static_cast<size_t>(b) * S * p.ld_in + static_cast<size_t>(h) * D;
    const unsigned in_bytes = (static_cast<unsigned>(S - 1) * static_cast<unsigned>(p.ld_in) + D) * 2u;
    const __amdgpu_buffer_rsrc_t rsrc_q =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(p.q + in_base), 0, static_cast<int>(in_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_k =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(p.k + in_base), 0, static_cast<int>(in_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_v =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(p.v + in_base), 0, static_cast<int>(in_bytes), 0x00020000);

    // Direct loads: instruction i of wavefront w fills rows (i*4 + w)*8 .. +7 of a stage, eight lanes per row; the lane
    // at chunk position c of row r fetches the chunk that the swizzle stores there.  (The stage's offset is added
    // into the vector offset: the descriptor's range check, which returns zeros for rows past the end of the context,
    // does not see the scalar offset.)
    const unsigned row_bytes = static_cast<unsigned>(p.ld_in) * 2u;
    unsigned k_voff[2], v_voff[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = (i * 4 + wave) * 8 + (lane >> 3);
        const int c = lane & 7;
        k_voff[i] = static_cast<unsigned>(r) * row_bytes + static_cast<unsigned>((c ^ ((r >> 1) & 7)) * 16);
        v_voff[i] = static_cast<unsigned>(r) * row_bytes + static_cast<unsigned>((c ^ (((r >> 1) & 1) * 4)) * 16);
    }
    auto load_stage = [&](int stage) {
        const unsigned first = static_cast<unsigned>(stage) * BKV * row_bytes;
#pragma unroll
        for (int i = 0; i < 2; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_k, (lds_void_ptr16)(k_lds + (stage & 1) * STAGE + (i * 4 + wave) * 1024), 16,
                                                     k_voff[i] + first, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 2; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_v, (lds_void_ptr16)(v_lds + (stage & 1) * STAGE + (i * 4 + wave) * 1024), 16,
                                                     v_voff[i] + first, 0, 0, 0);
    };

    // Fragment addresses within a stage.  K: lane (li, lh) reads row t*32 + li, chunk 2c + lh.  V (transposing read):
    // within each 16-lane group lane i16 supplies row i16/4 and 8-byte piece i16%4 of a 4-row × 16-column block.
    unsigned k_read[KC];
#pragma unroll
    for (int c = 0; c < KC; ++c) k_read[c] = static_cast<unsigned>(li * 128 + (((2 * c + lh) ^ ((li >> 1) & 7)) * 16));
    const int i16 = lane & 15, c16 = (lane >> 4) & 1;
    unsigned v_read[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const int row = lh * 4 + (i16 >> 2);
        const int chunk = dt * 4 + c16 * 2 + ((i16 & 3) >> 1);
        v_read[dt] = static_cast<unsigned>(reinterpret_cast<uintptr_t>((lds_void_ptr16)v_lds)) +
                     static_cast<unsigned>(row * 128 + ((chunk ^ (((i16 >> 3) & 1) * 4)) * 16) + (i16 & 1) * 8);
    }
    // The four transposing reads of one 16-key group of a V stage (two head-dim tiles × two groups of four keys),
    // followed by the wait for them.  Written as one assembly block: the compiler does not know which memory this
    // read touches and would otherwise wait for every direct-to-LDS load in flight — the prefetch of the next stage
    // — before the first of them.
    auto read_v_group = [&](auto group_tag, unsigned a0, unsigned a1, bf16x8 (&out)[DT]) {
        constexpr int base = decltype(group_tag)::value * 2048;  // 16 rows of 128 bytes
        u32x2_t r0, r1, r2, r3;
        asm volatile("ds_read_b64_tr_b16 %0, %4 offset:%6\n"
                     "ds_read_b64_tr_b16 %1, %4 offset:%7\n"
                     "ds_read_b64_tr_b16 %2, %5 offset:%6\n"
                     "ds_read_b64_tr_b16 %3, %5 offset:%7\n"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
                     : "v"(a0), "v"(a1), "n"(base), "n"(base + 1024)
                     : "memory");
        auto join = [](u32x2_t lo, u32x2_t hi) {
            const u32x4_t v = {lo[0], lo[1], hi[0], hi[1]};
            return __builtin_bit_cast(bf16x8, v);
        };
        out[0] = join(r0, r1);  // head-dim tile 0
        out[1] = join(r2, r3);  // head-dim tile 1
    };

    bf16x8 qf[KC];
#pragma unroll
    for (int c = 0; c < KC; ++c) {
        u32x4_t raw = __builtin_amdgcn_raw_buffer_load_b128(
            rsrc_q, (static_cast<unsigned>(my_q) * static_cast<unsigned>(p.ld_in) + c * 16 + lh * 8) * 2u, 0, 0);
        if (p.scale < 0.0f) raw ^= 0x80008000u;
        qf[c] = __builtin_bit_cast(bf16x8, raw);
    }

    f32x16 oacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
        oacc[t] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float run_max = -INFINITY;
    float run_sum = 0.0f;

    const int key_end = CAUSAL ? min(S, q0 + kBQ16) : S;
    const int stages = (key_end + BKV - 1) / BKV;
    const float scale_log2e = fmaxf(fabsf(p.scale) * kLog2e16, 1e-30f);
    const float lag = 8.0f / scale_log2e;

    // NT = number of 32-key tiles of this stage this wavefront works on (1 or 2).
    // MAY_MASK = false: the caller knows that every key of the stage exists and (causal) lies at or below every query
    // row of this wavefront.
    auto compute = [&](auto nt_tag, auto may_mask_tag, int stage, int key0) {
        constexpr int NT = decltype(nt_tag)::value;
        constexpr bool MAY_MASK = decltype(may_mask_tag)::value;
        const unsigned char *ks = k_lds + stage * STAGE;
        f32x16 sacc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t)
            sacc[t] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            bf16x8 kf[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) kf[t] = *reinterpret_cast<const bf16x8 *>(ks + t * 4096 + k_read[c]);
#pragma unroll
            for (int t = 0; t < NT; ++t) sacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[t], qf[c], sacc[t], 0, 0, 0);
        }
        const bool need_mask = MAY_MASK && ((key0 + NT * 32 > S) || (CAUSAL && key0 + NT * 32 - 1 > wq0));
        float tile_max = -INFINITY;
        // the last key this lane's query sees: one comparison per score (a causal row never looks past the sequence end)
        const int last_key = CAUSAL ? min(my_q, S - 1) : S - 1;
        if (need_mask) {
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = key0 + t * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                    float v = sacc[t][r];
                    if (key > last_key) v = -INFINITY;
                    sacc[t][r] = v;
                    tile_max = fmaxf(tile_max, v);
                }
        } else {
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) tile_max = fmaxf(tile_max, sacc[t][r]);
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32));
        if (__any(tile_max > run_max + lag)) {  // wavefront-uniform
            const float new_max = fmaxf(run_max, tile_max);
            const float new_safe = new_max == -INFINITY ? 0.0f : new_max;
            const float alpha = __builtin_amdgcn_exp2f((run_max - new_safe) * scale_log2e);  // run_max = -inf -> 0
            run_sum *= alpha;
#pragma unroll
            for (int t = 0; t < DT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[t][r] *= alpha;
            run_max = new_max;
        }
        const float safe_max = run_max == -INFINITY ? 0.0f : run_max;
        const float shift = -safe_max * scale_log2e;
        float tile_sum = 0.0f;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float pr = __builtin_amdgcn_exp2f(fmaf(sacc[t][r], scale_log2e, shift));
                sacc[t][r] = pr;
                tile_sum += pr;
            }
        run_sum += tile_sum;
        const unsigned v_stage0 = v_read[0] + stage * STAGE, v_stage1 = v_read[1] + stage * STAGE;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                u32x4_t packed;
#pragma unroll
                for (int e = 0; e < 4; ++e) packed[e] = pack_bf16x2(sacc[t][8 * j + 2 * e], sacc[t][8 * j + 2 * e + 1]);
                const bf16x8 pf = __builtin_bit_cast(bf16x8, packed);
                bf16x8 vf[DT];
                if (t == 0 && j == 0) read_v_group(std::integral_constant<int, 0>{}, v_stage0, v_stage1, vf);
                else if (t == 0) read_v_group(std::integral_constant<int, 1>{}, v_stage0, v_stage1, vf);
                else if (j == 0) read_v_group(std::integral_constant<int, 2>{}, v_stage0, v_stage1, vf);
                else read_v_group(std::integral_constant<int, 3>{}, v_stage0, v_stage1, vf);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[dt], pf, oacc[dt], 0, 0, 0);
            }
    };

    load_stage(0);
    __builtin_amdgcn_s_waitcnt(0x0070 | (15 << 8));  // vmcnt(0): Q and stage 0 have landed
    __syncthreads();
    // The stages whose 64 keys all exist and need no causal mask for any row of this wavefront come first, in a loop
    // with one path through it: a loop body that branches between the one-tile, the two-tile and the skipped form has
    // the output accumulators merged after the branch, and the compiler then copies all 32 of their registers twice
    // per stage — behind the stage's last matrix instructions, whose latency the copies wait out.  The stages on and
    // beyond the diagonal (two per workgroup at most) and a ragged last stage take the branching loop after it.
    const int limit = CAUSAL ? min(S, wq0 + 32) : S;
    const int plain_stages = min(stages, (CAUSAL ? min(S, wq0 + 1) : S) / BKV);
    int t = 0;
    for (; t < plain_stages; ++t) {
        if (t + 1 < stages) load_stage(t + 1);
        compute(std::integral_constant<int, 2>{}, std::false_type{}, t & 1, t * BKV);
        __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0), lgkmcnt(0): the next stage has landed, this one has been read
        __syncthreads();
    }
    for (; t < stages; ++t) {
        const bool more = t + 1 < stages;
        if (more) load_stage(t + 1);
        const int key0 = t * BKV;
        if (key0 + 32 < limit) compute(std::integral_constant<int, 2>{}, std::true_type{}, t & 1, key0);
        else if (key0 < limit) compute(std::integral_constant<int, 1>{}, std::true_type{}, t & 1, key0);
        __builtin_amdgcn_s_waitcnt(0x0070);
        __syncthreads();
    }

    const float total = run_sum + __shfl_xor(run_sum, 32);
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    if (my_q < S) {
        uint16_t *orow = p.out + (static_cast<size_t>(b) * S + my_q) * p.ld_out + static_cast<size_t>(h) * D;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = t * 32 + g * 8 + lh * 4;
                u32x2_t packed;
                packed[0] = pack_bf16x2(oacc[t][g * 4 + 0] * inv, oacc[t][g * 4 + 1] * inv);
                packed[1] = pack_bf16x2(oacc[t][g * 4 + 2] * inv, oacc[t][g * 4 + 3] * inv);
                *reinterpret_cast<u32x2_t *>(orow + d) = packed;
            }
    }
}

template <bool CAUSAL>
hipError_t launch_d64(const AttnBf16Args &args, hipStream_t stream)
{
    constexpr size_t lds_bytes = 4 * 64 * 64 * sizeof(uint16_t);  // two K stages + two V stages
    auto kernel = attention_bf16_d64_kernel<CAUSAL>;
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    const size_t blocks = static_cast<size_t>(args.batch) * args.heads * args.q_tiles;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), lds_bytes, stream, args);
    return hipGetLastError();
}

template <int D, bool CAUSAL>
hipError_t launch_variant(const AttnBf16Args &args, hipStream_t stream)
{
    constexpr size_t lds_bytes = 2 * (static_cast<size_t>(64) * (D + 8) + static_cast<size_t>(64) * (D + 8)) * sizeof(uint16_t);
    auto kernel = attention_bf16_kernel<D, CAUSAL>;
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    const size_t blocks = static_cast<size_t>(args.batch) * args.heads * args.q_tiles;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), lds_bytes, stream, args);
    return hipGetLastError();
}

}  // namespace

bool attention_bf16_supported(size_t sequence, size_t head_dim, size_t ld_in, size_t ld_out, const void *q,
                              const void *k, const void *v, const void *out)
{
    auto aligned = [](const void *ptr, uintptr_t a) { return (reinterpret_cast<uintptr_t>(ptr) & (a - 1)) == 0; };
    if (head_dim != 64 && head_dim != 128) return false;
    if (ld_in % 8 != 0 || ld_out % 4 != 0) return false;
    if (!aligned(q, 16) || !aligned(k, 16) || !aligned(v, 16) || !aligned(out, 8)) return false;
    // one context is addressed through a 32-bit byte offset
    return sequence == 0 || ((sequence - 1) * ld_in + head_dim) * 2 < (1ull << 31);
}

hipError_t launch_attention_bf16(size_t batch, size_t heads, size_t sequence, size_t head_dim, float scale, bool causal,
                                 const uint16_t *q, const uint16_t *k, const uint16_t *v, size_t ld_in, uint16_t *out,
                                 size_t ld_out, hipStream_t stream)
{
    if (batch == 0 || heads == 0 || sequence == 0) return hipSuccess;
    if (!attention_bf16_supported(sequence, head_dim, ld_in, ld_out, q, k, v, out)) return hipErrorInvalidValue;
    AttnBf16Args args;
    args.q = q;
    args.k = k;
    args.v = v;
    args.out = out;
    args.batch = static_cast<int>(batch);
    args.heads = static_cast<int>(heads);
    args.S = static_cast<int>(sequence);
    args.ld_in = static_cast<int>(ld_in);
    args.ld_out = static_cast<int>(ld_out);
    args.q_tiles = static_cast<int>((sequence + kBQ16 - 1) / kBQ16);
    const size_t contexts = batch * heads;
    if (contexts * static_cast<size_t>(args.q_tiles) > 0x7fffffffu) return hipErrorInvalidConfiguration;
    args.swizzle = (contexts % 8 == 0) ? 1 : 0;
    args.scale = scale;
    if (head_dim == 64) return causal ? launch_d64<true>(args, stream) : launch_d64<false>(args, stream);
    return causal ? launch_variant<128, true>(args, stream) : launch_variant<128, false>(args, stream);
}

}  // namespace sthip
