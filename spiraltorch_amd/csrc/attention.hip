// Scaled-dot-product attention with online softmax on the f32 matrix cores of gfx950
// (flash-style: the S×S score matrix lives only in registers).
//
// Semantics: Tensor::scaled_dot_attention_with_backend / fused_attention_cpu,
// crates/st-tensor/src/pure.rs:4083-4354,11845-11919:
//   logit[i][j] = (q_i·k_j)*scale (+ z_bias[c][j]) (+ attn_bias[c*S+i][j]);  out_i = softmax_j(logit) · V
// `causal` keeps keys 0..=i (crates/st-core/src/backend/cuda_attention.cu:160-164).  The CPU path keeps
// a normalised accumulator per key; this kernel keeps the un-normalised sum and divides once at the end,
// which is the same value up to rounding.
//
// Work split: a 256-thread workgroup owns 128 consecutive queries of one context, 32 per wavefront, and
// streams K/V tiles of BKV keys through two LDS stages.  Everything is computed TRANSPOSED so that one
// lane owns one query:
//   Sᵀ(32 keys × 32 queries) = K_tile · Qᵀ   — A operand = K rows from LDS (one 128-bit read per 4 MFMAs,
//                                              k issued as the pairs {s, s+4}), B operand = Q from registers
//   Oᵀ(D × 32 queries)      += Vᵀ · Pᵀ       — B operand = the probabilities exactly where the Sᵀ
//                                              accumulator left them (register r of lane half h holds key
//                                              (r/4)*8 + 4h + r%4), A operand = V[that key][d] from LDS
// so the running max / sum / rescale factors are per-lane scalars, and the only cross-lane traffic of
// the softmax is one exchange between lane l and lane l^32 for the row maximum.
#include <type_traits>
#include <vector>

#include "device_math.h"
#include "kernels.h"

namespace sthip {

namespace {

struct AttnArgs {
    const float *q;
    const float *k;
    const float *v;
    const float *z_bias;
    const float *attn_bias;
    float *out;
    int contexts, S, D;
    int q_tiles;
    int swizzle;
    float scale;
    // Keys split over workgroups (non-causal fast kernel only): workgroup (…, split) covers keys_per_split keys
    // (a multiple of 64) and leaves its un-normalised output rows in part_o[split][context·S + query][D] and their
    // (reference maximum, sum) in part_ml[split][context·S + query][2]; attention_merge_splits_kernel combines them.
    // Causal calls split per query tile: tile j sees (j + 1)·128 keys, i.e. j / r + 1 chunks of keys_per_split = 128·r
    // keys; causal_items is the number of (tile, chunk) workgroups per context and key_splits the most chunks a tile has.
    int key_splits, keys_per_split;
    int causal_items;
    float *part_o;
    float *part_ml;
};

constexpr int kBQ = 128;
constexpr float kLog2e = 1.4426950408889634f;

// What workgroup `block` of the fast kernel works on.  The kernel and the host-side launch checks share this one
// function, so the grid the launcher asks for and the items the kernel decodes cannot drift apart unnoticed.
//   unit        query tile (non-causal) or the index of a tile pair (causal: tiles q_tiles-1-unit and unit)
//   split       which chunk of keys_per_split keys
//   split_tile  causal launch with split keys: the (single) query tile, -1 otherwise
struct FastItem {
    int ctx, unit, split, split_tile;
};

template <bool CAUSAL>
__host__ __device__ inline FastItem decode_fast_block(const int contexts, const int q_tiles, const int swizzle, const int key_splits,
                                                      const int keys_per_split, const int causal_items, const int block)
{
    // Workgroup -> (context, query tiles).  Workgroup ids are dealt round-robin to the 8 XCDs, so id & 7 picks the
    // XCD; each XCD keeps its own slice of the contexts and walks it context by context, so the workgroups that run
    // together read the same K/V and those stay in that XCD's L2.  Under the causal mask a query tile's cost grows
    // with its index, so a workgroup takes a PAIR of tiles, j and q_tiles-1-j, one after the other: every workgroup
    // then does the same amount of work (q_tiles+1 key tiles), which balances the chip without spreading each
    // context's tiles over the whole launch (longest-first across all contexts balanced as well, but re-read K/V
    // from memory three times over).
    const int per_ctx = CAUSAL ? (q_tiles + 1) / 2 : q_tiles;  // workgroups per context
    FastItem item{0, 0, 0, -1};
    if (swizzle) {
        const int per_xcd = contexts >> 3;
        const int xcd = block & 7, i = block >> 3;
        item.ctx = xcd * per_xcd + i / per_ctx;
        item.unit = i % per_ctx;
        return item;
    }
    int id = block;
    if (CAUSAL && key_splits > 1) {
        // (tile, chunk) items of a context, tiles from the last (most chunks) to the first
        item.ctx = id / causal_items;
        int rest = id - item.ctx * causal_items;
        const int r = keys_per_split / kBQ;
        int j = q_tiles - 1;
        for (; j > 0; --j) {
            const int chunks = j / r + 1;
            if (rest < chunks) break;
            rest -= chunks;
        }
        item.split_tile = j;
        item.split = rest;
        return item;
    }
    if (!CAUSAL) {  // the splits of one query tile are neighbours: they share its Q rows in the L2
        item.split = id % key_splits;
        id /= key_splits;
    }
    item.ctx = id / per_ctx;
    item.unit = id % per_ctx;
    return item;
}

template <bool VEC>
__device__ __forceinline__ float4 load_d4(const float *row, int d, int D, bool row_valid)
{
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (!row_valid) return v;
    if (VEC) {
        if (d < D) v = *reinterpret_cast<const float4 *>(row + d);
    } else {
        if (d + 0 < D) v.x = row[d + 0];
        if (d + 1 < D) v.y = row[d + 1];
        if (d + 2 < D) v.z = row[d + 2];
        if (d + 3 < D) v.w = row[d + 3];
    }
    return v;
}

template <int DPAD, int BKV, bool CAUSAL, bool BIAS, bool VEC>
__global__ __launch_bounds__(256) void attention_f32_kernel(AttnArgs p)
{
    constexpr int KS = DPAD + 4;  // K row stride (floats): 128-bit row reads, rows 16 B skewed
    constexpr int VS = DPAD + 8;  // V row stride: lane halves read rows 4 apart -> different banks
    constexpr int K_ELEMS = BKV * KS, V_ELEMS = BKV * VS;
    constexpr int CHUNKS = DPAD / 8;    // groups of 8 head-dim values = 4 MFMAs each
    constexpr int DT = DPAD / 32;       // 32-row tiles of Oᵀ
    constexpr int KT = BKV / 32;        // 32-key tiles per stage
    constexpr int LOADS = BKV * DPAD / 4 / 256;  // float4 per thread per matrix per stage
    static_assert(LOADS >= 1, "stage too small");

    extern __shared__ __attribute__((aligned(16))) float attn_lds[];
    float *Ks = attn_lds;                 // [2][K_ELEMS]
    float *Vs = attn_lds + 2 * K_ELEMS;   // [2][V_ELEMS]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 31, lh = lane >> 5;
    const int S = p.S, D = p.D;

    int logical = blockIdx.x;
    if (p.swizzle) logical = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int ctx = logical / p.q_tiles;
    // Later query tiles see more keys under the causal mask; run them first.
    const int q_tile = CAUSAL ? (p.q_tiles - 1 - logical % p.q_tiles) : (logical % p.q_tiles);
    const int q0 = q_tile * kBQ;
    const int wq0 = q0 + wave * 32;  // first query of this wavefront
    const int my_q = wq0 + li;
    const size_t ctx_row0 = static_cast<size_t>(ctx) * S;

    // Q fragments: qf[c][s] = Q[my_q][8c + 4h + s]
    float qf[CHUNKS][4];
    {
        const float *qrow = p.q + (ctx_row0 + my_q) * D;
        const bool valid = my_q < S;
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const float4 v = load_d4<VEC>(qrow, c * 8 + lh * 4, D, valid);
            qf[c][0] = v.x; qf[c][1] = v.y; qf[c][2] = v.z; qf[c][3] = v.w;
        }
    }

    f32x16 oacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[t][r] = 0.0f;
    float run_max = -INFINITY;  // in log2 units
    float run_sum = 0.0f;       // this lane half's share of the row sum

    const int key_end = CAUSAL ? min(S, q0 + kBQ) : S;
    const int stages = (key_end + BKV - 1) / BKV;

    float4 rk[LOADS], rv[LOADS];
    auto load_global = [&](int key0) {
#pragma unroll
        for (int r = 0; r < LOADS; ++r) {
            const int f = tid + 256 * r;
            const int row = f / (DPAD / 4), c4 = (f % (DPAD / 4)) * 4;
            const bool valid = key0 + row < S;
            const size_t off = (ctx_row0 + key0 + row) * D;
            rk[r] = load_d4<VEC>(p.k + off, c4, D, valid);
            rv[r] = load_d4<VEC>(p.v + off, c4, D, valid);
        }
    };
    auto store_lds = [&](int stage) {
        float *ks = Ks + stage * K_ELEMS;
        float *vs = Vs + stage * V_ELEMS;
#pragma unroll
        for (int r = 0; r < LOADS; ++r) {
            const int f = tid + 256 * r;
            const int row = f / (DPAD / 4), c4 = (f % (DPAD / 4)) * 4;
            *reinterpret_cast<float4 *>(&ks[row * KS + c4]) = rk[r];
            *reinterpret_cast<float4 *>(&vs[row * VS + c4]) = rv[r];
        }
    };

    const float scale = p.scale;
    const float scale_log2e = p.scale * kLog2e;
    auto compute = [&](int stage, int key0) {
        const float *ks = Ks + stage * K_ELEMS;
        const float *vs = Vs + stage * V_ELEMS;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            const int tile_key0 = key0 + kt * 32;
            if (tile_key0 >= S) continue;                      // workgroup-uniform
            if (CAUSAL && tile_key0 > wq0 + 31) continue;      // wavefront-uniform: tile entirely masked
            f32x16 sacc;
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[r] = 0.0f;
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c) {
                const float4 kv = *reinterpret_cast<const float4 *>(&ks[(kt * 32 + li) * KS + c * 8 + lh * 4]);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.x, qf[c][0], sacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.y, qf[c][1], sacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.z, qf[c][2], sacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.w, qf[c][3], sacc, 0, 0, 0);
            }
            // logits in log2 units; masked entries become -inf
            const bool need_mask = (tile_key0 + 32 > S) || (CAUSAL && tile_key0 + 31 > wq0);
            float tile_max = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = tile_key0 + (r >> 2) * 8 + lh * 4 + (r & 3);
                float t;
                if (BIAS) {
                    // reference order: dot*scale, + z_bias, + attn_bias (pure.rs:11878-11887)
                    float logit = sacc[r] * scale;
                    if (key < S && my_q < S) {
                        if (p.z_bias) logit += p.z_bias[ctx_row0 + key];
                        if (p.attn_bias) logit += p.attn_bias[(ctx_row0 + my_q) * S + key];
                    }
                    t = logit * kLog2e;
                } else {
                    t = sacc[r] * scale_log2e;
                }
                if (need_mask) {
                    if (key >= S || (CAUSAL && key > my_q)) t = -INFINITY;
                }
                sacc[r] = t;
                tile_max = fmaxf(tile_max, t);
            }
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32));
            const float new_max = fmaxf(run_max, tile_max);
            const float safe_max = new_max == -INFINITY ? 0.0f : new_max;
            const float alpha = exp2f(run_max - safe_max);  // run_max = -inf -> 0
            float tile_sum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float pr = exp2f(sacc[r] - safe_max);
                sacc[r] = pr;
                tile_sum += pr;
            }
            run_sum = run_sum * alpha + tile_sum;
            run_max = new_max;
#pragma unroll
            for (int t = 0; t < DT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[t][r] *= alpha;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int krow = kt * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
#pragma unroll
                for (int t = 0; t < DT; ++t) {
                    const float vv = vs[krow * VS + t * 32 + li];
                    oacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv, sacc[r], oacc[t], 0, 0, 0);
                }
            }
        }
    };

    if (stages > 0) {
        load_global(0);
        store_lds(0);
    }
    __syncthreads();
    for (int t = 0; t < stages; ++t) {
        const bool more = t + 1 < stages;
        if (more) load_global((t + 1) * BKV);
        compute(t & 1, t * BKV);
        if (more) store_lds((t + 1) & 1);
        __syncthreads();
    }

    const float total = run_sum + __shfl_xor(run_sum, 32);
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    if (my_q < S) {
        float *orow = p.out + (ctx_row0 + my_q) * D;
#pragma unroll
        for (int t = 0; t < DT; ++t) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = t * 32 + g * 8 + lh * 4;
                if (VEC) {
                    if (d < D)
                        *reinterpret_cast<float4 *>(orow + d) =
                            make_float4(oacc[t][g * 4 + 0] * inv, oacc[t][g * 4 + 1] * inv, oacc[t][g * 4 + 2] * inv,
                                        oacc[t][g * 4 + 3] * inv);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (d + e < D) orow[d + e] = oacc[t][g * 4 + e] * inv;
                }
            }
        }
    }
}

// -------------------------------------------------------------------------------------------------
// Fast path: head_dim a multiple of 4, 16-byte aligned operands; BIAS adds z_bias / attn_bias where their rows can
// be read 128 bits at a time (sequence a multiple of 4), otherwise biased calls take the general kernel above.
//
// Same transposed formulation as the general kernel above, tuned for the matrix pipe:
//   * 64 keys (two 32-key tiles) per softmax step: the two QKᵀ accumulations are independent MFMA
//     chains, and the max / exchange / rescale bookkeeping is paid once per 64 keys;
//   * V is staged exactly as stored (rows = keys, 128-bit writes); the PV operand is one conflict-free 32-bit
//     read per MFMA at an immediate offset.  (Staging V transposed saved three of four reads, but its 32-bit
//     scatter writes spent more than half of the LDS cycles on bank conflicts.)
//   * the output accumulator is rescaled only when some lane's running maximum actually moved
//     (wavefront-uniform test) — after the first few key tiles it almost never does;
//   * exp2 is the bare v_exp_f32 (arguments are <= 0; results below 2^-126 may flush to zero);
//   * K/V rows are fetched through a buffer descriptor that covers exactly this context, so rows past
//     the sequence end read as zero without branches; masking code runs only on the tiles that
//     touch the sequence end or the causal diagonal.
// -------------------------------------------------------------------------------------------------
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

// (Up to head_dim 64 two workgroups fit a compute unit, i.e. two wavefronts per SIMD: the register allocation is
// held to that; the 128-wide form has LDS for one workgroup only.)
template <int DPAD, bool CAUSAL, bool BIAS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(DPAD <= 64 ? 2 : 1))) void attention_f32_fast_kernel(AttnArgs p)
{
    constexpr int BKV = 64;
    constexpr int KS = DPAD + 4;   // K row stride (floats)
    constexpr int VS = DPAD + 8;   // V row stride (floats): four rows are 32 banks apart (see the PV reads)
    constexpr int K_ELEMS = BKV * KS, V_ELEMS = BKV * VS;
    constexpr int CHUNKS = DPAD / 8;
    constexpr int DT = DPAD / 32;
    constexpr int LOADS = BKV * DPAD / 4 / 256;
    extern __shared__ __attribute__((aligned(16))) float attn_lds[];
    float *Ks = attn_lds;                // [2][K_ELEMS]
    float *Vs = attn_lds + 2 * K_ELEMS;  // [2][V_ELEMS]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same in every lane, and known to be
    const int li = lane & 31, lh = lane >> 5;
    const int S = p.S, D = p.D;

    const FastItem item = decode_fast_block<CAUSAL>(p.contexts, p.q_tiles, p.swizzle, p.key_splits, p.keys_per_split,
                                                    p.causal_items, static_cast<int>(blockIdx.x));
    const int ctx = item.ctx, unit = item.unit, split = item.split;
    const int split_tile = item.split_tile;  // causal with split keys: this workgroup's query tile (no pairing then)
    const size_t ctx_elem0 = static_cast<size_t>(ctx) * S * D;
    const unsigned ctx_bytes = static_cast<unsigned>(S) * static_cast<unsigned>(D) * 4u;
    const __amdgpu_buffer_rsrc_t rsrc_q =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.q + ctx_elem0), 0, static_cast<int>(ctx_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_k =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.k + ctx_elem0), 0, static_cast<int>(ctx_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_v =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.v + ctx_elem0), 0, static_cast<int>(ctx_bytes), 0x00020000);
    const bool ragged_d = D != DPAD;  // chunks past head_dim must read as zero

    auto fetch4 = [&](const __amdgpu_buffer_rsrc_t &rsrc, int row, int d) -> float4 {
        const u32x4_t raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (static_cast<unsigned>(row) * D + d) * 4u, 0, 0);
        float4 v = make_float4(__uint_as_float(raw.x), __uint_as_float(raw.y), __uint_as_float(raw.z), __uint_as_float(raw.w));
        if (ragged_d && d >= D) v = make_float4(0.f, 0.f, 0.f, 0.f);
        return v;
    };

    const int passes = (CAUSAL && split_tile < 0 && unit != p.q_tiles - 1 - unit) ? 2 : 1;
    for (int pass = 0; pass < passes; ++pass) {
    const int q_tile = !CAUSAL ? unit : split_tile >= 0 ? split_tile : (pass == 0 ? p.q_tiles - 1 - unit : unit);  // the long tile first
    const int q0 = q_tile * kBQ;
    const int wq0 = q0 + wave * 32;
    const int my_q = wq0 + li;
    // Q fragments: qf[c][s] = Q[my_q][8c + 4h + s]; rows past the end read as zero.
    float qf[CHUNKS][4];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const float4 v = fetch4(rsrc_q, my_q, c * 8 + lh * 4);
        qf[c][0] = v.x; qf[c][1] = v.y; qf[c][2] = v.z; qf[c][3] = v.w;
        // A negative scale is moved into Q so that the scale applied below is never negative and the running
        // maximum can be taken over the raw dot products.
        if (p.scale < 0.0f) {
            qf[c][0] = -qf[c][0]; qf[c][1] = -qf[c][1]; qf[c][2] = -qf[c][2]; qf[c][3] = -qf[c][3];
        }
    }

    f32x16 oacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
        oacc[t] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float run_max = -INFINITY;
    float run_sum = 0.0f;

    const bool split_keys = !CAUSAL || split_tile >= 0;
    const int key_first = split_keys ? split * p.keys_per_split : 0;
    const int key_end = min(CAUSAL ? min(S, q0 + kBQ) : S, split_keys ? key_first + p.keys_per_split : S);
    const int stages = (key_end - key_first + BKV - 1) / BKV;

    float4 rk[LOADS], rv[LOADS];
    auto load_global = [&](int key0) {
#pragma unroll
        for (int r = 0; r < LOADS; ++r) {
            const int f = tid + 256 * r;
            const int row = f / (DPAD / 4), c4 = (f % (DPAD / 4)) * 4;
            rk[r] = fetch4(rsrc_k, key0 + row, c4);
            rv[r] = fetch4(rsrc_v, key0 + row, c4);
        }
    };
    auto store_lds = [&](int stage) {
        float *ks = Ks + stage * K_ELEMS;
        float *vs = Vs + stage * V_ELEMS;
#pragma unroll
        for (int r = 0; r < LOADS; ++r) {
            const int f = tid + 256 * r;
            const int row = f / (DPAD / 4), c4 = (f % (DPAD / 4)) * 4;
            *reinterpret_cast<float4 *>(&ks[row * KS + c4]) = rk[r];
            *reinterpret_cast<float4 *>(&vs[row * VS + c4]) = rv[r];
        }
    };

    // The maximum is kept in units of the raw dot product and the scale is folded into the exponent:
    // p = exp2(fma(dot, scale·log2e, −max·scale·log2e)).  (Floored at a tiny positive value so that a zero scale
    // still turns masked (−inf) logits into weight 0 instead of −inf·0.)
    const float scale_log2e = fmaxf(fabsf(p.scale) * kLog2e, 1e-30f);
    // With additive biases the logits are formed explicitly (dot·scale·log2e + bias·log2e) before the maximum is
    // taken, so everything after that works in log2 units: the factor applied in the exponent is then 1.
    const float exp_scale = BIAS ? 1.0f : scale_log2e;
    const float lag = 8.0f / exp_scale;  // 2^8 in the units the maximum is kept in, see below
    const float *zb_ctx = BIAS && p.z_bias ? p.z_bias + static_cast<size_t>(ctx) * S : nullptr;
    const float *ab_row = BIAS && p.attn_bias && my_q < S
                              ? p.attn_bias + (static_cast<size_t>(ctx) * S + my_q) * static_cast<size_t>(S) : nullptr;
    // NT = number of 32-key tiles of this stage this wavefront works on (1 or 2).
    // MAY_MASK = false: the caller knows that every key of the stage exists and (causal) lies at or below every query
    // row of this wavefront.
    auto compute = [&](auto nt_tag, auto may_mask_tag, int stage, int key0) {
        constexpr int NT = decltype(nt_tag)::value;
        constexpr bool MAY_MASK = decltype(may_mask_tag)::value;
        const float *ks = Ks + stage * K_ELEMS;
        const float *vs = Vs + stage * V_ELEMS;
        f32x16 sacc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t)
            sacc[t] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        // Biases of this lane's query for the keys its registers hold (four consecutive keys per register group: one
        // 128-bit load each; S is a multiple of 4 on this path, so a group is inside the sequence or past it as a
        // whole), requested before the QKᵀ MFMAs so that they arrive behind them.
        float4 bias4[BIAS ? NT : 1][4];
        if constexpr (BIAS) {
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int key = key0 + t * 32 + g * 8 + lh * 4;
                    float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (key < S) {
                        if (ab_row) b = *reinterpret_cast<const float4 *>(ab_row + key);
                        if (zb_ctx) {
                            const float4 z = *reinterpret_cast<const float4 *>(zb_ctx + key);
                            b.x += z.x; b.y += z.y; b.z += z.z; b.w += z.w;
                        }
                    }
                    bias4[t][g] = b;
                }
        }
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            float4 kv[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) kv[t] = *reinterpret_cast<const float4 *>(&ks[(t * 32 + li) * KS + c * 8 + lh * 4]);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                sacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[t].x, qf[c][0], sacc[t], 0, 0, 0);
                sacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[t].y, qf[c][1], sacc[t], 0, 0, 0);
                sacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[t].z, qf[c][2], sacc[t], 0, 0, 0);
                sacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[t].w, qf[c][3], sacc[t], 0, 0, 0);
            }
        }
        if constexpr (BIAS) {
            // logit = (dot·scale + z_bias) + attn_bias of pure.rs:11870-11880, in log2 units
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const float b[4] = {bias4[t][g].x, bias4[t][g].y, bias4[t][g].z, bias4[t][g].w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) sacc[t][g * 4 + e] = fmaf(sacc[t][g * 4 + e], scale_log2e, b[e] * kLog2e);
                }
        }
        // logits in log2 units; the masking code only runs where a tile crosses the sequence end or the diagonal
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
        // The reference maximum in the exponent may lag the true running maximum by up to 2^8 (weights then reach
        // 256 instead of 1, which changes nothing in f32 but the exponent); the accumulators are rescaled only when
        // some row's maximum has moved by more than that, which after the first key tiles is rare.
        if (__any(tile_max > run_max + lag)) {  // wavefront-uniform
            const float new_max = fmaxf(run_max, tile_max);
            const float new_safe = new_max == -INFINITY ? 0.0f : new_max;
            const float alpha = __builtin_amdgcn_exp2f((run_max - new_safe) * exp_scale);  // run_max = -inf -> 0
            run_sum *= alpha;
#pragma unroll
            for (int t = 0; t < DT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[t][r] *= alpha;
            run_max = new_max;
        }
        const float safe_max = run_max == -INFINITY ? 0.0f : run_max;
        const float shift = -safe_max * exp_scale;
        float tile_sum = 0.0f;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float pr = __builtin_amdgcn_exp2f(fmaf(sacc[t][r], exp_scale, shift));
                sacc[t][r] = pr;
                tile_sum += pr;
            }
        run_sum += tile_sum;
        // Oᵀ += Vᵀ·Pᵀ with V as stored (rows = keys): probability register r of lane half h belongs to key
        // (r/4)*8 + 4h + r%4, so the A operand of that MFMA is V[that key][32·dt + li] — one 32-bit read whose 64
        // lanes cover 32 consecutive floats of two rows four apart, 32 banks apart with the row stride above: no
        // bank conflicts, nothing transposed on the way into LDS, and every address is this lane's base plus an
        // immediate.
        const float *v_lane = vs + (lh * 4) * VS + li;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float vv[DT][4];
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int e = 0; e < 4; ++e) vv[dt][e] = v_lane[(t * 32 + g * 8 + e) * VS + dt * 32];
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv[dt][e], sacc[t][g * 4 + e], oacc[dt], 0, 0, 0);
            }
    };

    if (stages > 0) {
        load_global(key_first);
        store_lds(0);
    }
    __syncthreads();
    // The stages whose keys all exist and need no causal mask for any row of this wavefront come first, in a loop with
    // one path through it: a loop body that branches between the one-tile, the two-tile and the skipped form has the
    // output accumulators merged after the branch, and the compiler then copies all of their registers once per stage
    // behind the stage's last matrix instructions, whose latency the copies wait out.  The stages on and beyond the
    // diagonal, a ragged last stage and wavefronts whose rows lie past the sequence end take the branching loop after it.
    static_assert(BKV == 64, "a stage is two 32-key tiles");
    const int limit = wq0 >= S ? 0 : CAUSAL ? min(S, wq0 + 32) : S;
    const int plain_end = wq0 >= S ? key_first : CAUSAL ? min(S, wq0 + 1) : S;
    const int plain_stages = max(0, min(stages, (plain_end - key_first) / BKV));
    int t = 0;
    for (; t < plain_stages; ++t) {
        const bool more = t + 1 < stages;
        if (more) load_global(key_first + (t + 1) * BKV);
        compute(std::integral_constant<int, 2>{}, std::false_type{}, t & 1, key_first + t * BKV);
        if (more) store_lds((t + 1) & 1);
        __syncthreads();
    }
    for (; t < stages; ++t) {
        const bool more = t + 1 < stages;
        if (more) load_global(key_first + (t + 1) * BKV);
        const int key0 = key_first + t * BKV;
        // Tiles entirely past the sequence end or (causal) entirely above this wavefront's rows are skipped.
        // So is everything in a wavefront whose 32 query rows lie past the sequence end (the last tile of 197 rows).
        if (key0 + 32 < limit) compute(std::integral_constant<int, 2>{}, std::true_type{}, t & 1, key0);
        else if (key0 < limit) compute(std::integral_constant<int, 1>{}, std::true_type{}, t & 1, key0);
        if (more) store_lds((t + 1) & 1);
        __syncthreads();
    }

    const float total = run_sum + __shfl_xor(run_sum, 32);
    {
        if (p.key_splits > 1) {
            if (my_q < S) {
                const size_t row = (static_cast<size_t>(split) * p.contexts + ctx) * S + my_q;
                float *orow = p.part_o + row * D;
#pragma unroll
                for (int t = 0; t < DT; ++t)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int d = t * 32 + g * 8 + lh * 4;
                        if (d < D)
                            *reinterpret_cast<float4 *>(orow + d) =
                                make_float4(oacc[t][g * 4 + 0], oacc[t][g * 4 + 1], oacc[t][g * 4 + 2], oacc[t][g * 4 + 3]);
                    }
                if (lh == 0) *reinterpret_cast<float2 *>(p.part_ml + row * 2) = make_float2(run_max, total);
            }
            return;
        }
    }
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    if (my_q < S) {
        float *orow = p.out + ctx_elem0 + static_cast<size_t>(my_q) * D;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = t * 32 + g * 8 + lh * 4;
                if (d < D)
                    *reinterpret_cast<float4 *>(orow + d) = make_float4(oacc[t][g * 4 + 0] * inv, oacc[t][g * 4 + 1] * inv,
                                                                        oacc[t][g * 4 + 2] * inv, oacc[t][g * 4 + 3] * inv);
            }
    }
    }  // pass
}

// -------------------------------------------------------------------------------------------------
// Many short contexts (windowed attention: thousands of contexts of 16 to 64 positions).  The kernels above give a
// context a workgroup and a 128-row query tile, which is mostly padding here, and such launches are memory-bound:
// 16384 contexts of 16 × 64 took 218 µs, 1.2 TB/s.  Here ONE WAVEFRONT owns a context of up to 64 positions: it stages
// that context's K and V (rows past the end as zeros) in a slice of LDS of its own, so nothing in the kernel waits on
// a workgroup barrier, and with all keys present at once the softmax is the plain one, no running maximum.  Same
// transposed products as above: Sᵀ = K·Qᵀ leaves every lane the scores of its own query, which are the B operand of
// Oᵀ = Vᵀ·Pᵀ as they stand.  WAVES wavefronts (contexts) per workgroup: as many as fit the LDS.
// -------------------------------------------------------------------------------------------------
template <int DPAD, bool CAUSAL, int ROWS, int WAVES, bool KDIRECT>
__global__ __launch_bounds__(64 * WAVES) void attention_f32_tiny_kernel(AttnArgs p)
{
    constexpr int KS = DPAD + 4, VS = DPAD + 8;  // row strides as in the fast kernel (conflict-free fragment reads)
    // ROWS: 32 or 64 staged positions, at least S.  KDIRECT: the K fragments come straight from global memory into
    // registers, as Q's do (a lane's fragment is 16 contiguous bytes of one row), and only V is staged: half the LDS,
    // twice the wavefronts per SIMD to overlap one context's loads with another's products.
    constexpr int K_ELEMS = KDIRECT ? 0 : ROWS * KS, V_ELEMS = ROWS * VS;
    constexpr int NTMAX = ROWS / 32;
    constexpr int CHUNKS = DPAD / 8, DT = DPAD / 32;
    constexpr int QUADS = DPAD / 4;              // float4 per row
    constexpr int PER_LANE = ROWS * QUADS / 64;  // ROWS × QUADS float4 over 64 lanes
    constexpr int BATCH = PER_LANE < 8 ? PER_LANE : 8;
    extern __shared__ __attribute__((aligned(16))) float attn_lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int S = p.S, D = p.D;
    const int ctx = static_cast<int>(blockIdx.x) * WAVES + wave;
    if (ctx >= p.contexts) return;  // (no workgroup barrier anywhere below)
    float *ks = attn_lds + wave * (K_ELEMS + V_ELEMS);
    float *vs = ks + K_ELEMS;
    const size_t ctx_elem0 = static_cast<size_t>(ctx) * S * D;
    const float *q = p.q + ctx_elem0, *k = p.k + ctx_elem0, *v = p.v + ctx_elem0;

    float4 kreg[KDIRECT ? CHUNKS : 1][NTMAX];
    if constexpr (KDIRECT) {
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
            for (int t = 0; t < NTMAX; ++t) {
                const int row = t * 32 + li, d = c * 8 + lh * 4;
                kreg[c][t] = (row < S && d < D) ? *reinterpret_cast<const float4 *>(k + static_cast<size_t>(row) * D + d)
                                                : make_float4(0.f, 0.f, 0.f, 0.f);
            }
    }
    // Stage K and V: float4 number f = lane + 64·r of the ROWS × DPAD tile, BATCH of them requested before the first store.
#pragma unroll
    for (int r0 = 0; r0 < PER_LANE; r0 += BATCH) {
        float4 rk[BATCH], rv[BATCH];
#pragma unroll
        for (int r = 0; r < BATCH; ++r) {
            const int f = lane + 64 * (r0 + r);
            const int row = f / QUADS, c4 = (f % QUADS) * 4;
            const bool inside = row < S && c4 < D;
            rk[r] = (!KDIRECT && inside) ? *reinterpret_cast<const float4 *>(k + static_cast<size_t>(row) * D + c4) : make_float4(0.f, 0.f, 0.f, 0.f);
            rv[r] = inside ? *reinterpret_cast<const float4 *>(v + static_cast<size_t>(row) * D + c4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int r = 0; r < BATCH; ++r) {
            const int f = lane + 64 * (r0 + r);
            const int row = f / QUADS, c4 = (f % QUADS) * 4;
            if constexpr (!KDIRECT) *reinterpret_cast<float4 *>(&ks[row * KS + c4]) = rk[r];
            *reinterpret_cast<float4 *>(&vs[row * VS + c4]) = rv[r];
        }
    }
    // The wavefront's own LDS writes are visible to its later reads (LDS operations of a wavefront execute in order);
    // the fence keeps the compiler from moving the reads up.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    const float scale_log2e = p.scale * kLog2e;  // logits in log2 units: dot · scale · log2(e), either sign
    for (int q0 = 0; q0 < S; q0 += 32) {
        const int my_q = q0 + li;
        float qf[CHUNKS][4];
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int d = c * 8 + lh * 4;
            const float4 t = (my_q < S && d < D) ? *reinterpret_cast<const float4 *>(q + static_cast<size_t>(my_q) * D + d)
                                                 : make_float4(0.f, 0.f, 0.f, 0.f);
            qf[c][0] = t.x; qf[c][1] = t.y; qf[c][2] = t.z; qf[c][3] = t.w;
        }
        const int key_limit = CAUSAL ? min(S, q0 + 32) : S;  // keys this chunk of queries can see
        auto compute = [&](auto nt_tag) {
            constexpr int NT = decltype(nt_tag)::value;
            f32x16 sacc[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t)
                sacc[t] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c) {
                float4 kv[NT];
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    if constexpr (KDIRECT) kv[t] = kreg[c][t];
                    else kv[t] = *reinterpret_cast<const float4 *>(&ks[(t * 32 + li) * KS + c * 8 + lh * 4]);
                }
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    sacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[t].x, qf[c][0], sacc[t], 0, 0, 0);
                    sacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[t].y, qf[c][1], sacc[t], 0, 0, 0);
                    sacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[t].z, qf[c][2], sacc[t], 0, 0, 0);
                    sacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[t].w, qf[c][3], sacc[t], 0, 0, 0);
                }
            }
            // register r of lane half h is key 32t + (r/4)·8 + 4h + r%4 for this lane's query
            float top = -INFINITY;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = t * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                    float logit = sacc[t][r] * scale_log2e;
                    if (key >= S || (CAUSAL && key > my_q)) logit = -INFINITY;
                    sacc[t][r] = logit;
                    top = fmaxf(top, logit);
                }
            top = fmaxf(top, __shfl_xor(top, 32));  // key 0 is visible to every query: finite
            float sum = 0.0f;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float pr = __builtin_amdgcn_exp2f(sacc[t][r] - top);
                    sacc[t][r] = pr;
                    sum += pr;
                }
            sum += __shfl_xor(sum, 32);
            f32x16 oacc[DT];
#pragma unroll
            for (int t = 0; t < DT; ++t)
                oacc[t] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            const float *v_lane = vs + (lh * 4) * VS + li;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    float vv[DT][4];
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int e = 0; e < 4; ++e) vv[dt][e] = v_lane[(t * 32 + g * 8 + e) * VS + dt * 32];
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv[dt][e], sacc[t][g * 4 + e], oacc[dt], 0, 0, 0);
                }
            const float inv = 1.0f / sum;
            if (my_q < S) {
                float *orow = p.out + ctx_elem0 + static_cast<size_t>(my_q) * D;
#pragma unroll
                for (int t = 0; t < DT; ++t)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int d = t * 32 + g * 8 + lh * 4;
                        if (d < D)
                            *reinterpret_cast<float4 *>(orow + d) = make_float4(oacc[t][g * 4 + 0] * inv, oacc[t][g * 4 + 1] * inv,
                                                                                oacc[t][g * 4 + 2] * inv, oacc[t][g * 4 + 3] * inv);
                    }
            }
        };
        if constexpr (ROWS > 32) {
            if (key_limit > 32) compute(std::integral_constant<int, 2>{});
            else compute(std::integral_constant<int, 1>{});
        } else {
            compute(std::integral_constant<int, 1>{});
        }
    }
}

template <int DPAD, bool CAUSAL, int ROWS>
hipError_t launch_tiny_rows(const AttnArgs &args, hipStream_t stream)
{
    // K in registers where the staged slices would leave one or two wavefronts per SIMD (64 positions: 49 × 32 94 → 88 µs,
    // 64 × 64 38.6 → 35.6 µs); at 32 positions it gains nothing, at 128 values a head it would take 128 registers a lane.
    constexpr bool KDIRECT = DPAD <= 64 && ROWS == 64;
    constexpr size_t wave_bytes = static_cast<size_t>(ROWS) * ((KDIRECT ? 0 : DPAD + 4) + (DPAD + 8)) * sizeof(float);
    constexpr int WAVES = wave_bytes * 4 <= 160 * 1024 ? 4 : 2;
    constexpr size_t lds_bytes = wave_bytes * WAVES;
    static_assert(lds_bytes <= 160 * 1024, "the wavefronts' K and V slices fit the LDS");
    if (args.S > ROWS) return hipErrorInvalidValue;
    auto kernel = attention_f32_tiny_kernel<DPAD, CAUSAL, ROWS, WAVES, KDIRECT>;
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    const unsigned blocks = static_cast<unsigned>((args.contexts + WAVES - 1) / WAVES);
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(64 * WAVES), lds_bytes, stream, args);
    return hipGetLastError();
}

template <int DPAD, bool CAUSAL>
hipError_t launch_tiny(const AttnArgs &args, hipStream_t stream)
{
    return args.S <= 32 ? launch_tiny_rows<DPAD, CAUSAL, 32>(args, stream) : launch_tiny_rows<DPAD, CAUSAL, 64>(args, stream);
}

// Combines the key splits of the fast kernel: with m = max over splits of their reference maxima,
// out = Σ_s 2^((m_s − m)·exp_scale)·O_s / Σ_s 2^((m_s − m)·exp_scale)·l_s, splits added in order.  One thread per four
// output values.
__global__ __launch_bounds__(256) void attention_merge_splits_kernel(AttnArgs p, float exp_scale, int causal_r)
{
    const int D = p.D;
    const int quads = D / 4;
    const size_t rows = static_cast<size_t>(p.contexts) * p.S;
    const size_t id = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (id >= rows * quads) return;
    const size_t row = id / quads;
    const int d = static_cast<int>(id % quads) * 4;
    // Eight splits at a time, all their loads requested before the first is used (a plain loop over the splits is a
    // chain of dependent memory round trips); splits past the end repeat the last one with weight zero.
    // causal: the query tile of this row has (tile / r) + 1 chunks of keys; the planes beyond were never written
    const int splits = causal_r > 0 ? (static_cast<int>(row % static_cast<size_t>(p.S)) / kBQ) / causal_r + 1 : p.key_splits;
    const int last = splits - 1;
    float top = -INFINITY;
    for (int s0 = 0; s0 < splits; s0 += 8) {
        float m[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) m[j] = p.part_ml[(min(s0 + j, last) * rows + row) * 2];
#pragma unroll
        for (int j = 0; j < 8; ++j) top = fmaxf(top, m[j]);
    }
    const float safe_top = top == -INFINITY ? 0.0f : top;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    float denom = 0.0f;
    for (int s0 = 0; s0 < splits; s0 += 8) {
        float2 ml[8];
        float4 o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const size_t at = min(s0 + j, last) * rows + row;
            ml[j] = *reinterpret_cast<const float2 *>(p.part_ml + at * 2);
            o[j] = *reinterpret_cast<const float4 *>(p.part_o + at * D + d);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            // a split with no weight: 2^-inf = 0
            const float w = s0 + j <= last ? __builtin_amdgcn_exp2f((ml[j].x - safe_top) * exp_scale) : 0.0f;
            acc.x = fmaf(w, o[j].x, acc.x); acc.y = fmaf(w, o[j].y, acc.y);
            acc.z = fmaf(w, o[j].z, acc.z); acc.w = fmaf(w, o[j].w, acc.w);
            denom = fmaf(w, ml[j].y, denom);
        }
    }
    const float inv = denom > 0.0f ? 1.0f / denom : 0.0f;
    *reinterpret_cast<float4 *>(p.out + row * D + d) = make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv);
}

// Launch plan of the fast kernel: fills the split fields of `args` and returns the number of workgroups; `causal_r` is
// the r of the causal key split (0 when the launch is not split that way).  Pure host arithmetic.
size_t plan_fast(AttnArgs &args, const bool causal, int *causal_r)
{
    size_t blocks = static_cast<size_t>(args.contexts) * (causal ? (args.q_tiles + 1) / 2 : args.q_tiles);
    args.key_splits = 1;
    args.keys_per_split = args.S;
    args.causal_items = 0;
    *causal_r = 0;
    constexpr size_t kTargetBlocks = 512;
    if (blocks * 2 > kTargetBlocks || args.S < 256) return blocks;
    if (causal) {
        // Few contexts: pairs of query tiles leave most of the chip idle (8 contexts of 2048: 64 workgroups, slower than
        // the non-causal call that does twice the work).  Split every tile's keys into chunks of 128·r instead, with the
        // largest r that still gives about two workgroups per compute unit; all (tile, chunk) items then cost the same.
        const size_t tiles = static_cast<size_t>(args.q_tiles);
        auto items = [&](size_t r) {
            size_t total = 0;
            for (size_t j = 0; j < tiles; ++j) total += j / r + 1;
            return total;
        };
        size_t r = tiles;
        while (r > 1 && static_cast<size_t>(args.contexts) * items(r) < kTargetBlocks) --r;
        const size_t per_context = items(r);
        // (r == tiles would be one chunk per tile: nothing to merge, and the kernel tells the two forms apart by
        // key_splits > 1 — such launches keep the pairing.)
        if (r < tiles && static_cast<size_t>(args.contexts) * per_context > blocks) {
            *causal_r = static_cast<int>(r);
            args.keys_per_split = static_cast<int>(r) * kBQ;
            args.key_splits = static_cast<int>((tiles - 1) / r + 1);
            args.causal_items = static_cast<int>(per_context);
            blocks = static_cast<size_t>(args.contexts) * per_context;
        }
    } else {
        // Few query tiles (the reference's own caller attends within one context: crates/st-nn/src/z_rba/attention.rs:586):
        // split the keys over workgroups until the launch offers about two workgroups per compute unit, 128 keys at least
        // per split, and merge the partial rows in a second kernel.
        const size_t want = (kTargetBlocks + blocks - 1) / blocks;
        const size_t most = static_cast<size_t>(args.S) / 128;
        const size_t splits = std::min(want, most);
        const size_t per = ((static_cast<size_t>(args.S) + splits - 1) / splits + 63) / 64 * 64;
        args.keys_per_split = static_cast<int>(per);
        args.key_splits = static_cast<int>((static_cast<size_t>(args.S) + per - 1) / per);
        blocks *= static_cast<size_t>(args.key_splits);
    }
    if (args.key_splits > 1) args.swizzle = 0;
    return blocks;
}

// True when workgroup `block` of a planned launch decodes to a (context, query tile, key chunk) inside the operands.
bool fast_block_in_range(const AttnArgs &args, const bool causal, const size_t block)
{
    const FastItem item = causal ? decode_fast_block<true>(args.contexts, args.q_tiles, args.swizzle, args.key_splits,
                                                           args.keys_per_split, args.causal_items, static_cast<int>(block))
                                 : decode_fast_block<false>(args.contexts, args.q_tiles, args.swizzle, args.key_splits,
                                                            args.keys_per_split, args.causal_items, static_cast<int>(block));
    if (item.ctx < 0 || item.ctx >= args.contexts || item.split < 0 || item.split >= args.key_splits) return false;
    if (item.split_tile >= 0) {  // causal, split keys: chunk `split` of the (tile + 1)·128 keys the tile sees
        return item.split_tile < args.q_tiles && item.split * args.keys_per_split < std::min(args.S, (item.split_tile + 1) * kBQ);
    }
    if (causal) return item.unit >= 0 && item.unit < (args.q_tiles + 1) / 2;
    return item.unit >= 0 && item.unit < args.q_tiles && item.split * args.keys_per_split < args.S;
}

// The launch arithmetic, checked before every launch of the fast kernel: the grid is what the decode assumes, fits
// the 32-bit ids the kernel computes with, and its first and last workgroups decode to items inside the operands.
bool fast_plan_consistent(const AttnArgs &args, const bool causal, const size_t blocks)
{
    if (blocks == 0 || blocks > 0x7fffffffu) return false;
    if (args.swizzle && (args.contexts % 8 != 0 || args.key_splits != 1)) return false;
    const size_t per_ctx = causal ? (args.key_splits > 1 ? static_cast<size_t>(args.causal_items) : (args.q_tiles + 1) / 2)
                                  : static_cast<size_t>(args.q_tiles) * args.key_splits;
    if (blocks != static_cast<size_t>(args.contexts) * per_ctx) return false;
    if (args.key_splits > 1 && (args.keys_per_split <= 0 || args.keys_per_split % 64 != 0)) return false;
    return fast_block_in_range(args, causal, 0) && fast_block_in_range(args, causal, blocks - 1);
}

template <int DPAD, bool CAUSAL, bool BIAS = false>
hipError_t launch_fast(AttnArgs args, hipStream_t stream)
{
    constexpr size_t lds_bytes = 2 * static_cast<size_t>(64) * ((DPAD + 4) + (DPAD + 8)) * sizeof(float);
    auto kernel = attention_f32_fast_kernel<DPAD, CAUSAL, BIAS>;
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    args.part_o = args.part_ml = nullptr;
    int causal_r = 0;
    const size_t blocks = plan_fast(args, CAUSAL, &causal_r);
    if (!fast_plan_consistent(args, CAUSAL, blocks)) return hipErrorInvalidConfiguration;
    if (args.key_splits > 1) {
        const size_t rows = static_cast<size_t>(args.contexts) * args.S;
        const size_t o_bytes = static_cast<size_t>(args.key_splits) * rows * args.D * sizeof(float);
        const size_t ml_bytes = static_cast<size_t>(args.key_splits) * rows * 2 * sizeof(float);
        void *workspace = nullptr;
        rc = stream_workspace(stream, o_bytes + ml_bytes, &workspace);
        if (rc != hipSuccess) return rc;
        args.part_o = static_cast<float *>(workspace);
        args.part_ml = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) + o_bytes);
    }
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), lds_bytes, stream, args);
    rc = hipGetLastError();
    if (rc != hipSuccess || args.key_splits == 1) return rc;
    const float scale_log2e = fmaxf(fabsf(args.scale) * kLog2e, 1e-30f);
    const size_t work = static_cast<size_t>(args.contexts) * args.S * (args.D / 4);
    hipLaunchKernelGGL(attention_merge_splits_kernel, dim3(static_cast<unsigned>((work + 255) / 256)), dim3(256), 0, stream, args,
                       BIAS ? 1.0f : scale_log2e, causal_r);
    return hipGetLastError();
}

template <int DPAD, int BKV, bool CAUSAL, bool BIAS, bool VEC>
hipError_t launch_variant(const AttnArgs &args, hipStream_t stream)
{
    constexpr size_t lds_bytes = 2 * static_cast<size_t>(BKV) * ((DPAD + 4) + (DPAD + 8)) * sizeof(float);
    auto kernel = attention_f32_kernel<DPAD, BKV, CAUSAL, BIAS, VEC>;
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    const size_t blocks = static_cast<size_t>(args.contexts) * args.q_tiles;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), lds_bytes, stream, args);
    return hipGetLastError();
}

template <int DPAD, int BKV>
hipError_t launch_dpad(const AttnArgs &args, bool causal, bool bias, bool vec, hipStream_t stream)
{
    if (causal) {
        if (bias) return vec ? launch_variant<DPAD, BKV, true, true, true>(args, stream)
                             : launch_variant<DPAD, BKV, true, true, false>(args, stream);
        return vec ? launch_variant<DPAD, BKV, true, false, true>(args, stream)
                   : launch_variant<DPAD, BKV, true, false, false>(args, stream);
    }
    if (bias) return vec ? launch_variant<DPAD, BKV, false, true, true>(args, stream)
                         : launch_variant<DPAD, BKV, false, true, false>(args, stream);
    return vec ? launch_variant<DPAD, BKV, false, false, true>(args, stream)
               : launch_variant<DPAD, BKV, false, false, false>(args, stream);
}

}  // namespace

AttentionPlanReport attention_f32_plan_report(size_t contexts, size_t sequence, size_t head_dim, bool causal, bool biased)
{
    AttentionPlanReport report{};
    if (contexts == 0 || sequence == 0 || head_dim == 0 || head_dim > static_cast<size_t>(kAttentionMaxHeadDim)) return report;
    AttnArgs args{};
    args.contexts = static_cast<int>(contexts);
    args.S = static_cast<int>(sequence);
    args.D = static_cast<int>(head_dim);
    args.q_tiles = static_cast<int>((sequence + kBQ - 1) / kBQ);
    args.swizzle = (contexts % 8 == 0) ? 1 : 0;
    args.key_splits = 1;
    args.keys_per_split = args.S;
    const bool vec = head_dim % 4 == 0;
    const bool fits_buffer = sequence * head_dim * sizeof(float) < (1ull << 31);
    report.key_splits = 1;
    report.keys_per_split = args.S;
    if (!biased && vec && fits_buffer && head_dim <= 128 && sequence <= 64 && contexts >= 256) {
        report.kernel = ST_HIP_ATTN_KERNEL_TINY;  // a wavefront per context, four (or two) contexts a workgroup
        report.workgroups = (contexts + 3) / 4;
        report.items = report.items_expected = contexts;
        return report;
    }
    const bool fast = vec && fits_buffer && (biased ? head_dim <= 64 && sequence % 4 == 0 : head_dim <= 128);
    if (!fast) {
        report.kernel = ST_HIP_ATTN_KERNEL_GENERAL;  // one workgroup per (context, query tile), decoded by division
        report.workgroups = contexts * static_cast<size_t>(args.q_tiles);
        report.items = report.items_expected = report.workgroups;
        return report;
    }
    report.kernel = biased ? ST_HIP_ATTN_KERNEL_FAST_BIASED : ST_HIP_ATTN_KERNEL_FAST;
    int causal_r = 0;
    const size_t blocks = plan_fast(args, causal, &causal_r);
    report.workgroups = blocks;
    report.key_splits = args.key_splits;
    report.keys_per_split = args.keys_per_split;
    report.consistent = fast_plan_consistent(args, causal, blocks) ? 1 : 0;
    const size_t tiles = static_cast<size_t>(args.q_tiles), splits = static_cast<size_t>(args.key_splits);
    if (causal && args.key_splits > 1) {
        for (size_t j = 0; j < tiles; ++j) report.items_expected += contexts * (j / static_cast<size_t>(causal_r) + 1);
    } else if (causal) {
        report.items_expected = contexts * tiles;
    } else {
        report.items_expected = contexts * tiles * splits;
    }
    if (blocks > (1ull << 26)) return report;  // the walk below is for tests; launches are covered by `consistent`
    std::vector<unsigned char> seen(contexts * tiles * splits, 0);
    auto mark = [&](int ctx, int tile, int split) {
        unsigned char &cell = seen[(static_cast<size_t>(ctx) * tiles + tile) * splits + split];
        if (cell) ++report.duplicates; else ++report.items;
        cell = 1;
    };
    for (size_t block = 0; block < blocks; ++block) {
        if (!fast_block_in_range(args, causal, block)) {
            ++report.out_of_range;
            continue;
        }
        const FastItem item = causal ? decode_fast_block<true>(args.contexts, args.q_tiles, args.swizzle, args.key_splits,
                                                               args.keys_per_split, args.causal_items, static_cast<int>(block))
                                     : decode_fast_block<false>(args.contexts, args.q_tiles, args.swizzle, args.key_splits,
                                                                args.keys_per_split, args.causal_items, static_cast<int>(block));
        if (item.split_tile >= 0) {
            mark(item.ctx, item.split_tile, item.split);
        } else if (causal) {
            mark(item.ctx, args.q_tiles - 1 - item.unit, 0);
            if (item.unit != args.q_tiles - 1 - item.unit) mark(item.ctx, item.unit, 0);
        } else {
            mark(item.ctx, item.unit, item.split);
        }
    }
    return report;
}

hipError_t launch_attention_f32(size_t contexts, size_t sequence, size_t head_dim, float scale, bool causal,
                                const float *q, const float *k, const float *v, const float *z_bias,
                                const float *attn_bias, float *out, hipStream_t stream)
{
    if (contexts == 0 || sequence == 0 || head_dim == 0) return hipSuccess;
    if (head_dim > static_cast<size_t>(kAttentionMaxHeadDim)) return hipErrorInvalidValue;
    AttnArgs args;
    args.q = q;
    args.k = k;
    args.v = v;
    args.z_bias = z_bias;
    args.attn_bias = attn_bias;
    args.out = out;
    args.contexts = static_cast<int>(contexts);
    args.S = static_cast<int>(sequence);
    args.D = static_cast<int>(head_dim);
    args.q_tiles = static_cast<int>((sequence + kBQ - 1) / kBQ);
    const size_t blocks = contexts * static_cast<size_t>(args.q_tiles);
    if (blocks > 0x7fffffffu) return hipErrorInvalidConfiguration;
    args.swizzle = (contexts % 8 == 0) ? 1 : 0;  // each XCD gets whole contexts
    args.scale = scale;
    args.key_splits = 1;
    args.keys_per_split = args.S;
    args.causal_items = 0;
    args.part_o = args.part_ml = nullptr;
    const bool bias = z_bias != nullptr || attn_bias != nullptr;
    auto aligned = [](const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; };
    const bool vec = (head_dim % 4 == 0) && aligned(q) && aligned(k) && aligned(v) && aligned(out);
    // The fast kernel addresses one context through a 32-bit buffer range.
    const bool fits_buffer = sequence * head_dim * sizeof(float) < (1ull << 31);
    // Many contexts of at most 64 positions: a wavefront per context.
    if (!bias && vec && fits_buffer && head_dim <= 128 && sequence <= 64 && contexts >= 256) {
        if (head_dim <= 32) return causal ? launch_tiny<32, true>(args, stream) : launch_tiny<32, false>(args, stream);
        if (head_dim <= 64) return causal ? launch_tiny<64, true>(args, stream) : launch_tiny<64, false>(args, stream);
        return causal ? launch_tiny<128, true>(args, stream) : launch_tiny<128, false>(args, stream);
    }
    if (!bias && vec && fits_buffer && head_dim <= 128) {
        if (head_dim <= 32) return causal ? launch_fast<32, true>(args, stream) : launch_fast<32, false>(args, stream);
        if (head_dim <= 64) return causal ? launch_fast<64, true>(args, stream) : launch_fast<64, false>(args, stream);
        return causal ? launch_fast<128, true>(args, stream) : launch_fast<128, false>(args, stream);
    }
    // The same kernel with the additive biases folded in, where their rows can be read 128 bits at a time.
    const bool bias_vec = sequence % 4 == 0 && aligned(z_bias) && aligned(attn_bias);
    if (bias && bias_vec && vec && fits_buffer && head_dim <= 64) {
        if (head_dim <= 32) return causal ? launch_fast<32, true, true>(args, stream) : launch_fast<32, false, true>(args, stream);
        return causal ? launch_fast<64, true, true>(args, stream) : launch_fast<64, false, true>(args, stream);
    }
    if (head_dim <= 32) return launch_dpad<32, 64>(args, causal, bias, vec, stream);
    if (head_dim <= 64) return launch_dpad<64, 64>(args, causal, bias, vec, stream);
    if (head_dim <= 128) return launch_dpad<128, 64>(args, causal, bias, vec, stream);
    return launch_dpad<256, 32>(args, causal, bias, vec, stream);
}

}  // namespace sthip
