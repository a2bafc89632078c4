// Byte-level pre-LayerNorm decoder forward, composed on the device from the library's own operators.
// Block order follows crates/st-vision/src/models/vit.rs:256-265
// (h = x + Attn(LN1(x)); y = h + FC2(GELU(FC1(LN2(h))))), linear layers follow
// crates/st-nn/src/layers/linear.rs:49-64,96-104 (W is (in, out), y = x·W + b).
// Every GEMM takes bf16 operands (weights rounded once at creation, activations rounded by the
// producing kernel) and accumulates in f32 — including the two matrix products inside the attention,
// whose q, k, v are the bf16 output of the fused projection; layer-norm, softmax, bias, residual and
// GELU run in f32.
#include <new>
#include <vector>

#include "kernels.h"

namespace sthip {

namespace {

struct LayerWeights {
    float *ln1_g, *ln1_b, *b_qkv, *b_o, *ln2_g, *ln2_b, *b_fc1, *b_fc2;
    uint16_t *w_qkv, *w_o, *w_fc1, *w_fc2;
};

struct Decoder {
    st_hip_decoder_config cfg;
    std::vector<void *> allocations;
    float *embed = nullptr;
    std::vector<LayerWeights> layers;
    float *lnf_g = nullptr, *lnf_b = nullptr, *b_head = nullptr;
    uint16_t *w_head = nullptr;
    // activations
    float *x = nullptr, *x2 = nullptr, *qkv = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *ctx = nullptr;
    uint16_t *h16 = nullptr, *attn16 = nullptr, *u16 = nullptr, *qkv16 = nullptr;
    bool fused_attention = false;  // bf16 attention straight from the fused [Q | K | V] projection

    ~Decoder()
    {
        (void)hipDeviceSynchronize();
        for (void *ptr : allocations) (void)hipFree(ptr);
    }
    template <typename T>
    int alloc(T **out, size_t count)
    {
        void *ptr = nullptr;
        ST_HIP_TRY(hipMalloc(&ptr, (count ? count : 1) * sizeof(T)), "hipMalloc");
        allocations.push_back(ptr);
        *out = static_cast<T *>(ptr);
        return ST_HIP_OK;
    }
};

size_t per_layer_count(const st_hip_decoder_config &c)
{
    const size_t d = c.d_model, ff = c.d_ff;
    return 2 * d + d * 3 * d + 3 * d + d * d + d + 2 * d + d * ff + ff + ff * d + d;
}

int validate_config(const st_hip_decoder_config *c)
{
    if (!c) return fail(ST_HIP_ERR_INVALID, "decoder config is null");
    if (c->vocab == 0 || c->d_model == 0 || c->heads == 0 || c->d_ff == 0 || c->batch == 0 || c->seq == 0)
        return fail(ST_HIP_ERR_INVALID, "decoder dimensions must be positive");
    if (c->d_model % c->heads != 0)
        return fail(ST_HIP_ERR_INVALID, "decoder d_model %zu is not divisible by heads %zu", c->d_model, c->heads);
    if (c->d_model / c->heads > static_cast<size_t>(kAttentionMaxHeadDim))
        return fail(ST_HIP_ERR_UNSUPPORTED, "decoder head_dim exceeds the attention kernel limit %d",
                    kAttentionMaxHeadDim);
    const size_t tokens = c->batch * c->seq;
    const size_t widest = c->d_ff > 3 * c->d_model ? c->d_ff : 3 * c->d_model;
    if (tokens > kMaxDim || widest > kMaxDim || tokens * widest > kMaxDim || c->vocab > kMaxDim)
        return fail(ST_HIP_ERR_UNSUPPORTED, "decoder activation volume exceeds i32");
    if (!std::isfinite(c->ln_eps) || c->ln_eps < 0.0f) return fail(ST_HIP_ERR_INVALID, "decoder ln_eps must be finite");
    return ST_HIP_OK;
}

}  // namespace
}  // namespace sthip

using namespace sthip;

extern "C" {

size_t st_hip_decoder_weight_count(const st_hip_decoder_config *c)
{
    if (!c) return 0;
    return c->vocab * c->d_model + c->layers * per_layer_count(*c) + 2 * c->d_model + c->d_model * c->vocab + c->vocab;
}

int st_hip_decoder_create(const st_hip_decoder_config *config, const float *host_weights, size_t weight_len,
                          void **decoder)
{
    ST_HIP_CHECK(ensure_init());
    if (!decoder) return fail(ST_HIP_ERR_INVALID, "decoder out-pointer is null");
    *decoder = nullptr;
    ST_HIP_CHECK(validate_config(config));
    const size_t expected = st_hip_decoder_weight_count(config);
    if (weight_len != expected)
        return fail(ST_HIP_ERR_INVALID, "weight buffer length %zu does not match the configuration's %zu", weight_len,
                    expected);
    if (!host_weights) return fail(ST_HIP_ERR_INVALID, "decoder weights pointer is null");

    Decoder *dec = new (std::nothrow) Decoder();
    if (!dec) return fail(ST_HIP_ERR_RUNTIME, "out of host memory");
    dec->cfg = *config;
    const size_t d = config->d_model, ff = config->d_ff, vocab = config->vocab;
    const size_t tokens = config->batch * config->seq;

    // Stage the whole blob on the device once; f32 parameters are sliced out of it, GEMM weights are
    // rounded to bf16 into their own buffers.
    float *blob = nullptr;
    int status = dec->alloc(&blob, weight_len);
    if (status == ST_HIP_OK) {
        hipError_t rc = hipMemcpy(blob, host_weights, weight_len * sizeof(float), hipMemcpyHostToDevice);
        if (rc != hipSuccess) status = hip_fail(rc, "hipMemcpy(H2D)");
    }
    // GEMM weights: (in, out) f32 -> bf16 -> packed (out, in), the layout in which neither GEMM operand needs
    // transposing on its way to the matrix cores (PackedB, crates/st-tensor/src/pure.rs:1285-1323; the reference's
    // Linear packs its weight once per parameter the same way, crates/st-nn/src/module.rs:674).
    std::vector<void *> staging;
    auto to_bf16 = [&](uint16_t **dst, const float *src, size_t in, size_t out) {
        if (status != ST_HIP_OK) return;
        status = dec->alloc(dst, in * out);
        if (status != ST_HIP_OK) return;
        void *rounded = nullptr;
        hipError_t rc = hipMalloc(&rounded, (in * out ? in * out : 1) * sizeof(uint16_t));
        if (rc != hipSuccess) { status = hip_fail(rc, "hipMalloc"); return; }
        staging.push_back(rounded);
        rc = launch_f32_to_bf16(in * out, src, static_cast<uint16_t *>(rounded), nullptr);
        if (rc == hipSuccess) rc = launch_transpose_u16(in, out, static_cast<const uint16_t *>(rounded), *dst, nullptr);
        if (rc != hipSuccess) status = hip_fail(rc, "weight packing launch");
    };
    float *p = blob;
    dec->embed = p; p += vocab * d;
    dec->layers.resize(config->layers);
    for (size_t l = 0; l < config->layers && status == ST_HIP_OK; ++l) {
        LayerWeights &w = dec->layers[l];
        w.ln1_g = p; p += d;
        w.ln1_b = p; p += d;
        to_bf16(&w.w_qkv, p, d, 3 * d); p += d * 3 * d;
        w.b_qkv = p; p += 3 * d;
        to_bf16(&w.w_o, p, d, d); p += d * d;
        w.b_o = p; p += d;
        w.ln2_g = p; p += d;
        w.ln2_b = p; p += d;
        to_bf16(&w.w_fc1, p, d, ff); p += d * ff;
        w.b_fc1 = p; p += ff;
        to_bf16(&w.w_fc2, p, ff, d); p += ff * d;
        w.b_fc2 = p; p += d;
    }
    dec->lnf_g = p; p += d;
    dec->lnf_b = p; p += d;
    to_bf16(&dec->w_head, p, d, vocab); p += d * vocab;
    dec->b_head = p;

    if (status == ST_HIP_OK) status = dec->alloc(&dec->x, tokens * d);
    if (status == ST_HIP_OK) status = dec->alloc(&dec->x2, tokens * d);
    const size_t head_dim = d / config->heads;
    dec->fused_attention = (head_dim == 64 || head_dim == 128) && ((config->seq - 1) * 3 * d + head_dim) * 2 < (1ull << 31);
    if (dec->fused_attention) {
        if (status == ST_HIP_OK) status = dec->alloc(&dec->qkv16, tokens * 3 * d);
    } else {
        if (status == ST_HIP_OK) status = dec->alloc(&dec->qkv, tokens * 3 * d);
        if (status == ST_HIP_OK) status = dec->alloc(&dec->q, tokens * d);
        if (status == ST_HIP_OK) status = dec->alloc(&dec->k, tokens * d);
        if (status == ST_HIP_OK) status = dec->alloc(&dec->v, tokens * d);
        if (status == ST_HIP_OK) status = dec->alloc(&dec->ctx, tokens * d);
    }
    if (status == ST_HIP_OK) status = dec->alloc(&dec->h16, tokens * d);
    if (status == ST_HIP_OK) status = dec->alloc(&dec->attn16, tokens * d);
    if (status == ST_HIP_OK) status = dec->alloc(&dec->u16, tokens * ff);
    {
        hipError_t rc = hipDeviceSynchronize();
        if (rc != hipSuccess && status == ST_HIP_OK) status = hip_fail(rc, "hipDeviceSynchronize");
        for (void *ptr : staging) (void)hipFree(ptr);
    }
    if (status != ST_HIP_OK) {
        delete dec;
        return status;
    }
    *decoder = dec;
    return ST_HIP_OK;
}

int st_hip_decoder_forward_dev(void *decoder, const float *tokens, float *logits, void *stream_handle)
{
    if (!decoder || !tokens || !logits) return fail(ST_HIP_ERR_INVALID, "decoder forward received a null pointer");
    Decoder &dec = *static_cast<Decoder *>(decoder);
    const st_hip_decoder_config &c = dec.cfg;
    hipStream_t stream = as_stream(stream_handle);
    const size_t d = c.d_model, ff = c.d_ff, heads = c.heads, hd = d / heads;
    const size_t T = c.batch * c.seq;
    const float scale = 1.0f / sqrtf(static_cast<float>(hd));

#define ST_LAUNCH(call, ctx)                                  \
    do {                                                      \
        hipError_t st_launch_rc_ = (call);                    \
        if (st_launch_rc_ != hipSuccess) return hip_fail(st_launch_rc_, ctx); \
    } while (0)

    // The lookup and the layer norm that reads it (the first layer's, or the final one of a stack without layers) are
    // one launch: the embedded rows go to the residual stream and, normalised, to the first GEMM's operand.
    const float *first_gamma = dec.layers.empty() ? dec.lnf_g : dec.layers.front().ln1_g;
    const float *first_beta = dec.layers.empty() ? dec.lnf_b : dec.layers.front().ln1_b;
    ST_LAUNCH(launch_embedding_layer_norm_f32(T, c.vocab, d, tokens, dec.embed, dec.x, first_gamma, first_beta, c.ln_eps,
                                              dec.h16, stream),
              "embedding + layer_norm launch");
    for (const LayerWeights &w : dec.layers) {
        GemmEpilogue ep;
        if (&w != &dec.layers.front())
            ST_LAUNCH(launch_layer_norm_f32(T, d, dec.x, nullptr, w.ln1_g, w.ln1_b, c.ln_eps, nullptr, dec.h16, stream),
                      "layer_norm launch");
        ep = GemmEpilogue();
        ep.bias = w.b_qkv;
        if (dec.fused_attention) {
            // q, k, v leave the projection as bf16 and are consumed in place, head by head.
            ST_LAUNCH(launch_gemm_bf16(T, 3 * d, d, dec.h16, w.w_qkv, nullptr, dec.qkv16, ep, stream, true), "qkv gemm launch");
            ST_LAUNCH(launch_attention_bf16(c.batch, heads, c.seq, hd, scale, true, dec.qkv16, dec.qkv16 + d,
                                            dec.qkv16 + 2 * d, 3 * d, dec.attn16, d, stream),
                      "attention launch");
        } else {
            // Head sizes the bf16 kernel does not cover: same rounding points (q, k, v rounded to bf16,
            // attention output rounded to bf16), carried out by the f32 attention kernel.
            ST_LAUNCH(launch_gemm_bf16(T, 3 * d, d, dec.h16, w.w_qkv, dec.qkv, nullptr, ep, stream, true), "qkv gemm launch");
            ST_LAUNCH(launch_split_heads_f32(c.batch, c.seq, heads, hd, dec.qkv, dec.q, dec.k, dec.v, true, stream),
                      "split_heads launch");
            ST_LAUNCH(launch_attention_f32(c.batch * heads, c.seq, hd, scale, true, dec.q, dec.k, dec.v, nullptr,
                                           nullptr, dec.ctx, stream),
                      "attention launch");
            ST_LAUNCH(launch_merge_heads_f32(c.batch, c.seq, heads, hd, dec.ctx, nullptr, dec.attn16, stream),
                      "merge_heads launch");
        }
        ep = GemmEpilogue();
        ep.bias = w.b_o;
        ep.residual = dec.x;
        ST_LAUNCH(launch_gemm_bf16(T, d, d, dec.attn16, w.w_o, dec.x2, nullptr, ep, stream, true), "out-proj gemm launch");
        ST_LAUNCH(launch_layer_norm_f32(T, d, dec.x2, nullptr, w.ln2_g, w.ln2_b, c.ln_eps, nullptr, dec.h16, stream),
                  "layer_norm launch");
        ep = GemmEpilogue();
        ep.bias = w.b_fc1;
        ep.activation = ST_HIP_ACT_GELU;
        ST_LAUNCH(launch_gemm_bf16(T, ff, d, dec.h16, w.w_fc1, nullptr, dec.u16, ep, stream, true), "fc1 gemm launch");
        ep = GemmEpilogue();
        ep.bias = w.b_fc2;
        ep.residual = dec.x2;
        ST_LAUNCH(launch_gemm_bf16(T, d, ff, dec.u16, w.w_fc2, dec.x, nullptr, ep, stream, true), "fc2 gemm launch");
    }
    if (!dec.layers.empty())
        ST_LAUNCH(launch_layer_norm_f32(T, d, dec.x, nullptr, dec.lnf_g, dec.lnf_b, c.ln_eps, nullptr, dec.h16, stream),
                  "layer_norm launch");
    GemmEpilogue head;
    head.bias = dec.b_head;
    ST_LAUNCH(launch_gemm_bf16(T, c.vocab, d, dec.h16, dec.w_head, logits, nullptr, head, stream, true), "head gemm launch");
#undef ST_LAUNCH
    return ST_HIP_OK;
}

int st_hip_decoder_destroy(void *decoder)
{
    delete static_cast<Decoder *>(decoder);
    return ST_HIP_OK;
}

}  // extern "C"
