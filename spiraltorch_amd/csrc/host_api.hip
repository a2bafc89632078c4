// Operator half of the C ABI: the host-slice (drop-in) entry points with the reference's validation
// order and error texts, and the device-resident entry points the benchmarks and the decoder use.
//
// Host-slice calls mirror crates/st-backend-hip/src/real.rs:699-757,817-957: copy operands to the
// device, run on a private stream, copy the result back, and never release a device buffer before the
// stream has drained — also on error paths (StreamCompletionGuard, real.rs:669-697).  Instead of the
// reference's per-call hipMalloc/hipStreamCreate, buffers and streams come from a pool of workspaces;
// a workspace is used by one call at a time, so concurrent callers never share device memory.
#include <cmath>
#include <cstring>
#include <mutex>
#include <vector>

#include "kernels.h"

namespace sthip {

namespace {

constexpr int kWorkspaceBuffers = 6;

struct Workspace {
    hipStream_t stream = nullptr;
    void *buffers[kWorkspaceBuffers] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    size_t capacity[kWorkspaceBuffers] = {0, 0, 0, 0, 0, 0};
};

class WorkspacePool {
  public:
    Workspace *acquire(int *status)
    {
        {
            std::lock_guard<std::mutex> lock(mutex_);
            if (!idle_.empty()) {
                Workspace *ws = idle_.back();
                idle_.pop_back();
                *status = ST_HIP_OK;
                return ws;
            }
        }
        Workspace *ws = new Workspace();
        hipError_t rc = hipStreamCreate(&ws->stream);
        if (rc != hipSuccess) {
            delete ws;
            *status = hip_fail(rc, "hipStreamCreate");
            return nullptr;
        }
        *status = ST_HIP_OK;
        return ws;
    }
    void release(Workspace *ws)
    {
        std::lock_guard<std::mutex> lock(mutex_);
        idle_.push_back(ws);
    }

  private:
    std::mutex mutex_;
    std::vector<Workspace *> idle_;
};

WorkspacePool &pool()
{
    static WorkspacePool instance;
    return instance;
}

// Holds a workspace for one host-slice call; the destructor drains the stream before the workspace
// (and with it the device buffers) can be handed to another caller.
class Lease {
  public:
    Lease() { ws_ = pool().acquire(&status_); }
    ~Lease()
    {
        if (ws_) {
            (void)hipStreamSynchronize(ws_->stream);
            pool().release(ws_);
        }
    }
    Lease(const Lease &) = delete;
    Lease &operator=(const Lease &) = delete;
    int status() const { return status_; }
    hipStream_t stream() const { return ws_->stream; }
    // Device buffer `slot`, grown to at least `bytes`.
    int buffer(int slot, size_t bytes, void **out)
    {
        if (ws_->capacity[slot] < bytes || ws_->buffers[slot] == nullptr) {
            ST_HIP_TRY(hipStreamSynchronize(ws_->stream), "hipStreamSynchronize");
            if (ws_->buffers[slot]) {
                ST_HIP_TRY(hipFree(ws_->buffers[slot]), "hipFree");
                ws_->buffers[slot] = nullptr;
                ws_->capacity[slot] = 0;
            }
            const size_t rounded = ((bytes ? bytes : 1) + 255) & ~static_cast<size_t>(255);
            ST_HIP_TRY(hipMalloc(&ws_->buffers[slot], rounded), "hipMalloc");
            ws_->capacity[slot] = rounded;
        }
        *out = ws_->buffers[slot];
        return ST_HIP_OK;
    }
    int upload(int slot, const void *host, size_t bytes, void **device)
    {
        ST_HIP_CHECK(buffer(slot, bytes, device));
        if (bytes) {
            count_transfer(true, bytes);
            ST_HIP_TRY(hipMemcpyAsync(*device, host, bytes, hipMemcpyHostToDevice, ws_->stream),
                       "hipMemcpyAsync(H2D)");
        }
        return ST_HIP_OK;
    }
    int download(void *host, const void *device, size_t bytes)
    {
        if (bytes) {
            count_transfer(false, bytes);
            ST_HIP_TRY(hipMemcpyAsync(host, device, bytes, hipMemcpyDeviceToHost, ws_->stream),
                       "hipMemcpyAsync(D2H)");
        }
        ST_HIP_TRY(hipStreamSynchronize(ws_->stream), "hipStreamSynchronize");
        return ST_HIP_OK;
    }

  private:
    Workspace *ws_ = nullptr;
    int status_ = ST_HIP_OK;
};

// ---- validators (crates/st-backend-hip/src/lib.rs:446-523) -----------------------------------

int validate_gemm_dimensions(size_t m, size_t n, size_t k, size_t lhs_len, size_t rhs_len, size_t out_len)
{
    size_t expected_lhs, expected_rhs, expected_out;
    if (!checked_mul(m, k, &expected_lhs))
        return fail(ST_HIP_ERR_INVALID, "gemm dimensions overflow while validating lhs");
    if (!checked_mul(k, n, &expected_rhs))
        return fail(ST_HIP_ERR_INVALID, "gemm dimensions overflow while validating rhs");
    if (!checked_mul(m, n, &expected_out))
        return fail(ST_HIP_ERR_INVALID, "gemm dimensions overflow while validating output");
    if (lhs_len != expected_lhs)
        return fail(ST_HIP_ERR_INVALID, "lhs buffer length %zu does not match m*k=%zu", lhs_len, expected_lhs);
    if (rhs_len != expected_rhs)
        return fail(ST_HIP_ERR_INVALID, "rhs buffer length %zu does not match k*n=%zu", rhs_len, expected_rhs);
    if (out_len != expected_out)
        return fail(ST_HIP_ERR_INVALID, "output buffer length %zu does not match m*n=%zu", out_len, expected_out);
    return ST_HIP_OK;
}

int validate_gemm_scale(float scale)
{
    if (std::isfinite(scale)) return ST_HIP_OK;
    // Rust prints non-finite f32 as "inf", "-inf" or "NaN".
    const char *text = std::isnan(scale) ? "NaN" : (scale > 0 ? "inf" : "-inf");
    return fail(ST_HIP_ERR_INVALID, "gemm scale must be finite, received %s", text);
}

int validate_gemm_epilogue(size_t m, size_t n, size_t bias_len, bool has_residual, size_t residual_len)
{
    if (bias_len != n) return fail(ST_HIP_ERR_INVALID, "bias buffer length %zu does not match n=%zu", bias_len, n);
    if (has_residual) {
        size_t expected;
        if (!checked_mul(m, n, &expected))
            return fail(ST_HIP_ERR_INVALID, "gemm dimensions overflow while validating residual");
        if (residual_len != expected)
            return fail(ST_HIP_ERR_INVALID, "residual buffer length %zu does not match m*n=%zu", residual_len,
                        expected);
    }
    return ST_HIP_OK;
}

// Dimensions must fit i32 at the kernel boundary (real.rs:605-610, hip_dense.rs:55-73).
int validate_kernel_dims(size_t m, size_t n, size_t k)
{
    if (m > kMaxDim) return fail(ST_HIP_ERR_UNSUPPORTED, "gemm m dimension overflow (exceeds i32)");
    if (n > kMaxDim) return fail(ST_HIP_ERR_UNSUPPORTED, "gemm n dimension overflow (exceeds i32)");
    if (k > kMaxDim) return fail(ST_HIP_ERR_UNSUPPORTED, "gemm k dimension overflow (exceeds i32)");
    return ST_HIP_OK;
}

int validate_activation(int activation, bool allow_none)
{
    if (activation == ST_HIP_ACT_RELU || activation == ST_HIP_ACT_GELU) return ST_HIP_OK;
    if (allow_none && activation == ST_HIP_ACT_NONE) return ST_HIP_OK;
    return fail(ST_HIP_ERR_INVALID, "unknown activation code %d", activation);
}

int reject_null(const void *ptr, size_t len, const char *what)
{
    if (ptr == nullptr && len != 0)
        return fail(ST_HIP_ERR_INVALID, "%s received a null pointer; provide contiguous row-major buffers", what);
    return ST_HIP_OK;
}

int launch_status(hipError_t rc, const char *ctx)
{
    if (rc != hipSuccess) return hip_fail(rc, ctx);
    return ST_HIP_OK;
}

// First non-finite value of a host slice, reported like TensorError::NonFiniteValue
// (crates/st-tensor/src/pure.rs:5521-5533).
int validate_finite_slice(const char *label, const float *values, size_t len)
{
    for (size_t i = 0; i < len; ++i) {
        if (!std::isfinite(values[i]))
            return fail(ST_HIP_ERR_NONFINITE, "non-finite value encountered in %s: %g", label,
                        static_cast<double>(values[i]));
    }
    return ST_HIP_OK;
}

struct ConvPlan {
    ConvShape shape;
    size_t input_len, weight_len, out_len;
};

int plan_conv(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out, size_t kh, size_t kw,
              size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
              ConvPlan *plan)
{
    // validate_positive(...) of Conv2d::new, crates/st-nn/src/layers/conv.rs:631-640.
    const struct { size_t value; const char *name; } positives[] = {
        {c_in, "in_channels"}, {c_out, "out_channels"}, {kh, "kernel_h"}, {kw, "kernel_w"},
        {stride_h, "stride_h"}, {stride_w, "stride_w"}, {dil_h, "dilation_h"}, {dil_w, "dilation_w"},
        {h, "input_height"}, {w, "input_width"}};
    for (const auto &item : positives)
        if (item.value == 0) return fail(ST_HIP_ERR_INVALID, "conv2d %s must be positive", item.name);
    size_t oh, ow;
    ST_HIP_CHECK(st_hip_conv2d_output_hw(h, w, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, &oh, &ow));
    const size_t values[] = {batch, c_in, h, w, c_out, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, oh, ow};
    for (size_t v : values)
        if (v > kMaxDim) return fail(ST_HIP_ERR_UNSUPPORTED, "conv2d dimension exceeds i32");
    size_t chw, span, spatial, ochw;
    if (!checked_mul(c_in, h, &chw) || !checked_mul(chw, w, &chw) || !checked_mul(batch, chw, &plan->input_len) ||
        !checked_mul(c_in, kh, &span) || !checked_mul(span, kw, &span) || !checked_mul(c_out, span, &plan->weight_len) ||
        !checked_mul(oh, ow, &spatial) || !checked_mul(c_out, spatial, &ochw) ||
        !checked_mul(batch, ochw, &plan->out_len))
        return fail(ST_HIP_ERR_INVALID, "conv2d dimensions overflow");
    if (chw > kMaxDim || ochw > kMaxDim || span > kMaxDim)
        return fail(ST_HIP_ERR_UNSUPPORTED, "conv2d per-image extent exceeds i32");
    ConvShape &s = plan->shape;
    s.batch = static_cast<int>(batch); s.c_in = static_cast<int>(c_in); s.h = static_cast<int>(h);
    s.w = static_cast<int>(w); s.c_out = static_cast<int>(c_out); s.kh = static_cast<int>(kh);
    s.kw = static_cast<int>(kw); s.stride_h = static_cast<int>(stride_h); s.stride_w = static_cast<int>(stride_w);
    s.pad_h = static_cast<int>(pad_h); s.pad_w = static_cast<int>(pad_w); s.dil_h = static_cast<int>(dil_h);
    s.dil_w = static_cast<int>(dil_w); s.oh = static_cast<int>(oh); s.ow = static_cast<int>(ow);
    return ST_HIP_OK;
}

// With a kernel family forced (st_hip_conv2d_force_family), a shape that family cannot serve is an error rather
// than a silent switch to another kernel.
int check_conv_family(const ConvShape &shape, int direction, const void *weight, const void *out)
{
    const bool weight_aligned = (reinterpret_cast<uintptr_t>(weight) & 15u) == 0;
    const bool out_aligned = (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    const int kernel = direction == 0 ? planned_conv_kernel(shape, weight_aligned, out_aligned)
                                      : planned_conv_grad_input_kernel(shape);
    if (kernel == 0)
        return fail(ST_HIP_ERR_UNSUPPORTED, "the forced conv2d kernel family cannot serve this shape (%s)",
                    direction == 0 ? "forward" : "grad_input");
    return ST_HIP_OK;
}

struct AttentionPlan {
    size_t rows, qkv_len, z_len, bias_len;
};

int plan_attention(size_t contexts, size_t sequence, size_t head_dim, AttentionPlan *plan)
{
    if (!checked_mul(contexts, sequence, &plan->rows))
        return fail(ST_HIP_ERR_INVALID, "attention contexts*sequence exceeds the addressable volume");
    if (!checked_mul(plan->rows, head_dim, &plan->qkv_len) || !checked_mul(plan->rows, sequence, &plan->bias_len))
        return fail(ST_HIP_ERR_INVALID, "attention dimensions overflow");
    plan->z_len = plan->rows;
    return ST_HIP_OK;
}

int check_attention_kernel_limits(size_t contexts, size_t sequence, size_t head_dim)
{
    if (contexts > kMaxDim || sequence > kMaxDim)
        return fail(ST_HIP_ERR_UNSUPPORTED, "attention contexts/sequence exceed i32");
    if (head_dim > static_cast<size_t>(kAttentionMaxHeadDim))
        return fail(ST_HIP_ERR_UNSUPPORTED, "attention head_dim %zu exceeds the kernel limit %d", head_dim,
                    kAttentionMaxHeadDim);
    return ST_HIP_OK;
}

}  // namespace
}  // namespace sthip

using namespace sthip;

extern "C" {

// ---------------------------------------------------------------------------------------------
// Host-slice forms
// ---------------------------------------------------------------------------------------------

int st_hip_gemm_f32(size_t m, size_t n, size_t k, float scale, int lhs_transposed, const float *lhs,
                    size_t lhs_len, const float *rhs, size_t rhs_len, float *out, size_t out_len)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_CHECK(validate_gemm_dimensions(m, n, k, lhs_len, rhs_len, out_len));
    ST_HIP_CHECK(validate_gemm_scale(scale));
    ST_HIP_CHECK(reject_null(lhs, lhs_len, "gemm"));
    ST_HIP_CHECK(reject_null(rhs, rhs_len, "gemm"));
    ST_HIP_CHECK(reject_null(out, out_len, "gemm"));
    if (out_len == 0) return ST_HIP_OK;
    ST_HIP_CHECK(validate_kernel_dims(m, n, k));

    Lease lease;
    ST_HIP_CHECK(lease.status());
    void *d_lhs, *d_rhs, *d_out;
    ST_HIP_CHECK(lease.upload(0, lhs, lhs_len * sizeof(float), &d_lhs));
    ST_HIP_CHECK(lease.upload(1, rhs, rhs_len * sizeof(float), &d_rhs));
    ST_HIP_CHECK(lease.buffer(2, out_len * sizeof(float), &d_out));
    GemmEpilogue epilogue;
    epilogue.scale = scale;
    ST_HIP_CHECK(launch_status(launch_gemm_f32(m, n, k, lhs_transposed != 0, static_cast<const float *>(d_lhs),
                                               static_cast<const float *>(d_rhs), static_cast<float *>(d_out),
                                               epilogue, lease.stream()),
                               "gemm_f32 launch"));
    return lease.download(out, d_out, out_len * sizeof(float));
}

int st_hip_gemm_f32_raw(size_t m, size_t n, size_t k, const float *lhs, const float *rhs, float *out)
{
    // crates/st-backend-hip/src/lib.rs:779-798: null check first, then the slice lengths, then gemm_f32.
    if (!lhs || !rhs || !out)
        return fail(ST_HIP_ERR_INVALID, "gemm received a null pointer; provide contiguous row-major buffers");
    size_t lhs_len, rhs_len, out_len;
    if (!checked_mul(m, k, &lhs_len)) return fail(ST_HIP_ERR_INVALID, "gemm dimensions overflow while constructing lhs slice");
    if (!checked_mul(k, n, &rhs_len)) return fail(ST_HIP_ERR_INVALID, "gemm dimensions overflow while constructing rhs slice");
    if (!checked_mul(m, n, &out_len)) return fail(ST_HIP_ERR_INVALID, "gemm dimensions overflow while constructing output slice");
    return st_hip_gemm_f32(m, n, k, 1.0f, 0, lhs, lhs_len, rhs, rhs_len, out, out_len);
}

int st_hip_gemm_bias_act_f32(size_t m, size_t n, size_t k, int activation, const float *lhs, size_t lhs_len,
                             const float *rhs, size_t rhs_len, const float *bias, size_t bias_len,
                             const float *residual, size_t residual_len, float *out, size_t out_len)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_CHECK(validate_gemm_dimensions(m, n, k, lhs_len, rhs_len, out_len));
    ST_HIP_CHECK(validate_gemm_epilogue(m, n, bias_len, residual != nullptr, residual_len));
    ST_HIP_CHECK(validate_activation(activation, false));
    ST_HIP_CHECK(reject_null(lhs, lhs_len, "gemm"));
    ST_HIP_CHECK(reject_null(rhs, rhs_len, "gemm"));
    ST_HIP_CHECK(reject_null(bias, bias_len, "gemm"));
    ST_HIP_CHECK(reject_null(out, out_len, "gemm"));
    if (out_len == 0) return ST_HIP_OK;  // real.rs:828-830
    ST_HIP_CHECK(validate_kernel_dims(m, n, k));

    Lease lease;
    ST_HIP_CHECK(lease.status());
    void *d_lhs, *d_rhs, *d_out, *d_bias, *d_residual = nullptr;
    ST_HIP_CHECK(lease.upload(0, lhs, lhs_len * sizeof(float), &d_lhs));
    ST_HIP_CHECK(lease.upload(1, rhs, rhs_len * sizeof(float), &d_rhs));
    ST_HIP_CHECK(lease.buffer(2, out_len * sizeof(float), &d_out));
    ST_HIP_CHECK(lease.upload(3, bias, bias_len * sizeof(float), &d_bias));
    if (residual) ST_HIP_CHECK(lease.upload(4, residual, residual_len * sizeof(float), &d_residual));
    GemmEpilogue epilogue;
    epilogue.bias = static_cast<const float *>(d_bias);
    epilogue.residual = static_cast<const float *>(d_residual);
    epilogue.activation = activation;
    ST_HIP_CHECK(launch_status(launch_gemm_f32(m, n, k, false, static_cast<const float *>(d_lhs),
                                               static_cast<const float *>(d_rhs), static_cast<float *>(d_out),
                                               epilogue, lease.stream()),
                               "gemm_bias_act_f32 launch"));
    return lease.download(out, d_out, out_len * sizeof(float));
}

int st_hip_gemm_prepacked_bias_act_f32(size_t m, size_t n, size_t k, int activation, const float *lhs, size_t lhs_len,
                                       const float *packed_rhs, size_t packed_len, const float *bias, size_t bias_len,
                                       const float *residual, size_t residual_len, float *out, size_t out_len)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_CHECK(validate_gemm_dimensions(m, n, k, lhs_len, packed_len, out_len));
    if (bias != nullptr || bias_len != 0) ST_HIP_CHECK(validate_gemm_epilogue(m, n, bias_len, false, 0));
    if (residual != nullptr) ST_HIP_CHECK(validate_gemm_epilogue(m, n, n, true, residual_len));
    ST_HIP_CHECK(validate_activation(activation, true));
    ST_HIP_CHECK(reject_null(lhs, lhs_len, "gemm"));
    ST_HIP_CHECK(reject_null(packed_rhs, packed_len, "gemm"));
    ST_HIP_CHECK(reject_null(bias, bias_len, "gemm"));
    ST_HIP_CHECK(reject_null(out, out_len, "gemm"));
    if (out_len == 0) return ST_HIP_OK;
    ST_HIP_CHECK(validate_kernel_dims(m, n, k));

    Lease lease;
    ST_HIP_CHECK(lease.status());
    void *d_lhs, *d_rhs, *d_out, *d_bias = nullptr, *d_residual = nullptr;
    ST_HIP_CHECK(lease.upload(0, lhs, lhs_len * sizeof(float), &d_lhs));
    ST_HIP_CHECK(lease.upload(1, packed_rhs, packed_len * sizeof(float), &d_rhs));
    ST_HIP_CHECK(lease.buffer(2, out_len * sizeof(float), &d_out));
    if (bias) ST_HIP_CHECK(lease.upload(3, bias, bias_len * sizeof(float), &d_bias));
    if (residual) ST_HIP_CHECK(lease.upload(4, residual, residual_len * sizeof(float), &d_residual));
    GemmEpilogue epilogue;
    epilogue.bias = static_cast<const float *>(d_bias);
    epilogue.residual = static_cast<const float *>(d_residual);
    epilogue.activation = activation;
    ST_HIP_CHECK(launch_status(launch_gemm_f32_packed(m, n, k, static_cast<const float *>(d_lhs),
                                                      static_cast<const float *>(d_rhs), static_cast<float *>(d_out),
                                                      epilogue, lease.stream()),
                               "gemm_prepacked launch"));
    return lease.download(out, d_out, out_len * sizeof(float));
}

int st_hip_gemm_bf16_f32acc(size_t m, size_t n, size_t k, const uint16_t *lhs, size_t lhs_len,
                            const uint16_t *rhs, size_t rhs_len, float *out, size_t out_len)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_CHECK(validate_gemm_dimensions(m, n, k, lhs_len, rhs_len, out_len));
    ST_HIP_CHECK(reject_null(lhs, lhs_len, "gemm"));
    ST_HIP_CHECK(reject_null(rhs, rhs_len, "gemm"));
    ST_HIP_CHECK(reject_null(out, out_len, "gemm"));
    if (out_len == 0) return ST_HIP_OK;
    ST_HIP_CHECK(validate_kernel_dims(m, n, k));

    Lease lease;
    ST_HIP_CHECK(lease.status());
    void *d_lhs, *d_rhs, *d_out;
    ST_HIP_CHECK(lease.upload(0, lhs, lhs_len * sizeof(uint16_t), &d_lhs));
    ST_HIP_CHECK(lease.upload(1, rhs, rhs_len * sizeof(uint16_t), &d_rhs));
    ST_HIP_CHECK(lease.buffer(2, out_len * sizeof(float), &d_out));
    ST_HIP_CHECK(launch_status(launch_gemm_bf16(m, n, k, static_cast<const uint16_t *>(d_lhs),
                                                static_cast<const uint16_t *>(d_rhs), static_cast<float *>(d_out),
                                                nullptr, GemmEpilogue(), lease.stream()),
                               "gemm_bf16 launch"));
    return lease.download(out, d_out, out_len * sizeof(float));
}

int st_hip_conv2d_output_hw(size_t h, size_t w, size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                            size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w, size_t *oh, size_t *ow)
{
    // crates/st-nn/src/layers/conv.rs:685-700 with dilated_extent :106-114.
    if (!oh || !ow) return fail(ST_HIP_ERR_INVALID, "conv2d output_hw received a null out-pointer");
    if (kh == 0 || kw == 0 || stride_h == 0 || stride_w == 0 || dil_h == 0 || dil_w == 0)
        return fail(ST_HIP_ERR_INVALID, "conv2d kernel, stride and dilation must be positive");
    size_t eff_kh, eff_kw, padded_h, padded_w;
    if (!checked_mul(kh - 1, dil_h, &eff_kh) || !checked_mul(kw - 1, dil_w, &eff_kw) || eff_kh + 1 < eff_kh ||
        eff_kw + 1 < eff_kw)
        return fail(ST_HIP_ERR_INVALID, "conv2d dilated kernel extent overflows");
    eff_kh += 1;
    eff_kw += 1;
    if (!checked_mul(2, pad_h, &padded_h) || !checked_mul(2, pad_w, &padded_w) || padded_h + h < h || padded_w + w < w)
        return fail(ST_HIP_ERR_INVALID, "conv2d padded extent overflows");
    padded_h += h;
    padded_w += w;
    if (padded_h < eff_kh || padded_w < eff_kw)
        return fail(ST_HIP_ERR_INVALID, "conv2d padded input (%zu, %zu) is smaller than the dilated kernel (%zu, %zu)",
                    padded_h, padded_w, eff_kh, eff_kw);
    *oh = (padded_h - eff_kh) / stride_h + 1;
    *ow = (padded_w - eff_kw) / stride_w + 1;
    return ST_HIP_OK;
}

int st_hip_conv2d_force_family(int family)
{
    if (family < ST_HIP_CONV_FAMILY_AUTO || family > ST_HIP_CONV_FAMILY_STRIP)
        return fail(ST_HIP_ERR_INVALID, "unknown conv2d kernel family %d", family);
    set_conv_forced_family(family);
    return ST_HIP_OK;
}

int st_hip_conv2d_planned_kernel(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out, size_t kh, size_t kw,
                                 size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w, size_t dil_h,
                                 size_t dil_w, int direction, int *kernel)
{
    if (!kernel) return fail(ST_HIP_ERR_INVALID, "conv2d planned_kernel received a null out-pointer");
    if (direction != 0 && direction != 1) return fail(ST_HIP_ERR_INVALID, "unknown conv2d direction %d", direction);
    ConvPlan plan;
    ST_HIP_CHECK(plan_conv(batch, c_in, h, w, c_out, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, &plan));
    *kernel = direction == 0 ? planned_conv_kernel(plan.shape, true, true) : planned_conv_grad_input_kernel(plan.shape);
    return ST_HIP_OK;
}

int st_hip_attention_f32_launch_plan(size_t contexts, size_t sequence, size_t head_dim, int causal, int biased,
                                     st_hip_attention_plan *plan)
{
    if (!plan) return fail(ST_HIP_ERR_INVALID, "attention launch_plan received a null out-pointer");
    size_t rows = 0, volume = 0;
    if (contexts > kMaxDim || sequence > kMaxDim || head_dim > kMaxDim || !checked_mul(contexts, sequence, &rows) ||
        !checked_mul(rows, head_dim, &volume))
        return fail(ST_HIP_ERR_INVALID, "attention dimensions overflow");
    if (head_dim > static_cast<size_t>(kAttentionMaxHeadDim))
        return fail(ST_HIP_ERR_UNSUPPORTED, "attention head_dim %zu exceeds %d", head_dim, kAttentionMaxHeadDim);
    const AttentionPlanReport report = attention_f32_plan_report(contexts, sequence, head_dim, causal != 0, biased != 0);
    plan->kernel = report.kernel;
    plan->key_splits = report.key_splits;
    plan->keys_per_split = report.keys_per_split;
    plan->consistent = report.kernel == ST_HIP_ATTN_KERNEL_FAST || report.kernel == ST_HIP_ATTN_KERNEL_FAST_BIASED ? report.consistent : 1;
    plan->workgroups = report.workgroups;
    plan->items = report.items;
    plan->items_expected = report.items_expected;
    plan->out_of_range = report.out_of_range;
    plan->duplicates = report.duplicates;
    return ST_HIP_OK;
}

int st_hip_probe_mfma_bf16_dev(size_t workgroups, size_t iterations, const uint16_t *operands, float *sink, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    if (!operands || !sink) return fail(ST_HIP_ERR_INVALID, "mfma probe received a null pointer");
    if ((reinterpret_cast<uintptr_t>(operands) & 15u) != 0) return fail(ST_HIP_ERR_UNSUPPORTED, "mfma probe operands must be 16-byte aligned");
    return launch_status(launch_probe_mfma_bf16(workgroups, iterations, operands, sink, as_stream(stream)), "mfma probe launch");
}

int st_hip_probe_mfma_f32_dev(size_t workgroups, size_t iterations, const float *operands, float *sink, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    if (!operands || !sink) return fail(ST_HIP_ERR_INVALID, "mfma probe received a null pointer");
    return launch_status(launch_probe_mfma_f32(workgroups, iterations, operands, sink, as_stream(stream)), "mfma probe launch");
}

int st_hip_probe_stream_lds_dev(size_t workgroups, size_t iterations, const void *region, size_t region_bytes, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    if (!region) return fail(ST_HIP_ERR_INVALID, "stream probe received a null pointer");
    if (region_bytes < 65536 || region_bytes >= (1ull << 31))
        return fail(ST_HIP_ERR_UNSUPPORTED, "stream probe takes a region of 64 KiB to below 2 GiB (received %zu bytes)", region_bytes);
    return launch_status(launch_probe_stream_lds(workgroups, iterations, region, region_bytes, as_stream(stream)), "stream probe launch");
}

int st_hip_gemm_bf16_tile_plan(size_t m, size_t n, size_t k, st_hip_gemm_tile_plan *plan)
{
    if (!plan) return fail(ST_HIP_ERR_INVALID, "gemm tile_plan received a null out-pointer");
    if (m > kMaxDim || n > kMaxDim || k > kMaxDim) return fail(ST_HIP_ERR_INVALID, "gemm dimensions exceed i32");
    if (m == 0 || n == 0 || k < 64 || k % 64 != 0)
        return fail(ST_HIP_ERR_UNSUPPORTED, "the 256-row kernels take k a positive multiple of 64 (received %zu)", k);
    const GemmTilePlanReport report = gemm_bf16_tile_plan_report(m, n, k);
    plan->tile_cols = report.tile_cols;
    plan->tiles_m = report.tiles_m;
    plan->tiles_n = report.tiles_n;
    plan->k_splits = report.k_splits;
    plan->k_tiles_per_split = report.k_tiles_per_split;
    plan->consistent = report.consistent;
    plan->workgroups = report.workgroups;
    plan->items = report.items;
    plan->out_of_range = report.out_of_range;
    plan->duplicates = report.duplicates;
    return ST_HIP_OK;
}

size_t st_hip_gemm_row_block(size_t k, size_t element_bytes)
{
    size_t row_bytes = 0;
    if (!checked_mul(k, element_bytes, &row_bytes)) return 0;
    return gemm_row_block(k, element_bytes);
}

int st_hip_conv2d_bias_act_f32(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out, size_t kh, size_t kw,
                               size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w, size_t dil_h,
                               size_t dil_w, int activation, const float *input, size_t input_len,
                               const float *weight, size_t weight_len, const float *bias, size_t bias_len,
                               float *out, size_t out_len)
{
    ST_HIP_CHECK(ensure_init());
    ConvPlan plan;
    ST_HIP_CHECK(plan_conv(batch, c_in, h, w, c_out, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, &plan));
    ST_HIP_CHECK(validate_activation(activation, true));
    if (input_len != plan.input_len)
        return fail(ST_HIP_ERR_INVALID, "input buffer length %zu does not match batch*c_in*h*w=%zu", input_len,
                    plan.input_len);
    if (weight_len != plan.weight_len)
        return fail(ST_HIP_ERR_INVALID, "weight buffer length %zu does not match c_out*c_in*kh*kw=%zu", weight_len,
                    plan.weight_len);
    if (bias != nullptr && bias_len != c_out)
        return fail(ST_HIP_ERR_INVALID, "bias buffer length %zu does not match c_out=%zu", bias_len, c_out);
    if (out_len != plan.out_len)
        return fail(ST_HIP_ERR_INVALID, "output buffer length %zu does not match batch*c_out*oh*ow=%zu", out_len,
                    plan.out_len);
    ST_HIP_CHECK(reject_null(input, input_len, "conv2d"));
    ST_HIP_CHECK(reject_null(weight, weight_len, "conv2d"));
    ST_HIP_CHECK(reject_null(out, out_len, "conv2d"));
    if (out_len == 0) return ST_HIP_OK;  // empty batch: conv.rs:4132-4137

    Lease lease;
    ST_HIP_CHECK(lease.status());
    void *d_in, *d_w, *d_out, *d_bias = nullptr;
    ST_HIP_CHECK(lease.upload(0, input, input_len * sizeof(float), &d_in));
    ST_HIP_CHECK(lease.upload(1, weight, weight_len * sizeof(float), &d_w));
    ST_HIP_CHECK(lease.buffer(2, out_len * sizeof(float), &d_out));
    if (bias) ST_HIP_CHECK(lease.upload(3, bias, bias_len * sizeof(float), &d_bias));
    ST_HIP_CHECK(check_conv_family(plan.shape, 0, d_w, d_out));
    ST_HIP_CHECK(launch_status(launch_conv2d_f32(plan.shape, activation, static_cast<const float *>(d_in),
                                                 static_cast<const float *>(d_w), static_cast<const float *>(d_bias),
                                                 static_cast<float *>(d_out), lease.stream()),
                               "conv2d launch"));
    return lease.download(out, d_out, out_len * sizeof(float));
}

int st_hip_conv2d_backward_f32(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out, size_t kh, size_t kw,
                               size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w, size_t dil_h, size_t dil_w,
                               const float *input, size_t input_len, const float *weight, size_t weight_len,
                               const float *grad_output, size_t grad_output_len, float *grad_input, size_t grad_input_len,
                               float *grad_weight, size_t grad_weight_len, float *grad_bias, size_t grad_bias_len)
{
    ST_HIP_CHECK(ensure_init());
    ConvPlan plan;
    ST_HIP_CHECK(plan_conv(batch, c_in, h, w, c_out, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, &plan));
    if (input_len != plan.input_len)
        return fail(ST_HIP_ERR_INVALID, "input buffer length %zu does not match batch*c_in*h*w=%zu", input_len, plan.input_len);
    if (weight_len != plan.weight_len)
        return fail(ST_HIP_ERR_INVALID, "weight buffer length %zu does not match c_out*c_in*kh*kw=%zu", weight_len,
                    plan.weight_len);
    if (grad_output_len != plan.out_len)
        return fail(ST_HIP_ERR_INVALID, "grad_output buffer length %zu does not match batch*c_out*oh*ow=%zu", grad_output_len,
                    plan.out_len);
    if (grad_input_len != plan.input_len)
        return fail(ST_HIP_ERR_INVALID, "grad_input buffer length %zu does not match batch*c_in*h*w=%zu", grad_input_len,
                    plan.input_len);
    if (grad_weight_len != plan.weight_len)
        return fail(ST_HIP_ERR_INVALID, "grad_weight buffer length %zu does not match c_out*c_in*kh*kw=%zu", grad_weight_len,
                    plan.weight_len);
    if (grad_bias_len != c_out)
        return fail(ST_HIP_ERR_INVALID, "grad_bias buffer length %zu does not match c_out=%zu", grad_bias_len, c_out);
    if (c_out * kh * kw > static_cast<size_t>(kMaxDim))
        return fail(ST_HIP_ERR_UNSUPPORTED, "conv2d backward reduction extent c_out*kh*kw=%zu exceeds i32", c_out * kh * kw);
    ST_HIP_CHECK(reject_null(input, input_len, "conv2d backward"));
    ST_HIP_CHECK(reject_null(weight, weight_len, "conv2d backward"));
    ST_HIP_CHECK(reject_null(grad_output, grad_output_len, "conv2d backward"));
    ST_HIP_CHECK(reject_null(grad_input, grad_input_len, "conv2d backward"));
    ST_HIP_CHECK(reject_null(grad_weight, grad_weight_len, "conv2d backward"));
    ST_HIP_CHECK(reject_null(grad_bias, grad_bias_len, "conv2d backward"));
    if (batch == 0) return ST_HIP_OK;  // conv.rs:787-789: an empty batch leaves the parameter gradients untouched
    ST_HIP_CHECK(check_conv_family(plan.shape, 1, nullptr, nullptr));

    Lease lease;
    ST_HIP_CHECK(lease.status());
    void *d_x, *d_w, *d_g, *d_gi, *d_gw, *d_gb;
    ST_HIP_CHECK(lease.upload(0, input, input_len * sizeof(float), &d_x));
    ST_HIP_CHECK(lease.upload(1, weight, weight_len * sizeof(float), &d_w));
    ST_HIP_CHECK(lease.upload(2, grad_output, grad_output_len * sizeof(float), &d_g));
    ST_HIP_CHECK(lease.buffer(3, grad_input_len * sizeof(float), &d_gi));
    ST_HIP_CHECK(lease.buffer(4, grad_weight_len * sizeof(float), &d_gw));
    ST_HIP_CHECK(lease.buffer(5, grad_bias_len * sizeof(float), &d_gb));
    const float scale = 1.0f / static_cast<float>(batch);  // conv.rs:793,799
    // The three kernels share the stream's workspace one after the other (stream order).
    ST_HIP_CHECK(launch_status(launch_conv2d_grad_weight_f32(plan.shape, static_cast<const float *>(d_x),
                                                             static_cast<const float *>(d_g), scale,
                                                             static_cast<float *>(d_gw), lease.stream()),
                               "conv2d grad_weight launch"));
    ST_HIP_CHECK(launch_status(launch_conv2d_grad_bias_f32(plan.shape, static_cast<const float *>(d_g), scale,
                                                           static_cast<float *>(d_gb), lease.stream()),
                               "conv2d grad_bias launch"));
    ST_HIP_CHECK(launch_status(launch_conv2d_grad_input_f32(plan.shape, static_cast<const float *>(d_g),
                                                            static_cast<const float *>(d_w), static_cast<float *>(d_gi),
                                                            lease.stream()),
                               "conv2d grad_input launch"));
    ST_HIP_CHECK(lease.download(grad_weight, d_gw, grad_weight_len * sizeof(float)));
    ST_HIP_CHECK(lease.download(grad_bias, d_gb, grad_bias_len * sizeof(float)));
    return lease.download(grad_input, d_gi, grad_input_len * sizeof(float));
}

int st_hip_attention_f32(size_t contexts, size_t sequence, size_t head_dim, float scale, int causal,
                         const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len,
                         const float *z_bias, size_t z_bias_len, const float *attn_bias, size_t attn_bias_len,
                         float *out, size_t out_len)
{
    ST_HIP_CHECK(ensure_init());
    AttentionPlan plan;
    ST_HIP_CHECK(plan_attention(contexts, sequence, head_dim, &plan));
    // Shape checks in the order of crates/st-tensor/src/pure.rs:4094-4146.
    if (q_len != plan.qkv_len)
        return fail(ST_HIP_ERR_INVALID, "query buffer length %zu does not match contexts*sequence*head_dim=%zu", q_len,
                    plan.qkv_len);
    if (k_len != plan.qkv_len)
        return fail(ST_HIP_ERR_INVALID, "key buffer length %zu does not match contexts*sequence*head_dim=%zu", k_len,
                    plan.qkv_len);
    if (v_len != plan.qkv_len)
        return fail(ST_HIP_ERR_INVALID, "value buffer length %zu does not match contexts*sequence*head_dim=%zu", v_len,
                    plan.qkv_len);
    if (z_bias != nullptr && z_bias_len != plan.z_len)
        return fail(ST_HIP_ERR_INVALID, "z_bias buffer length %zu does not match contexts*sequence=%zu", z_bias_len,
                    plan.z_len);
    if (attn_bias != nullptr && attn_bias_len != plan.bias_len)
        return fail(ST_HIP_ERR_INVALID, "attn_bias buffer length %zu does not match contexts*sequence*sequence=%zu",
                    attn_bias_len, plan.bias_len);
    if (out_len != plan.qkv_len)
        return fail(ST_HIP_ERR_INVALID, "output buffer length %zu does not match contexts*sequence*head_dim=%zu",
                    out_len, plan.qkv_len);
    ST_HIP_CHECK(reject_null(q, q_len, "attention"));
    ST_HIP_CHECK(reject_null(k, k_len, "attention"));
    ST_HIP_CHECK(reject_null(v, v_len, "attention"));
    ST_HIP_CHECK(reject_null(out, out_len, "attention"));
    // Finite checks, pure.rs:4148-4157.
    if (!std::isfinite(scale))
        return fail(ST_HIP_ERR_NONFINITE, "non-finite value encountered in scaled_dot_attention_scale: %g",
                    static_cast<double>(scale));
    ST_HIP_CHECK(validate_finite_slice("scaled_dot_attention_query", q, q_len));
    ST_HIP_CHECK(validate_finite_slice("scaled_dot_attention_key", k, k_len));
    ST_HIP_CHECK(validate_finite_slice("scaled_dot_attention_value", v, v_len));
    if (z_bias) ST_HIP_CHECK(validate_finite_slice("scaled_dot_attention_z_bias", z_bias, z_bias_len));
    if (attn_bias) ST_HIP_CHECK(validate_finite_slice("scaled_dot_attention_attn_bias", attn_bias, attn_bias_len));
    if (plan.rows == 0 || head_dim == 0) return ST_HIP_OK;  // zeros(rows, head_dim): pure.rs:4171-4193
    ST_HIP_CHECK(check_attention_kernel_limits(contexts, sequence, head_dim));

    Lease lease;
    ST_HIP_CHECK(lease.status());
    void *d_q, *d_k, *d_v, *d_out, *d_z = nullptr, *d_b = nullptr;
    ST_HIP_CHECK(lease.upload(0, q, q_len * sizeof(float), &d_q));
    ST_HIP_CHECK(lease.upload(1, k, k_len * sizeof(float), &d_k));
    ST_HIP_CHECK(lease.upload(2, v, v_len * sizeof(float), &d_v));
    ST_HIP_CHECK(lease.buffer(3, out_len * sizeof(float), &d_out));
    if (z_bias) ST_HIP_CHECK(lease.upload(4, z_bias, z_bias_len * sizeof(float), &d_z));
    if (attn_bias) ST_HIP_CHECK(lease.upload(5, attn_bias, attn_bias_len * sizeof(float), &d_b));
    ST_HIP_CHECK(launch_status(
        launch_attention_f32(contexts, sequence, head_dim, scale, causal != 0, static_cast<const float *>(d_q),
                             static_cast<const float *>(d_k), static_cast<const float *>(d_v),
                             static_cast<const float *>(d_z), static_cast<const float *>(d_b),
                             static_cast<float *>(d_out), lease.stream()),
        "attention launch"));
    ST_HIP_CHECK(lease.download(out, d_out, out_len * sizeof(float)));
    // Output finite check, pure.rs:4206-4210.  The CPU path reports the first overflowing intermediate
    // (dot/logit/denom/...); on the GPU any such overflow surfaces here as a non-finite output.
    return validate_finite_slice("scaled_dot_attention_output", out, out_len);
}

// ---------------------------------------------------------------------------------------------
// Device-resident forms
// ---------------------------------------------------------------------------------------------

int st_hip_gemm_f32_dev(size_t m, size_t n, size_t k, float scale, int lhs_transposed, const float *lhs,
                        const float *rhs, float *out, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_CHECK(validate_gemm_scale(scale));
    ST_HIP_CHECK(validate_kernel_dims(m, n, k));
    if (m == 0 || n == 0) return ST_HIP_OK;
    if (!out || (k != 0 && (!lhs || !rhs)))
        return fail(ST_HIP_ERR_INVALID, "gemm received a null pointer; provide contiguous row-major buffers");
    GemmEpilogue epilogue;
    epilogue.scale = scale;
    return launch_status(launch_gemm_f32(m, n, k, lhs_transposed != 0, lhs, rhs, out, epilogue, as_stream(stream)),
                         "gemm_f32 launch");
}

int st_hip_gemm_bias_act_f32_dev(size_t m, size_t n, size_t k, int activation, const float *lhs, const float *rhs,
                                 const float *bias, const float *residual, float *out, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_CHECK(validate_activation(activation, true));
    ST_HIP_CHECK(validate_kernel_dims(m, n, k));
    if (m == 0 || n == 0) return ST_HIP_OK;
    if (!out || (k != 0 && (!lhs || !rhs)))
        return fail(ST_HIP_ERR_INVALID, "gemm received a null pointer; provide contiguous row-major buffers");
    GemmEpilogue epilogue;
    epilogue.bias = bias;
    epilogue.residual = residual;
    epilogue.activation = activation;
    return launch_status(launch_gemm_f32(m, n, k, false, lhs, rhs, out, epilogue, as_stream(stream)),
                         "gemm_bias_act_f32 launch");
}

int st_hip_gemm_prepacked_bias_act_f32_dev(size_t m, size_t n, size_t k, int activation, const float *lhs,
                                           const float *packed_rhs, const float *bias, const float *residual, float *out,
                                           void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_CHECK(validate_activation(activation, true));
    ST_HIP_CHECK(validate_kernel_dims(m, n, k));
    if (m == 0 || n == 0) return ST_HIP_OK;
    if (!out || (k != 0 && (!lhs || !packed_rhs)))
        return fail(ST_HIP_ERR_INVALID, "gemm received a null pointer; provide contiguous row-major buffers");
    GemmEpilogue epilogue;
    epilogue.bias = bias;
    epilogue.residual = residual;
    epilogue.activation = activation;
    return launch_status(launch_gemm_f32_packed(m, n, k, lhs, packed_rhs, out, epilogue, as_stream(stream)),
                         "gemm_prepacked launch");
}

int st_hip_pack_rhs_f32_dev(size_t k, size_t n, const float *rhs, float *packed, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_CHECK(validate_kernel_dims(1, n, k));
    if (k == 0 || n == 0) return ST_HIP_OK;
    if (!rhs || !packed) return fail(ST_HIP_ERR_INVALID, "pack_rhs received a null pointer");
    return launch_status(launch_transpose_f32(k, n, rhs, packed, as_stream(stream)), "pack_rhs launch");
}

int st_hip_gemm_bf16_f32acc_dev(size_t m, size_t n, size_t k, const uint16_t *lhs, const uint16_t *rhs, float *out,
                                void *stream)
{
    return st_hip_gemm_bf16_bias_act_dev(m, n, k, ST_HIP_ACT_NONE, lhs, rhs, nullptr, nullptr, out, nullptr, stream);
}

int st_hip_gemm_bf16_bias_act_dev(size_t m, size_t n, size_t k, int activation, const uint16_t *lhs,
                                  const uint16_t *rhs, const float *bias, const float *residual, float *out_f32,
                                  uint16_t *out_bf16, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_CHECK(validate_activation(activation, true));
    ST_HIP_CHECK(validate_kernel_dims(m, n, k));
    if (m == 0 || n == 0) return ST_HIP_OK;
    if ((!out_f32 && !out_bf16) || (k != 0 && (!lhs || !rhs)))
        return fail(ST_HIP_ERR_INVALID, "gemm received a null pointer; provide contiguous row-major buffers");
    GemmEpilogue epilogue;
    epilogue.bias = bias;
    epilogue.residual = residual;
    epilogue.activation = activation;
    return launch_status(launch_gemm_bf16(m, n, k, lhs, rhs, out_f32, out_bf16, epilogue, as_stream(stream)),
                         "gemm_bf16 launch");
}

int st_hip_gemm_bf16_prepacked_bias_act_dev(size_t m, size_t n, size_t k, int activation, const uint16_t *lhs,
                                            const uint16_t *packed_rhs, const float *bias, const float *residual,
                                            float *out_f32, uint16_t *out_bf16, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_CHECK(validate_activation(activation, true));
    ST_HIP_CHECK(validate_kernel_dims(m, n, k));
    if (m == 0 || n == 0) return ST_HIP_OK;
    if ((!out_f32 && !out_bf16) || (k != 0 && (!lhs || !packed_rhs)))
        return fail(ST_HIP_ERR_INVALID, "gemm received a null pointer; provide contiguous row-major buffers");
    GemmEpilogue epilogue;
    epilogue.bias = bias;
    epilogue.residual = residual;
    epilogue.activation = activation;
    return launch_status(launch_gemm_bf16(m, n, k, lhs, packed_rhs, out_f32, out_bf16, epilogue, as_stream(stream), true),
                         "gemm_bf16 prepacked launch");
}

int st_hip_gemm_bf16_prepacked_residual_layer_norm_dev(size_t m, size_t n, size_t k, const uint16_t *lhs,
                                                      const uint16_t *packed_rhs, const float *bias, const float *residual,
                                                      const float *gamma, const float *beta, float epsilon, float *out_f32,
                                                      uint16_t *out_ln_bf16, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_CHECK(validate_kernel_dims(m, n, k));
    if (!std::isfinite(epsilon) || epsilon < 0.0f)
        return fail(ST_HIP_ERR_INVALID, "layer_norm epsilon must be finite and non-negative, received %g", static_cast<double>(epsilon));
    if (m == 0 || n == 0) return ST_HIP_OK;
    if (!out_f32 || !out_ln_bf16 || !gamma || !beta || (k != 0 && (!lhs || !packed_rhs)))
        return fail(ST_HIP_ERR_INVALID, "gemm + layer_norm received a null pointer; provide contiguous row-major buffers");
    return launch_status(launch_gemm_bf16_residual_layer_norm(m, n, k, lhs, packed_rhs, bias, residual, gamma, beta, epsilon,
                                                              out_f32, out_ln_bf16, as_stream(stream)),
                         "gemm_bf16 + layer_norm launch");
}

int st_hip_pack_rhs_bf16_dev(size_t k, size_t n, const uint16_t *rhs, uint16_t *packed, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ST_HIP_CHECK(validate_kernel_dims(1, n, k));
    if (k == 0 || n == 0) return ST_HIP_OK;
    if (!rhs || !packed) return fail(ST_HIP_ERR_INVALID, "pack_rhs received a null pointer");
    return launch_status(launch_transpose_u16(k, n, rhs, packed, as_stream(stream)), "pack_rhs launch");
}

int st_hip_conv2d_bias_act_f32_dev(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out, size_t kh, size_t kw,
                                   size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w, size_t dil_h,
                                   size_t dil_w, int activation, const float *input, const float *weight,
                                   const float *bias, float *out, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ConvPlan plan;
    ST_HIP_CHECK(plan_conv(batch, c_in, h, w, c_out, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, &plan));
    ST_HIP_CHECK(validate_activation(activation, true));
    if (plan.out_len == 0) return ST_HIP_OK;
    if (!input || !weight || !out)
        return fail(ST_HIP_ERR_INVALID, "conv2d received a null pointer; provide contiguous buffers");
    ST_HIP_CHECK(check_conv_family(plan.shape, 0, weight, out));
    return launch_status(launch_conv2d_f32(plan.shape, activation, input, weight, bias, out, as_stream(stream)),
                         "conv2d launch");
}

int st_hip_conv2d_bias_act_bf16_dev(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out, size_t kh, size_t kw,
                                    size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w, size_t dil_h,
                                    size_t dil_w, int activation, const uint16_t *input, const uint16_t *weight,
                                    const float *bias, float *out_f32, uint16_t *out_bf16, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ConvPlan plan;
    ST_HIP_CHECK(plan_conv(batch, c_in, h, w, c_out, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, &plan));
    ST_HIP_CHECK(validate_activation(activation, true));
    if (plan.out_len == 0) return ST_HIP_OK;
    if (!input || !weight || (!out_f32 && !out_bf16))
        return fail(ST_HIP_ERR_INVALID, "conv2d received a null pointer; provide contiguous buffers");
    const auto misaligned = [](const void *ptr, uintptr_t a) { return (reinterpret_cast<uintptr_t>(ptr) & (a - 1)) != 0; };
    if (misaligned(out_f32, 16) || misaligned(out_bf16, 8))
        return fail(ST_HIP_ERR_UNSUPPORTED, "bf16 conv2d needs a 16-byte aligned f32 output and an 8-byte aligned bf16 output");
    if (!conv2d_bf16_supported(plan.shape))
        return fail(ST_HIP_ERR_UNSUPPORTED, "bf16 conv2d: the padded channels-last copy of the input or the re-laid weights exceed 2 GiB");
    return launch_status(launch_conv2d_bf16(plan.shape, activation, input, weight, bias, out_f32, out_bf16, as_stream(stream)),
                         "conv2d bf16 launch");
}

int st_hip_conv2d_grad_input_f32_dev(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out, size_t kh, size_t kw,
                                     size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w, size_t dil_h,
                                     size_t dil_w, const float *grad_output, const float *weight, float *grad_input,
                                     void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ConvPlan plan;
    ST_HIP_CHECK(plan_conv(batch, c_in, h, w, c_out, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, &plan));
    if (c_out * kh * kw > static_cast<size_t>(kMaxDim))
        return fail(ST_HIP_ERR_UNSUPPORTED, "conv2d backward reduction extent c_out*kh*kw=%zu exceeds i32", c_out * kh * kw);
    if (plan.input_len == 0) return ST_HIP_OK;
    if (!grad_output || !weight || !grad_input)
        return fail(ST_HIP_ERR_INVALID, "conv2d backward received a null pointer; provide contiguous buffers");
    ST_HIP_CHECK(check_conv_family(plan.shape, 1, nullptr, nullptr));
    return launch_status(launch_conv2d_grad_input_f32(plan.shape, grad_output, weight, grad_input, as_stream(stream)),
                         "conv2d grad_input launch");
}

int st_hip_conv2d_grad_input_f32_noalloc_dev(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out, size_t kh,
                                             size_t kw, size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w,
                                             size_t dil_h, size_t dil_w, const float *grad_output, const float *weight,
                                             float *grad_input, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ConvPlan plan;
    ST_HIP_CHECK(plan_conv(batch, c_in, h, w, c_out, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, &plan));
    if (c_out * kh * kw > static_cast<size_t>(kMaxDim))
        return fail(ST_HIP_ERR_UNSUPPORTED, "conv2d backward reduction extent c_out*kh*kw=%zu exceeds i32", c_out * kh * kw);
    if (plan.weight_len > kNoAllocScratchBytes / sizeof(float))
        return fail(ST_HIP_ERR_UNSUPPORTED,
                    "conv2d grad_input without allocation: the weights (%zu bytes) exceed the static scratch of %zu bytes; "
                    "use st_hip_conv2d_grad_input_f32_dev",
                    plan.weight_len * sizeof(float), kNoAllocScratchBytes);
    if (plan.input_len == 0) return ST_HIP_OK;
    if (!grad_output || !weight || !grad_input)
        return fail(ST_HIP_ERR_INVALID, "conv2d backward received a null pointer; provide contiguous buffers");
    ST_HIP_CHECK(check_conv_family(plan.shape, 1, nullptr, nullptr));
    void *scratch_ptr = nullptr;
    ST_HIP_TRY(noalloc_scratch(&scratch_ptr), "hipGetSymbolAddress(scratch)");
    return launch_status(launch_conv2d_grad_input_f32(plan.shape, grad_output, weight, grad_input, as_stream(stream),
                                                      static_cast<float *>(scratch_ptr)),
                         "conv2d grad_input launch");
}

int st_hip_conv2d_grad_weight_f32_dev(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out, size_t kh, size_t kw,
                                      size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w, size_t dil_h,
                                      size_t dil_w, const float *input, const float *grad_output, float scale,
                                      float *grad_weight, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ConvPlan plan;
    ST_HIP_CHECK(plan_conv(batch, c_in, h, w, c_out, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, &plan));
    if (!std::isfinite(scale)) return fail(ST_HIP_ERR_INVALID, "gemm scale must be finite, received %g", static_cast<double>(scale));
    if (!grad_weight || (batch != 0 && plan.out_len != 0 && (!input || !grad_output)))
        return fail(ST_HIP_ERR_INVALID, "conv2d backward received a null pointer; provide contiguous buffers");
    return launch_status(launch_conv2d_grad_weight_f32(plan.shape, input, grad_output, scale, grad_weight, as_stream(stream)),
                         "conv2d grad_weight launch");
}

int st_hip_conv2d_grad_bias_f32_dev(size_t batch, size_t c_in, size_t h, size_t w, size_t c_out, size_t kh, size_t kw,
                                    size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w, size_t dil_h,
                                    size_t dil_w, const float *grad_output, float scale, float *grad_bias, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    ConvPlan plan;
    ST_HIP_CHECK(plan_conv(batch, c_in, h, w, c_out, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, &plan));
    if (!std::isfinite(scale)) return fail(ST_HIP_ERR_INVALID, "gemm scale must be finite, received %g", static_cast<double>(scale));
    if (!grad_bias || (plan.out_len != 0 && !grad_output))
        return fail(ST_HIP_ERR_INVALID, "conv2d backward received a null pointer; provide contiguous buffers");
    return launch_status(launch_conv2d_grad_bias_f32(plan.shape, grad_output, scale, grad_bias, as_stream(stream)),
                         "conv2d grad_bias launch");
}

int st_hip_attention_f32_dev(size_t contexts, size_t sequence, size_t head_dim, float scale, int causal,
                             const float *q, const float *k, const float *v, const float *z_bias,
                             const float *attn_bias, float *out, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    AttentionPlan plan;
    ST_HIP_CHECK(plan_attention(contexts, sequence, head_dim, &plan));
    if (!std::isfinite(scale))
        return fail(ST_HIP_ERR_NONFINITE, "non-finite value encountered in scaled_dot_attention_scale: %g",
                    static_cast<double>(scale));
    if (plan.rows == 0 || head_dim == 0) return ST_HIP_OK;
    ST_HIP_CHECK(check_attention_kernel_limits(contexts, sequence, head_dim));
    if (!q || !k || !v || !out)
        return fail(ST_HIP_ERR_INVALID, "attention received a null pointer; provide contiguous buffers");
    return launch_status(launch_attention_f32(contexts, sequence, head_dim, scale, causal != 0, q, k, v, z_bias,
                                              attn_bias, out, as_stream(stream)),
                         "attention launch");
}

int st_hip_attention_bf16_dev(size_t batch, size_t heads, size_t sequence, size_t head_dim, float scale, int causal,
                              const uint16_t *q, const uint16_t *k, const uint16_t *v, size_t ld_in, uint16_t *out,
                              size_t ld_out, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    size_t contexts = 0, width = 0;
    if (!checked_mul(batch, heads, &contexts) || !checked_mul(heads, head_dim, &width))
        return fail(ST_HIP_ERR_INVALID, "attention dimensions overflow");
    AttentionPlan plan;
    ST_HIP_CHECK(plan_attention(contexts, sequence, head_dim, &plan));
    if (!std::isfinite(scale))
        return fail(ST_HIP_ERR_NONFINITE, "non-finite value encountered in scaled_dot_attention_scale: %g",
                    static_cast<double>(scale));
    if (plan.rows == 0 || head_dim == 0) return ST_HIP_OK;
    ST_HIP_CHECK(check_attention_kernel_limits(contexts, sequence, head_dim));
    if (!q || !k || !v || !out)
        return fail(ST_HIP_ERR_INVALID, "attention received a null pointer; provide contiguous buffers");
    if (ld_in < width || ld_out < width)
        return fail(ST_HIP_ERR_INVALID, "attention row stride %zu/%zu is smaller than heads*head_dim=%zu", ld_in, ld_out,
                    width);
    if (ld_in > kMaxDim || ld_out > kMaxDim) return fail(ST_HIP_ERR_UNSUPPORTED, "attention row stride exceeds i32");
    if (!attention_bf16_supported(sequence, head_dim, ld_in, ld_out, q, k, v, out))
        return fail(ST_HIP_ERR_UNSUPPORTED,
                    "bf16 attention needs head_dim 64 or 128 (got %zu), ld_in %% 8 == 0, ld_out %% 4 == 0 and aligned "
                    "buffers",
                    head_dim);
    return launch_status(launch_attention_bf16(batch, heads, sequence, head_dim, scale, causal != 0, q, k, v, ld_in, out,
                                               ld_out, as_stream(stream)),
                         "attention launch");
}

int st_hip_row_softmax_f32_dev(size_t rows, size_t cols, const float *in, float *out, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    if (rows > kMaxDim || cols > kMaxDim) return fail(ST_HIP_ERR_UNSUPPORTED, "row_softmax dimension exceeds i32");
    if (rows == 0 || cols == 0) return ST_HIP_OK;
    if (!in || !out) return fail(ST_HIP_ERR_INVALID, "row_softmax received a null pointer");
    return launch_status(launch_row_softmax_f32(rows, cols, in, out, as_stream(stream)), "row_softmax launch");
}

int st_hip_gelu_f32_dev(size_t count, const float *in, float *out, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    if (count == 0) return ST_HIP_OK;
    if (!in || !out) return fail(ST_HIP_ERR_INVALID, "gelu received a null pointer");
    return launch_status(launch_gelu_f32(count, in, out, as_stream(stream)), "gelu launch");
}

int st_hip_count_nonfinite_f32_dev(size_t count, const float *data, uint64_t *nonfinite, uint64_t *first_index,
                                   float *first_value, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    if (!nonfinite) return fail(ST_HIP_ERR_INVALID, "count_nonfinite received a null out-pointer");
    *nonfinite = 0;
    if (first_index) *first_index = 0;
    if (first_value) *first_value = 0.0f;
    if (count == 0) return ST_HIP_OK;
    if (!data) return fail(ST_HIP_ERR_INVALID, "count_nonfinite received a null pointer");
    hipStream_t s = as_stream(stream);
    void *workspace = nullptr;
    ST_HIP_TRY(stream_workspace(s, 16, &workspace), "hipMalloc");
    unsigned long long *status = static_cast<unsigned long long *>(workspace);
    const unsigned long long init[2] = {0ull, ~0ull};
    ST_HIP_TRY(hipMemcpyAsync(status, init, sizeof init, hipMemcpyHostToDevice, s), "hipMemcpyAsync(H2D)");
    ST_HIP_CHECK(launch_status(launch_nonfinite_probe_f32(count, data, status, s), "count_nonfinite launch"));
    unsigned long long result[2] = {0, 0};
    ST_HIP_TRY(hipMemcpyAsync(result, status, sizeof result, hipMemcpyDeviceToHost, s), "hipMemcpyAsync(D2H)");
    ST_HIP_TRY(hipStreamSynchronize(s), "hipStreamSynchronize");
    *nonfinite = result[0];
    if (result[0] != 0) {
        if (first_index) *first_index = result[1];
        if (first_value) {
            ST_HIP_TRY(hipMemcpyAsync(first_value, data + result[1], sizeof(float), hipMemcpyDeviceToHost, s), "hipMemcpyAsync(D2H)");
            ST_HIP_TRY(hipStreamSynchronize(s), "hipStreamSynchronize");
        }
    }
    return ST_HIP_OK;
}

int st_hip_gelu_backward_f32_dev(size_t count, const float *z, const float *grad, float *out, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    if (count == 0) return ST_HIP_OK;
    if (!z || !grad || !out) return fail(ST_HIP_ERR_INVALID, "gelu_backward received a null pointer");
    return launch_status(launch_gelu_backward_f32(count, z, grad, out, as_stream(stream)), "gelu_backward launch");
}

int st_hip_scale_f32_dev(size_t count, const float *in, float scale, float *out, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    if (!std::isfinite(scale))
        return fail(ST_HIP_ERR_NONFINITE, "non-finite value encountered in scale_factor: %g", static_cast<double>(scale));
    if (count == 0) return ST_HIP_OK;
    if (!in || !out) return fail(ST_HIP_ERR_INVALID, "scale received a null pointer");
    return launch_status(launch_scale_f32(count, in, scale, out, as_stream(stream)), "scale launch");
}

int st_hip_add_row_f32_dev(size_t rows, size_t cols, float *data, const float *bias, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    size_t count = 0;
    if (!checked_mul(rows, cols, &count)) return fail(ST_HIP_ERR_INVALID, "add_row dimensions overflow");
    if (cols > kMaxDim) return fail(ST_HIP_ERR_UNSUPPORTED, "add_row dimension exceeds i32");
    if (count == 0) return ST_HIP_OK;
    if (!data || !bias) return fail(ST_HIP_ERR_INVALID, "add_row received a null pointer");
    return launch_status(launch_add_row_f32(rows, cols, data, bias, as_stream(stream)), "add_row launch");
}

int st_hip_sum_axis0_f32_dev(size_t rows, size_t cols, const float *in, float scale, float *out, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    if (!std::isfinite(scale))
        return fail(ST_HIP_ERR_NONFINITE, "non-finite value encountered in sum_axis0_scaled_factor: %g",
                    static_cast<double>(scale));
    if (rows > kMaxDim || cols > kMaxDim) return fail(ST_HIP_ERR_UNSUPPORTED, "sum_axis0 dimension exceeds i32");
    if (cols == 0) return ST_HIP_OK;
    if (!out || (rows != 0 && !in)) return fail(ST_HIP_ERR_INVALID, "sum_axis0 received a null pointer");
    return launch_status(launch_sum_axis0_f32(rows, cols, in, scale, out, as_stream(stream)), "sum_axis0 launch");
}

int st_hip_layer_norm_f32_dev(size_t rows, size_t cols, const float *x, const float *residual, const float *gamma,
                              const float *beta, float epsilon, float *out_f32, uint16_t *out_bf16, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    if (rows > kMaxDim || cols > kMaxDim) return fail(ST_HIP_ERR_UNSUPPORTED, "layer_norm dimension exceeds i32");
    if (rows == 0 || cols == 0) return ST_HIP_OK;
    if (!x || !gamma || !beta || (!out_f32 && !out_bf16))
        return fail(ST_HIP_ERR_INVALID, "layer_norm received a null pointer");
    return launch_status(
        launch_layer_norm_f32(rows, cols, x, residual, gamma, beta, epsilon, out_f32, out_bf16, as_stream(stream)),
        "layer_norm launch");
}

int st_hip_embedding_f32_dev(size_t tokens, size_t vocab, size_t dim, const float *token_ids, const float *table,
                             float *out, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    if (vocab == 0) return fail(ST_HIP_ERR_INVALID, "embedding vocabulary must be non-empty");
    if (tokens > kMaxDim || vocab > kMaxDim || dim > kMaxDim)
        return fail(ST_HIP_ERR_UNSUPPORTED, "embedding dimension exceeds i32");
    if (tokens == 0 || dim == 0) return ST_HIP_OK;
    if (!token_ids || !table || !out) return fail(ST_HIP_ERR_INVALID, "embedding received a null pointer");
    return launch_status(launch_embedding_f32(tokens, vocab, dim, token_ids, table, out, as_stream(stream)),
                         "embedding launch");
}

int st_hip_f32_to_bf16_dev(size_t count, const float *in, uint16_t *out, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    if (count == 0) return ST_HIP_OK;
    if (!in || !out) return fail(ST_HIP_ERR_INVALID, "f32_to_bf16 received a null pointer");
    return launch_status(launch_f32_to_bf16(count, in, out, as_stream(stream)), "f32_to_bf16 launch");
}

int st_hip_split_heads_f32_dev(size_t batch, size_t seq, size_t heads, size_t head_dim, const float *qkv, float *q,
                               float *k, float *v, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    size_t total;
    if (!checked_mul(batch, seq, &total) || !checked_mul(total, heads, &total) ||
        !checked_mul(total, head_dim, &total) || total > kMaxDim / 3)
        return fail(ST_HIP_ERR_UNSUPPORTED, "split_heads volume exceeds i32");
    if (total == 0) return ST_HIP_OK;
    if (!qkv || !q || !k || !v) return fail(ST_HIP_ERR_INVALID, "split_heads received a null pointer");
    return launch_status(launch_split_heads_f32(batch, seq, heads, head_dim, qkv, q, k, v, false, as_stream(stream)),
                         "split_heads launch");
}

int st_hip_merge_heads_f32_dev(size_t batch, size_t seq, size_t heads, size_t head_dim, const float *contexts_in,
                               float *out_f32, uint16_t *out_bf16, void *stream)
{
    ST_HIP_CHECK(ensure_init());
    size_t total;
    if (!checked_mul(batch, seq, &total) || !checked_mul(total, heads, &total) ||
        !checked_mul(total, head_dim, &total) || total > kMaxDim)
        return fail(ST_HIP_ERR_UNSUPPORTED, "merge_heads volume exceeds i32");
    if (total == 0) return ST_HIP_OK;
    if (!contexts_in || (!out_f32 && !out_bf16)) return fail(ST_HIP_ERR_INVALID, "merge_heads received a null pointer");
    return launch_status(
        launch_merge_heads_f32(batch, seq, heads, head_dim, contexts_in, out_f32, out_bf16, as_stream(stream)),
        "merge_heads launch");
}

}  // extern "C"
