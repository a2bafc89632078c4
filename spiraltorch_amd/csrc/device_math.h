// Device-side scalar helpers shared by the kernels' epilogues.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "st_hip.h"

namespace sthip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

// tanh-GELU with the reference's constants (crates/st-tensor/src/pure.rs:12026-12031):
// 0.5·x·(1 + tanh(u)), u = 0.7978846·(x + 0.044715·x³).  Evaluated as x / (1 + e^(−2u)), which is the
// same function without the cancellation in 1 + tanh(u) and costs one v_exp_f32 and one division
// instead of a library tanhf; the two forms agree to a few 1e-7 relative wherever the reference's own
// rounding of 1 + tanh(u) is not the larger error.
__device__ __forceinline__ float gelu_tanh(float x)
{
    const float x_cubed = (x * x) * x;
    const float inner = 0.7978846f * (x + 0.044715f * x_cubed);
    const float e = __builtin_amdgcn_exp2f(inner * -2.8853900817779268f);  // e^(−2u); +inf for very negative u
    return x * __builtin_amdgcn_rcpf(1.0f + e);  // rcp(+inf) = 0: large negative x gives -0
}

// ReLU keeps `value` only when `value > 0`, so -0.0 and NaN become +0.0 (pure.rs:12021).
__device__ __forceinline__ float apply_activation(float value, int activation)
{
    if (activation == ST_HIP_ACT_RELU) return value > 0.0f ? value : 0.0f;
    if (activation == ST_HIP_ACT_GELU) return gelu_tanh(value);
    return value;
}

// ReLU when `relu` (a wavefront-uniform flag), else the value itself, without a branch: compare, select, select.
__device__ __forceinline__ float relu_or_identity(float value, bool relu)
{
    const float rectified = value > 0.0f ? value : 0.0f;
    return relu ? rectified : value;
}

// Sum and sum of squares of four neighbouring row values, with the association written out: the layer-norm kernel and
// the GEMM epilogue that normalises rows must add a row's values in the same order to give the same statistics.
__device__ __forceinline__ float sum4(const float4 &v) { return (v.x + v.y) + (v.z + v.w); }
__device__ __forceinline__ float sumsq4(const float4 &v) { return fmaf(v.x, v.x, v.y * v.y) + fmaf(v.z, v.z, v.w * v.w); }

// sqrt(var + epsilon) of a layer-norm row.  The reference fails a row whose sums, variance or denominator overflow
// (labels layer_norm_sumsq … layer_norm_denom, crates/st-tensor/src/pure.rs:4030-4045); an infinite denominator would
// instead turn the whole row into finite zeros here, so it becomes NaN and the caller's finite check on the result
// reports the row.  Finite denominators pass through unchanged.
__device__ __forceinline__ float layer_norm_denominator(float var, float epsilon)
{
    const float denom = sqrtf(var + epsilon);
    return denom < INFINITY ? denom : NAN;
}

// The two places of a layer-norm row where the compiler may or may not fuse a multiply with the addition behind it,
// in separately rounded steps as the reference computes them (crates/st-tensor/src/pure.rs:4030-4056; Rust does not
// contract): var = E[x²] − mean² clamped at 0, and normalised·γ + β.  Contraction is switched off for these statements
// (__fmul_rn and friends are plain operators here and fuse like any other): left to the compiler, the stand-alone
// kernels fused both while the GEMM kernel that normalises its own rows fused only the second, the variances of a few
// rows in a thousand differed in their last bit, and one value in two million came out one bf16 step apart.
__device__ __forceinline__ float layer_norm_variance(float sumsq, float mean, float cols_f)
{
#pragma clang fp contract(off)
    const float mean_of_squares = sumsq / cols_f;
    const float square_of_mean = mean * mean;
    return fmaxf(mean_of_squares - square_of_mean, 0.0f);
}
__device__ __forceinline__ float layer_norm_scale_shift(float normalised, float gamma, float beta)
{
#pragma clang fp contract(off)
    const float scaled = normalised * gamma;
    return scaled + beta;
}

// Runs `body(act, has_residual)` with the activation as a callable and the presence of a residual as a compile-time
// constant, chosen once from the (wavefront-uniform) launch arguments: an epilogue that decides them per element
// compiles to a chain of scalar branches around every store.
template <class Body>
__device__ __forceinline__ void with_epilogue_ops(int activation, bool has_residual, Body &&body)
{
    auto gelu = [](float v) { return gelu_tanh(v); };
    auto cheap = [relu = activation == ST_HIP_ACT_RELU](float v) { return relu_or_identity(v, relu); };
    if (activation == ST_HIP_ACT_GELU) {
        if (has_residual) body(gelu, std::true_type{});
        else body(gelu, std::false_type{});
    } else {
        if (has_residual) body(cheap, std::true_type{});
        else body(cheap, std::false_type{});
    }
}

// Round-to-nearest-even f32 -> bf16 bit pattern through the hardware conversion (v_cvt_pk_bf16_f32); NaN stays
// a quiet NaN.
typedef __bf16 bf16x2_hw __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2_rne(float lo, float hi)
{
    const bf16x2_hw v = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
    return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f)
{
    return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

}  // namespace sthip
