// Device-side scalar helpers shared by the kernels' epilogues.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "st_hip.h"

namespace sthip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

// tanh-GELU with the reference's constants and evaluation order
// (crates/st-tensor/src/pure.rs:12026-12031).
__device__ __forceinline__ float gelu_tanh(float x)
{
    const float x_cubed = (x * x) * x;
    const float inner = 0.7978846f * (x + 0.044715f * x_cubed);
    return (0.5f * x) * (1.0f + tanhf(inner));
}

// ReLU keeps `value` only when `value > 0`, so -0.0 and NaN become +0.0 (pure.rs:12021).
__device__ __forceinline__ float apply_activation(float value, int activation)
{
    if (activation == ST_HIP_ACT_RELU) return value > 0.0f ? value : 0.0f;
    if (activation == ST_HIP_ACT_GELU) return gelu_tanh(value);
    return value;
}

// Round-to-nearest-even f32 -> bf16 bit pattern; NaN stays a quiet NaN.
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

}  // namespace sthip
