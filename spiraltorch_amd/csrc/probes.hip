// Measurement aids that are part of the library so that benchmarks and profiles run committed code only: a loop of
// nothing but bf16 matrix instructions on register operands.  It shows what the matrix pipes of this chip deliver on
// given operand bits with no memory instruction in the way (the clock a chip settles at under matrix load depends on
// how many operand bits toggle), i.e. the ceiling the bf16 GEMM kernels are to be read against.
#include "kernels.h"

namespace sthip {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Four wavefronts per workgroup; a wavefront keeps 2 × 4 A and 2 × 4 B fragments (its lanes' 16 bytes each, read once
// from `operands`) and issues 32 v_mfma_f32_32x32x16_bf16 per iteration into sixteen independent accumulators — the
// 4 × 4 register blocking of the GEMM kernels' main loop.
__global__ __launch_bounds__(256) void probe_mfma_bf16_kernel(const u32x4 *operands, float *sink, int iterations)
{
    f32x16 acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
    bf16x8 a[2][4], b[2][4];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a[s][i] = __builtin_bit_cast(bf16x8, operands[threadIdx.x + 256 * (s * 8 + i)]);
            b[s][i] = __builtin_bit_cast(bf16x8, operands[threadIdx.x + 256 * (s * 8 + 4 + i)]);
        }
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s][i], b[s][j], acc[i * 4 + j], 0, 0, 0);
    }
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) total += acc[i][r];
    sink[static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x] = total;
}

}  // namespace

hipError_t launch_probe_mfma_bf16(size_t workgroups, size_t iterations, const uint16_t *operands, float *sink, hipStream_t stream)
{
    if (workgroups == 0 || iterations == 0) return hipSuccess;
    if (workgroups > 0x7fffffffu || iterations > 0x7fffffffu) return hipErrorInvalidValue;
    hipLaunchKernelGGL(probe_mfma_bf16_kernel, dim3(static_cast<unsigned>(workgroups)), dim3(256), 0, stream,
                       reinterpret_cast<const u32x4 *>(operands), sink, static_cast<int>(iterations));
    return hipGetLastError();
}

}  // namespace sthip
