// Measurement aids that are part of the library so that benchmarks and profiles run committed code only: a loop of
// nothing but bf16 matrix instructions on register operands.  It shows what the matrix pipes of this chip deliver on
// given operand bits with no memory instruction in the way (the clock a chip settles at under matrix load depends on
// how many operand bits toggle), i.e. the ceiling the bf16 GEMM kernels are to be read against; and a loop of nothing
// but direct-to-LDS loads, which shows what one compute unit can stream out of L2, the memory-side cache or HBM
// (depending on the size of the region it walks) with the GEMM kernels' own access shape.
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

// The same for the f32 matrix instruction of the f32 GEMM, convolution and attention kernels: four wavefronts per
// workgroup, 2 × 4 A and B values per lane (v_mfma_f32_32x32x2_f32 takes one f32 per lane and operand), 32 instructions
// per iteration into sixteen independent accumulators.
__global__ __launch_bounds__(256) void probe_mfma_f32_kernel(const float *operands, float *sink, int iterations)
{
    f32x16 acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
    float a[2][4], b[2][4];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a[s][i] = operands[threadIdx.x + 256 * (s * 8 + i)];
            b[s][i] = operands[threadIdx.x + 256 * (s * 8 + 4 + i)];
        }
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s][i], b[s][j], acc[i * 4 + j], 0, 0, 0);
    }
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) total += acc[i][r];
    sink[static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x] = total;
}

typedef __attribute__((address_space(3))) void *probe_lds_ptr;

// Eight wavefronts per workgroup; per iteration a wavefront issues eight buffer_load_dwordx4 ... lds of 1 KB — eight
// rows of 128 B at a row pitch of 1 KB, the shape of a bf16 operand k-tile at K = 512 — and waits for the eight of the
// iteration before, so 8 to 16 KB per wavefront are in flight.  Workgroups start at different places of the region and
// walk all of it.
__global__ __launch_bounds__(512) void probe_stream_lds_kernel(const unsigned char *region, unsigned region_bytes, int iterations)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char probe_lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char *>(region), 0, static_cast<int>(region_bytes), 0x00020000);
    const unsigned voff = (lane >> 3) * 1024u + (lane & 7) * 16u;
    const unsigned span = region_bytes - 8192u;  // a batch covers 8 KB from its first byte
    unsigned pos = (blockIdx.x * 7919u * 8192u + wave * 8192u) % span;
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int d = 0; d < 8; ++d)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (probe_lds_ptr)(probe_lds + wave * 8192 + d * 1024), 16, voff,
                                                     __builtin_amdgcn_readfirstlane(pos + d * 128u), 0, 0);
        pos = (pos + 8u * 8192u) % span;
        __builtin_amdgcn_s_waitcnt(8 | (7 << 4) | (15 << 8));  // vmcnt(8): the batch before this one has landed
    }
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));
}

}  // namespace

hipError_t launch_probe_stream_lds(size_t workgroups, size_t iterations, const void *region, size_t region_bytes, hipStream_t stream)
{
    if (workgroups == 0 || iterations == 0) return hipSuccess;
    if (workgroups > 0x7fffffffu || iterations > 0x7fffffffu || region_bytes < 65536 || region_bytes >= (1ull << 31))
        return hipErrorInvalidValue;
    constexpr size_t lds_bytes = 8 * 8192;
    hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(probe_stream_lds_kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (rc != hipSuccess) return rc;
    hipLaunchKernelGGL(probe_stream_lds_kernel, dim3(static_cast<unsigned>(workgroups)), dim3(512), lds_bytes, stream,
                       static_cast<const unsigned char *>(region), static_cast<unsigned>(region_bytes), static_cast<int>(iterations));
    return hipGetLastError();
}

hipError_t launch_probe_mfma_f32(size_t workgroups, size_t iterations, const float *operands, float *sink, hipStream_t stream)
{
    if (workgroups == 0 || iterations == 0) return hipSuccess;
    if (workgroups > 0x7fffffffu || iterations > 0x7fffffffu) return hipErrorInvalidValue;
    hipLaunchKernelGGL(probe_mfma_f32_kernel, dim3(static_cast<unsigned>(workgroups)), dim3(256), 0, stream, operands, sink,
                       static_cast<int>(iterations));
    return hipGetLastError();
}

hipError_t launch_probe_mfma_bf16(size_t workgroups, size_t iterations, const uint16_t *operands, float *sink, hipStream_t stream)
{
    if (workgroups == 0 || iterations == 0) return hipSuccess;
    if (workgroups > 0x7fffffffu || iterations > 0x7fffffffu) return hipErrorInvalidValue;
    hipLaunchKernelGGL(probe_mfma_bf16_kernel, dim3(static_cast<unsigned>(workgroups)), dim3(256), 0, stream,
                       reinterpret_cast<const u32x4 *>(operands), sink, static_cast<int>(iterations));
    return hipGetLastError();
}

}  // namespace sthip
