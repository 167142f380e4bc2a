// Diagnostics: what the matrix cores of this device sustain when nothing else runs.
//
// 256 workgroups of 8 wavefronts issue 32x32 matrix instructions back to back on eight independent accumulators, operands in
// registers: no LDS, no memory.  With all-zero operands the device holds its top clock and reaches the published rate; with
// operands that change from instruction to instruction, as a GEMM's do, power management lowers the clock.  The rate this
// loop reaches with random operands is the ceiling a GEMM kernel on the same data can be measured against; each workgroup
// also notes how many shader clocks and how many ticks of the constant 100 MHz counter its loop took, which gives the
// clock itself.
#include "mme_kernels.hpp"

namespace mme
{
namespace
{
typedef int   v8i __attribute__((ext_vector_type(8)));
typedef short v8s __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ __forceinline__ uint32_t mix32(uint32_t x)
{
    x ^= x >> 16;
    x *= 0x7feb352dU;
    x ^= x >> 15;
    x *= 0x846ca68bU;
    x ^= x >> 16;
    return x;
}

// KIND 0: fp8 e4m3 codes (top exponent bit of each byte cleared: no NaN); 1: bf16 values of magnitude below 2
template<int KIND>
__global__ __launch_bounds__(512) void matrix_core_rate_kernel(int iters, int random_operands, uint64_t* stamps, float* sink)
{
    v8i a[4], b[4];
    for (int s = 0; s < 4; s++)
        for (int i = 0; i < 8; i++)
        {
            const uint32_t ra = mix32(threadIdx.x * 131u + blockIdx.x * 7919u + s * 17u + i), rb = mix32(ra + 0x9e3779b9u);
            const uint32_t keep = KIND == 0 ? 0xbfbfbfbfu : 0xbfffbfffu;
            a[s][i] = random_operands ? (int) (ra & keep) : 0;
            b[s][i] = random_operands ? (int) (rb & keep) : 0;
        }
    v16f acc[8];
    for (int j = 0; j < 8; j++)
        for (int i = 0; i < 16; i++) acc[j][i] = 0.f;
    const uint64_t c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; it++)
    {
#pragma unroll
        for (int j = 0; j < 8; j++)
        {
            if constexpr (KIND == 0) acc[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[j & 3], b[(j >> 1) & 3], acc[j], 0, 0, 0, 0, 0, 0);
            else
            {
                // one 8-register operand set feeds two 32x32x16 instructions (4 registers = 8 bf16 values per lane each)
                const v8i av = a[j & 3], bv = b[(j >> 1) & 3];
                typedef int v4i __attribute__((ext_vector_type(4)));
                const v4i a0 = {av[0], av[1], av[2], av[3]}, b0 = {bv[0], bv[1], bv[2], bv[3]};
                const v4i a1 = {av[4], av[5], av[6], av[7]}, b1 = {bv[4], bv[5], bv[6], bv[7]};
                typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a0), __builtin_bit_cast(v8bf, b0), acc[j], 0, 0, 0);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a1), __builtin_bit_cast(v8bf, b1), acc[j], 0, 0, 0);
            }
        }
    }
    const uint64_t c1 = clock64(), w1 = wall_clock64();
    float s = 0;
    for (int j = 0; j < 8; j++)
        for (int i = 0; i < 16; i++) s += acc[j][i];
    if (s == 12345.678f) sink[0] = s; // keeps the accumulators alive
    if (threadIdx.x == 0)
    {
        stamps[blockIdx.x * 2] = c1 - c0;
        stamps[blockIdx.x * 2 + 1] = w1 - w0;
    }
}
} // namespace

hipError_t launch_matrix_core_rate(int kind, int random_operands, int iters, uint64_t* stamps, hipStream_t s)
{
    float* sink = (float*) (stamps + 512); // a cell behind the stamps that is never written in practice
    if (kind == 0) hipLaunchKernelGGL(matrix_core_rate_kernel<0>, dim3(256), dim3(512), 0, s, iters, random_operands, stamps, sink);
    else
        hipLaunchKernelGGL(matrix_core_rate_kernel<1>, dim3(256), dim3(512), 0, s, iters, random_operands, stamps, sink);
    return hipGetLastError();
}
} // namespace mme
