// gemm_large_tile_w4.hip -- the large-tile fp8 GEMM (one workgroup per 256 x 256 tile) with four wavefronts of 128 x 128
// outputs each instead of eight of 128 x 64 (gemm_large_tile_impl.hpp, NW = 4): one wavefront per SIMD with its 256
// accumulator registers in the upper half of the 512-register file.  A stage then takes 64 KiB of fragment reads from LDS
// instead of 96 KiB and half as many read instructions per matrix instruction; what the second wavefront of a SIMD
// covered (LDS latency, the wait for a stage, the barrier) has to be covered by the distance between a fragment's read and
// its use inside the one instruction stream.  Both operand policies: plain, and with the in-kernel look at the operand
// bytes (CHK).
// Replaces, for these shapes, doGemmWorkerFloat + Gaudi3Fp8Fma::fma_vec of the reference
// (mme/mme_reference/mme_reference_impl.cpp:1022-1053, chip_fma/gaudi3_fma.cpp:70-144).
#include "gemm_large_tile_impl.hpp"

namespace mme
{
namespace
{
template<int FMT, bool B_KC, bool CHK>
__global__ __launch_bounds__(256) void gemm_fp8_w4_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<1, FMT, B_KC, 0, FBM, false, false, CHK, FNST, 4>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT, bool CHK>
hipError_t launch_fmt(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[2] = {false, false};
    return p.B.k_contig ? launch_fast(gemm_fp8_w4_kernel<FMT, true, CHK>, attr_done[0], p, grid, s, FBM, FNST, 256)
                        : launch_fast(gemm_fp8_w4_kernel<FMT, false, CHK>, attr_done[1], p, grid, s, FBM, FNST, 256);
}

template<bool CHK>
hipError_t launch_chk(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    switch ((p.fmt_a & 1) | ((p.fmt_b & 1) << 1))
    {
        case 0: return launch_fmt<0, CHK>(p, grid, s);
        case 1: return launch_fmt<1, CHK>(p, grid, s);
        case 2: return launch_fmt<2, CHK>(p, grid, s);
        default: return launch_fmt<3, CHK>(p, grid, s);
    }
}
} // namespace

hipError_t launch_gemm_large_tile_w4(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    return p.chk ? launch_chk<true>(p, grid, s) : launch_chk<false>(p, grid, s);
}
} // namespace mme
