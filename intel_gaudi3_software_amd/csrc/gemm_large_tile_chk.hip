// gemm_large_tile_chk.hip -- the large-tile fp8 GEMM (one workgroup per 256 x 256 tile) in the variant that checks its own
// operands for codes the hardware's fp8 formats read differently from Gaudi's (gemm_large_tile_impl.hpp, CHK): fp8_143 in
// full inf/NaN mode keeps exponent 15 for inf / NaN (fs_fma.cpp:6090-6100) where OCP e4m3 has 256 .. 448, and so on.  A clean
// operand, the usual case, then costs neither a scan launch nor a pass over memory.  A hit either raises the call's flag,
// and the exact fall-back enqueued behind this kernel rewrites the output, or -- when the tiles make one round and the host
// says so (GemmProblem::chk == 2) -- is noted in the launch's panel words, and the workgroups whose tiles it touches compute
// them once more, exactly, before the launch ends.
// Replaces, for these shapes, doGemmWorkerFloat + Gaudi3Fp8Fma::fma_vec of the reference
// (mme/mme_reference/mme_reference_impl.cpp:1022-1053, chip_fma/gaudi3_fma.cpp:70-144).
#include "gemm_large_tile_impl.hpp"

namespace mme
{
namespace
{
template<int FMT, bool B_KC>
__global__ __launch_bounds__(512) void gemm_fp8_fast_chk_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<1, FMT, B_KC, 0, FBM, false, false, true>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT>
hipError_t launch_fmt(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[2] = {false, false};
    return p.B.k_contig ? launch_fast(gemm_fp8_fast_chk_kernel<FMT, true>, attr_done[0], p, grid, s)
                        : launch_fast(gemm_fp8_fast_chk_kernel<FMT, false>, attr_done[1], p, grid, s);
}
} // namespace

hipError_t launch_gemm_large_tile_chk(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    switch ((p.fmt_a & 1) | ((p.fmt_b & 1) << 1))
    {
        case 0: return launch_fmt<0>(p, grid, s);
        case 1: return launch_fmt<1>(p, grid, s);
        case 2: return launch_fmt<2>(p, grid, s);
        default: return launch_fmt<3>(p, grid, s);
    }
}
} // namespace mme
