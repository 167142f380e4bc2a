// gemm_large_tile_persistent_chk.hip -- the walking fp8 GEMM (gemm_large_tile_persistent.hip) in the variant that checks its
// own operands for codes the hardware's fp8 formats read differently from Gaudi's (gemm_large_tile_impl.hpp, CHK).
// Replaces, for these shapes, doGemmWorkerFloat + Gaudi3Fp8Fma::fma_vec of the reference
// (mme/mme_reference/mme_reference_impl.cpp:1022-1053, chip_fma/gaudi3_fma.cpp:70-144).
#include "gemm_large_tile_impl.hpp"

namespace mme
{
namespace
{
constexpr int PERSIST_WGS = 256;
constexpr int PERSIST_LDS = FNST * FSTAGE + 32 * 1024;

template<int FMT, bool B_KC>
__global__ __launch_bounds__(512) void gemm_fp8_persistent_chk_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<1, FMT, B_KC, 0, FBM, false, true, true>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<class K>
hipError_t launch_persistent(K kernel, bool& attr_done, const GemmProblem& p, hipStream_t s)
{
    if (!attr_done)
    {
        hipError_t e = hipFuncSetAttribute((const void*) kernel, hipFuncAttributeMaxDynamicSharedMemorySize, PERSIST_LDS);
        if (e != hipSuccess) return e;
        attr_done = true;
    }
    hipLaunchKernelGGL(kernel, dim3(PERSIST_WGS), dim3(512), PERSIST_LDS, s, p);
    return hipGetLastError();
}

template<int FMT>
hipError_t launch_fmt(const GemmProblem& p, hipStream_t s)
{
    static bool attr_done[2] = {false, false};
    return p.B.k_contig ? launch_persistent(gemm_fp8_persistent_chk_kernel<FMT, true>, attr_done[0], p, s)
                        : launch_persistent(gemm_fp8_persistent_chk_kernel<FMT, false>, attr_done[1], p, s);
}
} // namespace

hipError_t launch_gemm_large_tile_persistent_chk(const GemmProblem& p, hipStream_t s)
{
    switch ((p.fmt_a & 1) | ((p.fmt_b & 1) << 1))
    {
        case 0: return launch_fmt<0>(p, s);
        case 1: return launch_fmt<1>(p, s);
        case 2: return launch_fmt<2>(p, s);
        default: return launch_fmt<3>(p, s);
    }
}
} // namespace mme
