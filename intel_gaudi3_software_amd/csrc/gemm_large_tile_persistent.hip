// gemm_large_tile_persistent.hip -- the large-tile fp8 / bf16 GEMM for problems with several tiles per compute unit: 256
// workgroups walk over the tiles, and each requests the first stages of its next tile before it converts and stores the
// finished one, so that pipeline fill and epilogue overlap (gemm_large_tile_impl.hpp, PERSIST).
// Replaces, for these shapes, doGemmWorkerFloat + Gaudi3Fp8Fma::fma_vec of the reference
// (mme/mme_reference/mme_reference_impl.cpp:1022-1053, chip_fma/gaudi3_fma.cpp:70-144).
#include "gemm_large_tile_impl.hpp"

namespace mme
{
namespace
{
constexpr int PERSIST_WGS = 256;                          // one per compute unit of the MI355X
constexpr int PERSIST_LDS = FNST * FSTAGE + 32 * 1024;    // the ring + the epilogue's staging area

template<int FMT, bool B_KC>
__global__ __launch_bounds__(512) void gemm_fp8_persistent_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<1, FMT, B_KC, 0, FBM, false, true>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<bool B_KC>
__global__ __launch_bounds__(512) void gemm_bf16_persistent_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, 0, B_KC, 0, FBM, false, true>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
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
    return p.B.k_contig ? launch_persistent(gemm_fp8_persistent_kernel<FMT, true>, attr_done[0], p, s)
                        : launch_persistent(gemm_fp8_persistent_kernel<FMT, false>, attr_done[1], p, s);
}
} // namespace

// whole 256 x 256 tiles of a plain fp8 or bf16 GEMM with A k-contiguous, at least two rounds of tiles on a 256-CU device, fused
// bf16 / fp8 output through the fast converters, no split-k
bool gemm_large_tile_persistent_applicable(const GemmProblem& p)
{
    static int cus = 0;
    if (!cus)
    {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) cus = -1;
    }
    if (cus != PERSIST_WGS) return false;
    if (!(p.dtype == DT_FP8_143 || p.dtype == DT_FP8_152 || p.dtype == DT_BF16) || p.tile_m == 128 || p.split_k > 1) return false;
    if (p.A.kind != VIEW_PLAIN || p.B.kind != VIEW_PLAIN || !p.A.k_contig) return false;
    if (p.M % FBM || p.N % FBN) return false;
    if (!p.epi.fused || !p.epi.fast_cast) return false;
    if (!(p.epi.out_dtype == DT_BF16 || p.epi.out_dtype == DT_FP8_143 || p.epi.out_dtype == DT_FP8_152)) return false;
    const long long tiles = (long long) (p.M / FBM) * (p.N / FBN) * p.batch[0] * p.batch[1] * p.batch[2];
    return tiles >= 2 * PERSIST_WGS && tiles < (1ll << 30);
}

hipError_t launch_gemm_large_tile_persistent(const GemmProblem& p, hipStream_t s)
{
    if (p.dtype == DT_BF16)
    {
        static bool attr_done[2] = {false, false};
        return p.B.k_contig ? launch_persistent(gemm_bf16_persistent_kernel<true>, attr_done[0], p, s)
                            : launch_persistent(gemm_bf16_persistent_kernel<false>, attr_done[1], p, s);
    }
    switch ((p.fmt_a & 1) | ((p.fmt_b & 1) << 1))
    {
        case 0: return launch_fmt<0>(p, s);
        case 1: return launch_fmt<1>(p, s);
        case 2: return launch_fmt<2>(p, s);
        default: return launch_fmt<3>(p, s);
    }
}
} // namespace mme
