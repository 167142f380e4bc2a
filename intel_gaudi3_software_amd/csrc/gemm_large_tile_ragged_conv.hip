// gemm_large_tile_ragged_conv.hip -- the large-tile convolution kernels (2-byte operands) for output column counts that are
// not a multiple of 256: any multiple of 16 from 128 (fwd: K output channels, dedx: C, dedw: K).  Same body
// (gemm_large_tile_impl.hpp) instantiated with RG: weight / dY loads of the partial column tile are clamped, its stores
// predicated.  fwd / dedx gather the pixels on the load side (AMODE 1), dedw walks them along k (AMODE 3).
#include "gemm_large_tile_impl.hpp"

namespace mme
{
namespace
{
template<int FMT, bool B_KC, int TM>
__global__ __launch_bounds__(512) void conv_2byte_ragged_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, FMT, B_KC, 1, TM, true>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT, int TM>
__global__ __launch_bounds__(512) void conv_dedw_2byte_ragged_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, FMT, false, 3, TM, true>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT, int TM>
hipError_t launch_conv(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[3] = {false, false, false};
    if (!p.A.pix_is_f) return launch_fast(conv_dedw_2byte_ragged_kernel<FMT, TM>, attr_done[2], p, grid, s, TM);
    return p.B.k_contig ? launch_fast(conv_2byte_ragged_kernel<FMT, true, TM>, attr_done[0], p, grid, s, TM)
                        : launch_fast(conv_2byte_ragged_kernel<FMT, false, TM>, attr_done[1], p, grid, s, TM);
}
} // namespace

hipError_t launch_gemm_large_tile_ragged_conv(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    const bool t128 = p.tile_m == 128;
    if (p.dtype == DT_FP16) return t128 ? launch_conv<1, 128>(p, grid, s) : launch_conv<1, 256>(p, grid, s);
    return t128 ? launch_conv<0, 128>(p, grid, s) : launch_conv<0, 256>(p, grid, s);
}
} // namespace mme
