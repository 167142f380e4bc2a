// gemm_large_tile_fp8_at.hip -- the large-tile kernel for fp8 operands whose A is contiguous along the tile's rows: the
// "atb" / "atbt" GEMM forms (AMODE 2) and dedw, whose pixels run along k (AMODE 3).  The A stage then has the layout of an
// n-contiguous fp8 B (64 k-rows x 256 bytes) and is read with the transposing ds_read_b64_tr_b8.  256-row tiles.
#include "gemm_large_tile_impl.hpp"

namespace mme
{
namespace
{
template<int FMT, bool B_KC>
__global__ __launch_bounds__(512) void gemm_fp8_at_fast_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<1, FMT, B_KC, 2>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT>
__global__ __launch_bounds__(512) void conv_dedw_fp8_fast_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<1, FMT, false, 3>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT>
hipError_t launch_fmt(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[3] = {false, false, false};
    if (p.A.kind == VIEW_CONV) return launch_fast(conv_dedw_fp8_fast_kernel<FMT>, attr_done[2], p, grid, s);
    return p.B.k_contig ? launch_fast(gemm_fp8_at_fast_kernel<FMT, true>, attr_done[0], p, grid, s)
                        : launch_fast(gemm_fp8_at_fast_kernel<FMT, false>, attr_done[1], p, grid, s);
}
} // namespace

hipError_t launch_gemm_large_tile_fp8_at(const GemmProblem& p, dim3 grid, hipStream_t s)
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
