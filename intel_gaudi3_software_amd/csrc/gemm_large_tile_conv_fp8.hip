// gemm_large_tile_conv_fp8.hip -- the large-tile kernel gathering a forward convolution or a dedx on its load side, fp8
// operands (both Gaudi flavours on either side): a stage is one filter tap x 64 channels, so the channel count has to be
// a multiple of 64.  Same body as the 2-byte gather (gemm_large_tile_impl.hpp, AMODE 1) with the fp8 matrix instruction,
// with 256-row tiles or, when those would occupy at most half of the compute units, 128-row ones.  The file also holds the
// plain fp8 GEMM (A k-contiguous) with 128-row tiles, for the same situation.
#include "gemm_large_tile_impl.hpp"

namespace mme
{
namespace
{
template<int FMT, bool B_KC, int TM>
__global__ __launch_bounds__(512) void conv_fp8_fast_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<1, FMT, B_KC, 1, TM>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT, bool B_KC>
__global__ __launch_bounds__(512) void gemm_fp8_fast128_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<1, FMT, B_KC, 0, 128>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT, int TM>
hipError_t launch_tm(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[2] = {false, false};
    return p.B.k_contig ? launch_fast(conv_fp8_fast_kernel<FMT, true, TM>, attr_done[0], p, grid, s, TM)
                        : launch_fast(conv_fp8_fast_kernel<FMT, false, TM>, attr_done[1], p, grid, s, TM);
}

template<int FMT>
hipError_t launch_fmt(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[2] = {false, false};
    if (p.A.kind != VIEW_CONV)
        return p.B.k_contig ? launch_fast(gemm_fp8_fast128_kernel<FMT, true>, attr_done[0], p, grid, s, 128)
                            : launch_fast(gemm_fp8_fast128_kernel<FMT, false>, attr_done[1], p, grid, s, 128);
    return p.tile_m == 128 ? launch_tm<FMT, 128>(p, grid, s) : launch_tm<FMT, 256>(p, grid, s);
}
} // namespace

hipError_t launch_gemm_large_tile_conv_fp8(const GemmProblem& p, dim3 grid, hipStream_t s)
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
