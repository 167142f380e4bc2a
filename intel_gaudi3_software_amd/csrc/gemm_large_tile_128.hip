// gemm_large_tile_128.hip -- the large-tile contraction kernels with 128 x 256 output tiles, for problems whose 256 x 256
// tiles would occupy at most half of the compute units (a 3 x 3 dedx of 32 x 28 x 28 x 256: 98 tiles on 256 units).  Same
// body (gemm_large_tile_impl.hpp): a wavefront owns 64 x 64 outputs, a stage is 8 KiB of A + 16 KiB of B, four MFMAs and
// three DMA requests per wavefront and stage.  2-byte operands (bf16, IEEE half); A plain rows, the convolution gather of
// fwd / dedx, or the pixels-along-k view of dedw (whose split-k workspace halves with twice the tiles at half the slices).
#include "gemm_large_tile_impl.hpp"

namespace mme
{
namespace
{
template<int FMT, bool B_KC>
__global__ __launch_bounds__(512) void gemm_2byte_fast128_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, FMT, B_KC, 0, 128>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT, bool B_KC>
__global__ __launch_bounds__(512) void conv_2byte_fast128_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, FMT, B_KC, 1, 128>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT>
__global__ __launch_bounds__(512) void conv_dedw_2byte_fast128_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, FMT, false, 3, 128>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT>
hipError_t launch_128(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[5] = {false, false, false, false, false};
    const bool  bkc = p.B.k_contig != 0;
    if (p.A.kind == VIEW_CONV && !p.A.pix_is_f) return launch_fast(conv_dedw_2byte_fast128_kernel<FMT>, attr_done[4], p, grid, s, 128);
    if (p.A.kind == VIEW_CONV)
        return bkc ? launch_fast(conv_2byte_fast128_kernel<FMT, true>, attr_done[0], p, grid, s, 128)
                   : launch_fast(conv_2byte_fast128_kernel<FMT, false>, attr_done[1], p, grid, s, 128);
    return bkc ? launch_fast(gemm_2byte_fast128_kernel<FMT, true>, attr_done[2], p, grid, s, 128)
               : launch_fast(gemm_2byte_fast128_kernel<FMT, false>, attr_done[3], p, grid, s, 128);
}
} // namespace

hipError_t launch_gemm_large_tile_128(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    return p.dtype == DT_FP16 ? launch_128<1>(p, grid, s) : launch_128<0>(p, grid, s);
}
} // namespace mme
