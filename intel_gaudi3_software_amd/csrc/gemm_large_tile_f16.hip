// gemm_large_tile_f16.hip -- the large-tile contraction kernels for IEEE half operands (fp16 tensors in full inf/NaN mode; an
// exponent bias other than 15 is a power of two in the epilogue multiplier).  Same body as the bf16 kernels of
// gemm_large_tile.hip, with v_mfma_f32_32x32x16_f16 as the matrix-core instruction; kept in its own translation unit so
// that the two compile side by side.
#include "gemm_large_tile_impl.hpp"

namespace mme
{
namespace
{
template<bool B_KC, bool A_KC>
__global__ __launch_bounds__(512) void gemm_f16_fast_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, 1, B_KC, A_KC ? 0 : 2>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

// dedw: pixels along k for both operands, dY plain and n-contiguous
__global__ __launch_bounds__(512) void conv_dedw_f16_fast_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, 1, false, 3>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

// fwd / dedx: pixels along f, gathered through the convolution view
template<bool B_KC>
__global__ __launch_bounds__(512) void conv_f16_fast_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, 1, B_KC, 1>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}
} // namespace

hipError_t launch_gemm_large_tile_f16(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[7] = {false, false, false, false, false, false, false};
    const bool  bkc = p.B.k_contig != 0, akc = p.A.k_contig != 0;
    if (p.A.kind == VIEW_CONV && p.A.pix_is_f)
        return bkc ? launch_fast(conv_f16_fast_kernel<true>, attr_done[5], p, grid, s) : launch_fast(conv_f16_fast_kernel<false>, attr_done[6], p, grid, s);
    if (p.A.kind == VIEW_CONV) return launch_fast(conv_dedw_f16_fast_kernel, attr_done[4], p, grid, s);
    if (akc) return bkc ? launch_fast(gemm_f16_fast_kernel<true, true>, attr_done[0], p, grid, s)
                        : launch_fast(gemm_f16_fast_kernel<false, true>, attr_done[1], p, grid, s);
    return bkc ? launch_fast(gemm_f16_fast_kernel<true, false>, attr_done[2], p, grid, s)
               : launch_fast(gemm_f16_fast_kernel<false, false>, attr_done[3], p, grid, s);
}
} // namespace mme
