// gemm_large_tile_ragged.hip -- the large-tile GEMM kernels for shapes that are not whole tiles: any M from 64 rows, N any
// multiple of 16 from 128 columns (plain operands, A k-contiguous: the "ab" and "abt" forms).  Same body
// (gemm_large_tile_impl.hpp) instantiated with RG: the loads of a partial tile are clamped to the operand's last row or
// last 16-byte chunk, its stores are predicated.  256- or 128-row tiles.
#include "gemm_large_tile_impl.hpp"

namespace mme
{
namespace
{
template<int FMT, bool B_KC, int TM>
__global__ __launch_bounds__(512) void gemm_fp8_ragged_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<1, FMT, B_KC, 0, TM, true>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT, bool B_KC, int TM>
__global__ __launch_bounds__(512) void gemm_2byte_ragged_kernel(GemmProblem g_by_value)
{
    (void) g_by_value;
    gemm_fast_body<2, FMT, B_KC, 0, TM, true>(*(KARG GemmProblem*) __builtin_amdgcn_kernarg_segment_ptr());
}

template<int FMT, int TM>
hipError_t launch_fp8_tm(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[2] = {false, false};
    return p.B.k_contig ? launch_fast(gemm_fp8_ragged_kernel<FMT, true, TM>, attr_done[0], p, grid, s, TM)
                        : launch_fast(gemm_fp8_ragged_kernel<FMT, false, TM>, attr_done[1], p, grid, s, TM);
}

template<int FMT>
hipError_t launch_fp8(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    return p.tile_m == 128 ? launch_fp8_tm<FMT, 128>(p, grid, s) : launch_fp8_tm<FMT, 256>(p, grid, s);
}

template<int FMT, int TM>
hipError_t launch_2byte(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    static bool attr_done[2] = {false, false};
    return p.B.k_contig ? launch_fast(gemm_2byte_ragged_kernel<FMT, true, TM>, attr_done[0], p, grid, s, TM)
                        : launch_fast(gemm_2byte_ragged_kernel<FMT, false, TM>, attr_done[1], p, grid, s, TM);
}
} // namespace

hipError_t launch_gemm_large_tile_ragged(const GemmProblem& p, dim3 grid, hipStream_t s)
{
    const bool t128 = p.tile_m == 128;
    if (p.dtype == DT_FP16) return t128 ? launch_2byte<1, 128>(p, grid, s) : launch_2byte<1, 256>(p, grid, s);
    if (p.dtype == DT_BF16) return t128 ? launch_2byte<0, 128>(p, grid, s) : launch_2byte<0, 256>(p, grid, s);
    switch ((p.fmt_a & 1) | ((p.fmt_b & 1) << 1))
    {
        case 0: return launch_fp8<0>(p, grid, s);
        case 1: return launch_fp8<1>(p, grid, s);
        case 2: return launch_fp8<2>(p, grid, s);
        default: return launch_fp8<3>(p, grid, s);
    }
}
} // namespace mme
