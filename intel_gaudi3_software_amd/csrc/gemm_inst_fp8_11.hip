// gemm_inst_fp8_11.hip -- instantiates the contraction kernel for one operand type (four memory layouts).
#include "gemm_impl.hpp"
namespace mme
{
void launch_gemm_fp8_11(const GemmProblem& p, dim3 grid, hipStream_t s) { launch_layout<1, 3>(p, grid, s); }
} // namespace mme
