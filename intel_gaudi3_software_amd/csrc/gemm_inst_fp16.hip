// gemm_inst_fp16.hip -- instantiates the contraction kernel for one operand type (four memory layouts).
#include "gemm_impl.hpp"
namespace mme
{
void launch_gemm_fp16(const GemmProblem& p, dim3 grid, hipStream_t s) { launch_layout<2, 1>(p, grid, s); }
} // namespace mme
