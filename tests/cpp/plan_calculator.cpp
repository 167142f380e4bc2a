// The planner through the C++ surface (MmeHip::Calculator::planBatchGemm / planConvolution): which kernel form a call would
// launch, asked from descriptors alone.  Needs no GPU: nothing is launched, the data pointers are never dereferenced.
// Prints one line per case and exits non-zero on the first failure.
#include "mme_hip_calculator.h"

#include <cstdio>
#include <cstring>

using MmeHip::Calculator;
using MmeHip::ConvolutionParams;
using MmeHip::MMEStackException;
using MmeHip::Tensor;
typedef Tensor::SizeArray SizeArray;

static int failures = 0;
#define EXPECT(cond)                                                                  \
    do                                                                                \
    {                                                                                 \
        if (!(cond))                                                                  \
        {                                                                             \
            std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);           \
            failures++;                                                               \
        }                                                                             \
    } while (0)

static void* const ALIGNED = (void*) (uintptr_t) 4096; // stands in for a device address

int main()
{
    {
        // the fp8 4096^3 GEMM with a fused bf16 output: one round of 256 x 256 tiles, four wavefronts of 128 x 128 outputs
        Tensor           a({4096, 4096, 1, 1, 1}, 2, MME_HIP_FP8_143, ALIGNED, 7), b({4096, 4096, 1, 1, 1}, 2, MME_HIP_FP8_143, ALIGNED, 7),
            y({4096, 4096, 1, 1, 1}, 2, MME_HIP_BF16, ALIGNED);
        mme_hip_epilogue e;
        std::memset(&e, 0, sizeof e);
        e.scale_exp = -10;
        e.clip_fp = 1;
        const Calculator::Form f = Calculator::planBatchGemm(y, a, b, MME_HIP_OP_AB, &e);
        EXPECT(f.largeTile == 1 && f.tileRows == 256 && f.splitK == 1 && f.wavefronts == 4);
        std::printf("ok    fp8 4096^3 -> bf16: large tile %d, rows %d, slices %d, wavefronts %d\n", f.largeTile, f.tileRows, f.splitK, f.wavefronts);
    }
    {
        // dedw of the 3 x 3 layer 32 x 28 x 28 x 256 -> 256: 128-row tiles, the reduction over the pixels in 14 slices
        Tensor            x({256, 28, 28, 1, 32}, 5, MME_HIP_BF16, ALIGNED), dy({256, 28, 28, 1, 32}, 5, MME_HIP_BF16, ALIGNED),
            dw({256, 256, 3, 3, 1}, 5, MME_HIP_FP32, ALIGNED);
        ConvolutionParams p;
        p.dim = 2;
        p.padding[0] = p.padding[1] = 1;
        const Calculator::Form f = Calculator::planConvolution(dw, x, dw, dy, p, MME_HIP_OP_DEDW);
        EXPECT(f.largeTile == 1 && f.tileRows == 128 && f.splitK == 14 && f.wavefronts == 8);
        std::printf("ok    bf16 dedw: large tile %d, rows %d, slices %d\n", f.largeTile, f.tileRows, f.splitK);
    }
    {
        // one odd dimension: K = 4100 leaves the large-tile kernels
        Tensor a({4100, 4096, 1, 1, 1}, 2, MME_HIP_BF16, ALIGNED), b({4096, 4100, 1, 1, 1}, 2, MME_HIP_BF16, ALIGNED), y({4096, 4096, 1, 1, 1}, 2, MME_HIP_FP32, ALIGNED);
        const Calculator::Form f = Calculator::planBatchGemm(y, a, b, MME_HIP_OP_AB);
        EXPECT(f.largeTile == 0);
        std::printf("ok    bf16 4096 x 4096 x 4100: large tile %d\n", f.largeTile);
    }
    {
        // refused like the real call, with the reference's message
        Tensor a({512, 512, 1, 1, 1}, 2, MME_HIP_BF16, ALIGNED), b({512, 500, 1, 1, 1}, 2, MME_HIP_BF16, ALIGNED), y({512, 512, 1, 1, 1}, 2, MME_HIP_FP32, ALIGNED);
        bool thrown = false;
        try
        {
            Calculator::planBatchGemm(y, a, b, MME_HIP_OP_AB);
        }
        catch (const MMEStackException& ex)
        {
            thrown = std::strstr(ex.what(), "Common dim") != nullptr;
        }
        EXPECT(thrown);
        std::printf("ok    mismatching common dimension refused\n");
    }
    std::printf(failures ? "%d FAILED\n" : "all ok\n", failures);
    return failures ? 1 : 0;
}
