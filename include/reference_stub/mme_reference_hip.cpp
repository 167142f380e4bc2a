// mme_reference_hip.cpp -- the reference-side binding: a second implementation of CPUCalculator's forwarding methods
// (mme/mme_reference/mme_reference_impl.cpp:2174-2328) that sends every call to the MI355X library instead of
// CPUCalculatorImpl.  A maintainer drops this file next to mme_reference_impl.cpp, compiles it instead of the forwarding
// block there (e.g. under -DMME_REFERENCE_USE_HIP) with this repository's include/ on the include path, and links
// libmme_hip.so.  CPUCalculator is a pimpl over an incomplete CPUCalculatorImpl (mme_reference.h:107,190), so the header
// and every caller stay as they are.
//
// The reference's MmeSimTensor, Matrix and ConvolutionParams pass straight through: MmeHip::Calculator reads them only
// through the accessors the reference's own calculator uses.  Enum casts keep the values (include/mme_hip.h uses the
// reference's integers, mme_common_enum.h:25-102,191-197,321-342).
#include "mme_reference.h"

#include "mme_hip_calculator.h"

class CPUCalculatorImpl : public MmeHip::Calculator
{
public:
    using MmeHip::Calculator::Calculator;
};

// MME_ASSERT throws MmeCommon::MMEStackException in release builds (mme/include/mme_assert.h:19-58); callers that catch
// std::exception (MMETest::run, mme_test.cpp:31-35) see MmeHip::MMEStackException the same way, its text is the library's.

CPUCalculator::CPUCalculator(MmeCommon::ChipType chip, int max_tensor_dims, int max_conv_dims, unsigned seed, uint32_t lfsrNumRegs, uint32_t* lfsr,
                             uint32_t polynomial)
: m_impl(std::make_unique<CPUCalculatorImpl>((int) chip, max_tensor_dims, max_conv_dims, seed, lfsrNumRegs, lfsr, polynomial))
{
}
CPUCalculator::~CPUCalculator() = default;

void CPUCalculator::limitNumOfThreads(unsigned numOfThreads) { m_impl->limitNumOfThreads(numOfThreads); }

void CPUCalculator::doGemm(Matrix& output, const Matrix& inputA, const Matrix& inputB, bool transposeA, bool transposeB, MmeCommon::RoundingMode rm,
                           unsigned fpBiasA, unsigned fpBiasB, bool clipFp, bool clipFpInfIn, MmeCommon::InfNanMode infNanModeA,
                           MmeCommon::InfNanMode infNanModeB, int* zeroPoints)
{
    m_impl->doGemm(output, inputA, inputB, transposeA, transposeB, (int) rm, fpBiasA, fpBiasB, clipFp, clipFpInfIn, (int) infNanModeA, (int) infNanModeB,
                   zeroPoints);
}

void CPUCalculator::doDma(MmeSimTensor& outputTensor, const MmeSimTensor& xTensor, MmeCommon::EMmeOpType op)
{
    m_impl->doDma(outputTensor, xTensor, (int) op); // throws: not a contraction, not built
}

void CPUCalculator::doBatchGemm(MmeSimTensor& outputTensor, const MmeSimTensor& xTensor, const MmeSimTensor& wTensor, MmeCommon::EMmeOpType op,
                                MmeCommon::RoundingMode rm, bool clipFp, bool clipFpInfIn, int* zeroPoints)
{
    m_impl->doBatchGemm(outputTensor, xTensor, wTensor, (int) op, (int) rm, clipFp, clipFpInfIn, zeroPoints);
}

void CPUCalculator::doConvolution(MmeSimTensor& outputTensor, const MmeSimTensor& xTensor, const MmeSimTensor& wTensor, const MmeSimTensor& yTensor,
                                  const ConvolutionParams& params, MmeCommon::EMmeOpType op, MmeCommon::RoundingMode rm, bool clipFp, bool clipFpInfIn,
                                  int* zeroPoints)
{
    m_impl->doConvolution(outputTensor, xTensor, wTensor, yTensor, params, (int) op, (int) rm, clipFp, clipFpInfIn, zeroPoints);
}

void CPUCalculator::doActivation(pMMESimTensor output, const pMMESimTensor acc, const pMMESimTensor res, const pMMESimTensor bias, bool relu,
                                 MmeCommon::RoundingMode rm, const ActivationParams* actParams, bool clipFp, bool clipInfIn, bool flushDenorms,
                                 bool stochasticFTZfp8)
{
    m_impl->doActivation(output, acc, res, bias, relu, (int) rm, actParams, clipFp, clipInfIn, flushDenorms, stochasticFTZfp8);
}

void CPUCalculator::doMemoryWrite(pMMESimTensor memory, const pMMESimTensor mmeOut, MmeCommon::EMmeReductionOp reductionOp,
                                  MmeCommon::EMmeReductionRm reductionRm, bool clipFp)
{
    m_impl->doMemoryWrite(memory, mmeOut, (int) reductionOp, (int) reductionRm, clipFp);
}

void CPUCalculator::activationGemmlowp(pMMESimTensor out, pMMESimTensor acc, pMMESimTensor res, pMMESimTensor bias, bool reluEn,
                                       MmeCommon::RoundingMode roundingMode, const ActivationParams* actParams)
{
    m_impl->activationGemmlowp(out, acc, res, bias, reluEn, (int) roundingMode, actParams); // throws: integer path, not built
}
