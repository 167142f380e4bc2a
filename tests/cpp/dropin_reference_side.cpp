// The genuine reference calculator under another name, for the drop-in demonstration of tests/cpp/dropin_reference_types.cpp:
// this file and the reference's mme_reference_impl.cpp are compiled with -DCPUCalculator=CPUCalculatorRef
// -DCPUCalculatorImpl=CPUCalculatorImplRef (oracle/Makefile, target ref_dropin), so that the reference's class and the one
// backed by the MI355X library live in one program and run on the same MmeSimTensor objects.
#include "convolution_params.h"
#include "mme_reference.h"
#include "sim_tensor.h"

void reference_side_batch_gemm(MmeSimTensor& y, const MmeSimTensor& a, const MmeSimTensor& b, MmeCommon::EMmeOpType op)
{
    CPUCalculator calc(MmeCommon::e_mme_Gaudi3, 5, 4);
    calc.doBatchGemm(y, a, b, op);
}

void reference_side_convolution(MmeSimTensor& out, const MmeSimTensor& x, const MmeSimTensor& w, const MmeSimTensor& y, const ConvolutionParams& p,
                                MmeCommon::EMmeOpType op)
{
    CPUCalculator calc(MmeCommon::e_mme_Gaudi3, 5, 4);
    calc.doConvolution(out, x, w, y, p, op);
}

void reference_side_activation(pMMESimTensor out, const pMMESimTensor acc, bool relu, MmeCommon::RoundingMode rm, bool clipFp)
{
    CPUCalculator calc(MmeCommon::e_mme_Gaudi3, 5, 4);
    calc.doActivation(out, acc, nullptr, nullptr, relu, rm, nullptr, clipFp);
}
