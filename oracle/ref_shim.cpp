// ref_shim.cpp -- extern "C" access to the UNMODIFIED reference calculator, for tests and the CPU baseline only.
//
// This file is compiled together with the reference's own translation units, taken from where they lie in the
// reference tree, into oracle/_ref/libmme_ref.so (see oracle/Makefile).  It holds no reference code: it only calls
// the reference's public classes and free functions and exposes them with the same PODs the product's C ABI uses,
// so that one test can hand the same descriptors to the oracle restatement (orc_*), to the compiled reference
// (ref_*) and to the HIP library (mme_hip_*).
//
// TEST INFRASTRUCTURE ONLY; the product library never links it.
#include <cstdint>
#include <cstring>
#include <exception>
#include <memory>
#include <string>
#include <cstdio>
#include <iostream>
#include <fcntl.h>
#include <unistd.h>

#include "mme_reference.h"             // CPUCalculator, MmeSimTensor, ConvolutionParams
#include "tensor_comparator.h"         // TensorComparator
#include "chip_fma/chip_fma.h"         // ChipFma::getChipFma
#include "fs_fma_gaudi3.h"             // gaudi3:: converters and trees
#include "../include/mme_hip.h"        // PODs shared with the product ABI

using namespace MmeCommon;

static thread_local std::string g_err;
static unsigned                 g_threads = 0;

static MmeSimTensor wrap(const mme_hip_tensor* t)
{
    SizeArray sizes, strides;
    for (int d = 0; d < 5; d++)
    {
        sizes[d] = t->sizes[d];
        strides[d] = t->strides[d];
    }
    // SizeArray constructor wraps caller memory without copying (sim_tensor.cpp:19-20)
    return MmeSimTensor(sizes, t->dim, (EMmeDataType) t->dtype, (char*) t->data, t->fp_bias,
                        (InfNanMode) t->inf_nan_mode, &strides);
}

static ConvolutionParams conv(const mme_hip_conv_params* p)
{
    ConvolutionParams c;
    c.dim = p->dim;
    c.paddingValue.int32 = p->padding_value;
    for (int i = 0; i < 4; i++)
    {
        c.padding[i] = p->padding[i];
        c.convStride[i] = p->conv_stride[i];
        c.dilation[i] = p->dilation[i];
    }
    c.relu = p->relu != 0;
    return c;
}

template<typename F>
static int guarded(F&& f)
{
    try
    {
        f();
        return 0;
    }
    catch (const std::exception& e)
    {
        g_err = e.what();
        return -1;
    }
}

extern "C" {

const char* ref_last_error(void) { return g_err.c_str(); }
void        ref_set_num_threads(int n) { g_threads = (unsigned) n; }

int ref_batch_gemm(const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w, int op)
{
    return guarded([&] {
        CPUCalculator calc(e_mme_Gaudi3);
        calc.limitNumOfThreads(g_threads);
        MmeSimTensor o = wrap(out), a = wrap(x), b = wrap(w);
        calc.doBatchGemm(o, a, b, (EMmeOpType) op);
    });
}

int ref_batch_gemm_clip(const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w, int op, int clip,
                        int clip_inf_in)
{
    return guarded([&] {
        CPUCalculator calc(e_mme_Gaudi3);
        calc.limitNumOfThreads(g_threads);
        MmeSimTensor o = wrap(out), a = wrap(x), b = wrap(w);
        calc.doBatchGemm(o, a, b, (EMmeOpType) op, RoundToNearest, clip != 0, clip_inf_in != 0);
    });
}

int ref_convolution(const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w,
                    const mme_hip_tensor* y, const mme_hip_conv_params* p, int op, int rm)
{
    return guarded([&] {
        CPUCalculator calc(e_mme_Gaudi3);
        calc.limitNumOfThreads(g_threads);
        MmeSimTensor o = wrap(out), a = wrap(x), b = wrap(w), c = wrap(y);
        calc.doConvolution(o, a, b, c, conv(p), (EMmeOpType) op, (RoundingMode) rm);
        // fwd / dedw replace the tensor's buffer (mme_reference_impl.cpp:862-868): copy the result back into
        // the caller's memory so that all three implementations are compared through out->data
        if ((void*) o.data() != out->data) memcpy(out->data, o.data(), o.getMemorySize());
    });
}

int ref_activation(const mme_hip_tensor* out, const mme_hip_tensor* acc, int relu, int rm, int clip, int clip_inf_in,
                   int ftz, int sftz, uint32_t* lfsr, uint32_t polynomial, uint32_t lfsr_regs)
{
    return guarded([&] {
        // polynomial 0 asks the reference to draw one from its seed; the shim always passes an explicit one
        CPUCalculator calc(e_mme_Gaudi3, MME_MAX_TENSOR_DIMS, MME_MAX_CONV_DIMS, 0, lfsr ? lfsr_regs : 256, lfsr,
                           polynomial ? polynomial : 1);
        auto o = std::make_shared<MmeSimTensor>(wrap(out));
        auto a = std::make_shared<MmeSimTensor>(wrap(acc));
        calc.doActivation(o, a, nullptr, nullptr, relu != 0, (RoundingMode) rm, nullptr, clip != 0, clip_inf_in != 0,
                          ftz != 0, sftz != 0);
    });
}

// ---- scalar functions, in bulk so that sweeps over millions of inputs stay fast from Python ---------------------

void ref_fp32_to_fp8_n(uint8_t* out, const uint32_t* in, size_t n, int E, int M, int bias, int rm, const uint32_t* lfsr,
                       int ftz, int clip, int clip_inf_in, int sftz, int mode)
{
    for (size_t i = 0; i < n; i++)
    {
        float f;
        memcpy(&f, &in[i], 4);
        out[i] = gaudi3::fp32_to_fp8(f, E, M, bias, rm, lfsr ? lfsr[i] : 0, ftz, clip, clip_inf_in, sftz, mode);
    }
}

void ref_fp8_to_fp32_n(uint32_t* out, const uint8_t* in, size_t n, int E, int M, int bias, int mode)
{
    for (size_t i = 0; i < n; i++) out[i] = gaudi3::fp8_to_fp32(in[i], E, M, bias, false, false, mode);
}

void ref_fp32_to_bf16_n(uint16_t* out, const uint32_t* in, size_t n, int rm, const uint32_t* lfsr, int clip, int ftz,
                        int clip_inf_in)
{
    for (size_t i = 0; i < n; i++)
    {
        float f;
        memcpy(&f, &in[i], 4);
        out[i] = gaudi3::fp32_to_bf16(f, rm, lfsr ? lfsr[i] : 0, clip, ftz, clip_inf_in);
    }
}

void ref_fp32_to_fp32_n(uint32_t* out, const uint32_t* in, size_t n, int rm, int clip, int ftz, int clip_inf_in)
{
    for (size_t i = 0; i < n; i++)
    {
        float f;
        memcpy(&f, &in[i], 4);
        out[i] = gaudi3::fp32_to_fp32(f, rm, clip, ftz, clip_inf_in);
    }
}

void ref_add_fp32_n(uint32_t* out, const uint32_t* a, const uint32_t* b, size_t n, int rm)
{
    for (size_t i = 0; i < n; i++) out[i] = gaudi3::add_fp32(a[i], b[i], rm);
    gaudi3::set_rounding_mode(0);
}

uint32_t ref_lfsr32(uint32_t prev, uint32_t poly) { return gaudi3::mme_lfsr32(prev, poly); }

// n trees over rows of 9 (a, b) pairs each, a[8] = accumulator, b[8] = 1.0f
void ref_tree9_n(uint32_t* out, const uint32_t* a, const uint32_t* b, size_t n, int fp32_emul)
{
    for (size_t i = 0; i < n; i++)
    {
        uint32_t ta[9], tb[9];
        memcpy(ta, a + 9 * i, sizeof ta);
        memcpy(tb, b + 9 * i, sizeof tb);
        // emulation kind 0: bf16 / fp8, 1: fp32 byte slices, 2: fp16 / tf32 slices (the flag sets of fs_fma.cpp)
        out[i] = fp32_emul == 2   ? gaudi3::fma_mul_add_tree_n(ta, tb, 0, gaudi3::RND_TO_0, 9, 4, 1, 1, 0, 1, 1, 0, 0, 1)
                 : fp32_emul == 1 ? gaudi3::fma_mul_add_tree_n(ta, tb, 0, gaudi3::RND_TO_0, 9, 4, 1, 1, 0, 0, 1, 0, 0, 1)
                                  : gaudi3::fma_mul_add_tree_n(ta, tb, 0, gaudi3::RND_TO_0, 9, 4, 0, 1, 0, 0, 0, 0, 0, 1);
    }
}

// ChipFma::fma_vec for one dot product (dense operands)
uint32_t ref_fma_vec(const void* a, const void* b, unsigned cd, int type_a, int type_b, unsigned bias_a,
                     unsigned bias_b, int mode_a, int mode_b)
{
    auto  fma = ChipFma::getChipFma(e_mme_Gaudi3, (EMmeDataType) type_a, (EMmeDataType) type_b, bias_a, bias_b,
                                    RoundToNearest, RoundToNearest, false, false, (InfNanMode) mode_a, (InfNanMode) mode_b);
    float v = fma->fma_vec(a, b, cd);
    uint32_t u;
    memcpy(&u, &v, 4);
    return u;
}

// ChipFma::fma_vec with the clipFp / clipFpInfIn flags, which the tf32 flavour reads
uint32_t ref_fma_vec_clip(const void* a, const void* b, unsigned cd, int type_a, int type_b, unsigned bias_a,
                          unsigned bias_b, int mode_a, int mode_b, int clip, int clip_inf_in)
{
    auto  fma = ChipFma::getChipFma(e_mme_Gaudi3, (EMmeDataType) type_a, (EMmeDataType) type_b, bias_a, bias_b,
                                    RoundToNearest, RoundToNearest, clip != 0, clip_inf_in != 0, (InfNanMode) mode_a,
                                    (InfNanMode) mode_b);
    float v = fma->fma_vec(a, b, cd);
    uint32_t u;
    memcpy(&u, &v, 4);
    return u;
}

void ref_fp32_to_cfp16_n(uint16_t* out, const uint32_t* in, size_t n, int E, int bias, int rm, const uint32_t* lfsr,
                         int ftz, int clip, int clip_inf_in, int no_inf_nan)
{
    for (size_t i = 0; i < n; i++)
    {
        float f;
        memcpy(&f, &in[i], 4);
        out[i] = gaudi3::fp32_to_cfp16(f, E, 10, bias, rm, lfsr ? lfsr[i] : 0, ftz, clip, clip_inf_in, no_inf_nan != 0);
    }
}

void ref_cfp16_to_fp32_n(uint32_t* out, const uint16_t* in, size_t n, int E, int bias, int no_inf_nan)
{
    for (size_t i = 0; i < n; i++) out[i] = gaudi3::cfp16_to_fp32(in[i], E, 10, bias, false, false, no_inf_nan != 0);
}

void ref_fp32_to_tf32_n(uint32_t* out, const uint32_t* in, size_t n, int clip, int clip_inf_in)
{
    for (size_t i = 0; i < n; i++)
    {
        float f;
        memcpy(&f, &in[i], 4);
        out[i] = gaudi3::fp32_to_tf32(f, 0, 0, clip != 0, clip_inf_in != 0);
    }
}

// TensorComparator::doCompare on n one-element tensors (the rule element by element): ok[i] = 1 when a[i] and b[i] are
// accepted.  The comparator reports every mismatch on stdout; that is sent to /dev/null for the duration of the call.
void ref_compare_elements(uint8_t* ok, const void* a, const void* b, size_t n, int dtype, unsigned bias, int mode, unsigned cd_size)
{
    fflush(stdout);
    std::cout.flush();
    const int saved = dup(1), devnull = open("/dev/null", O_WRONLY);
    dup2(devnull, 1);
    TensorComparator cmp(cd_size, (EMmeDataType) dtype, bias, (InfNanMode) mode);
    const size_t     es = dtype == e_type_fp8_143 || dtype == e_type_fp8_152 ? 1 : (dtype == e_type_fp32 || dtype == e_type_fp32_ieee ? 4 : 2);
    SizeArray        one = {1, 1, 1, 1, 1};
    for (size_t i = 0; i < n; i++)
    {
        auto ta = std::make_shared<MmeSimTensor>(one, 1, (EMmeDataType) dtype, (char*) a + i * es, bias, (InfNanMode) mode);
        auto tb = std::make_shared<MmeSimTensor>(one, 1, (EMmeDataType) dtype, (char*) b + i * es, bias, (InfNanMode) mode);
        ok[i] = cmp.doCompare(ta, "a", tb, "b", 0, "", 1, false) ? 1 : 0;
    }
    fflush(stdout);
    std::cout.flush();
    dup2(saved, 1);
    close(saved);
    close(devnull);
}

// whole tensors: returns 1 when equal, else 0 with the coordinates of the first mismatch in diff[5]
int ref_compare_tensors(const mme_hip_tensor* a, const mme_hip_tensor* b, unsigned cd_size, int bit_exact, uint32_t* diff)
{
    fflush(stdout);
    std::cout.flush();
    const int saved = dup(1), devnull = open("/dev/null", O_WRONLY);
    dup2(devnull, 1);
    TensorComparator cmp(cd_size, (EMmeDataType) a->dtype, a->fp_bias, (InfNanMode) a->inf_nan_mode);
    auto             ta = std::make_shared<MmeSimTensor>(wrap(a));
    auto             tb = std::make_shared<MmeSimTensor>(wrap(b));
    const bool       eq = bit_exact ? cmp.doCompareBitExact(ta, "a", tb, "b") : cmp.doCompare(ta, "a", tb, "b", 0, "", 1, false);
    if (!eq)
    {
        auto d = cmp.getDiffElement();
        if (d.is_set())
            for (int i = 0; i < 5; i++) diff[i] = d.value()[i];
    }
    fflush(stdout);
    std::cout.flush();
    dup2(saved, 1);
    close(saved);
    close(devnull);
    return eq ? 1 : 0;
}

// the partial-sum rule element by element: a holds n groups of num_partials partial values, b n sums; ok[i] = 1 when group i
// is accepted against b[i]
void ref_compare_elements_partials(uint8_t* ok, const void* a, const void* b, size_t n, unsigned num_partials, int dtype, unsigned bias, int mode,
                                   unsigned cd_size)
{
    fflush(stdout);
    std::cout.flush();
    const int saved = dup(1), devnull = open("/dev/null", O_WRONLY);
    dup2(devnull, 1);
    TensorComparator cmp(cd_size, (EMmeDataType) dtype, bias, (InfNanMode) mode);
    const size_t     es = dtype == e_type_fp8_143 || dtype == e_type_fp8_152 ? 1 : (dtype == e_type_fp32 || dtype == e_type_fp32_ieee ? 4 : 2);
    SizeArray        one = {1, 1, 1, 1, 1}, many = {num_partials, 1, 1, 1, 1};
    for (size_t i = 0; i < n; i++)
    {
        auto ta = std::make_shared<MmeSimTensor>(many, 1, (EMmeDataType) dtype, (char*) a + i * es * num_partials, bias, (InfNanMode) mode);
        auto tb = std::make_shared<MmeSimTensor>(one, 1, (EMmeDataType) dtype, (char*) b + i * es, bias, (InfNanMode) mode);
        ok[i] = cmp.doCompare(ta, "a", tb, "b", 0, "", num_partials, false) ? 1 : 0;
    }
    fflush(stdout);
    std::cout.flush();
    dup2(saved, 1);
    close(saved);
    close(devnull);
}

// doCompare with numPartials > 1: a holds num_partials partial results stacked along its last dimension, b their sum
int ref_compare_tensors_partials(const mme_hip_tensor* a, const mme_hip_tensor* b, unsigned cd_size, unsigned num_partials, uint32_t* diff)
{
    fflush(stdout);
    std::cout.flush();
    const int saved = dup(1), devnull = open("/dev/null", O_WRONLY);
    dup2(devnull, 1);
    TensorComparator cmp(cd_size, (EMmeDataType) a->dtype, a->fp_bias, (InfNanMode) a->inf_nan_mode);
    auto             ta = std::make_shared<MmeSimTensor>(wrap(a));
    auto             tb = std::make_shared<MmeSimTensor>(wrap(b));
    const bool       eq = cmp.doCompare(ta, "a", tb, "b", 0, "", num_partials, false);
    if (!eq)
    {
        auto d = cmp.getDiffElement();
        if (d.is_set())
            for (int i = 0; i < 5; i++) diff[i] = d.value()[i];
    }
    fflush(stdout);
    std::cout.flush();
    dup2(saved, 1);
    close(saved);
    close(devnull);
    return eq ? 1 : 0;
}

}  // extern "C"
