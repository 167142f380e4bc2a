/*
 * mme_hip_calculator.h -- the reference calculator's C++ surface over the C ABI of include/mme_hip.h.
 *
 * MmeHip::Calculator has the public methods of CPUCalculator (mme/mme_reference/mme_reference.h:108-191) with the same
 * argument order, defaults and error behaviour: a failed call throws MmeHip::MMEStackException with the library's
 * message, which is what MME_ASSERT does in the reference's release builds (mme/include/mme_assert.h:19-58).
 *
 * The methods are templates over the tensor type, so that they accept the reference's own MmeSimTensor /
 * MMESimTensorBase (mme/mme_reference/sim_tensor_base.h:55-158) without this header including it: the type only has
 * to offer data(), getSizes(), getStrides(), getDim(), getElementType(), getFpBias() and getInfNanMode(), which is how
 * the reference calculator itself reads a tensor (mme_reference_impl.cpp:454-462, 782-790).  MmeHip::Tensor below is a
 * small stand-alone type with those accessors for callers that do not link the reference.  Likewise the convolution
 * parameters may be the reference's ConvolutionParams (mme/mme_reference/convolution_params.h:7-29) or
 * MmeHip::ConvolutionParams.
 *
 * Header only; link with libmme_hip.so.  Nothing here touches HIP: tensors hold host pointers for the reference-
 * compatible methods, and device pointers for the *Dev methods (same descriptors, asynchronous on the handle's stream).
 */
#ifndef MME_HIP_CALCULATOR_H
#define MME_HIP_CALCULATOR_H

#include "mme_hip.h"

#include <array>
#include <cstdint>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>

namespace MmeHip
{
/* what MME_ASSERT throws (mme/include/mme_assert.h:19-47); status is the C ABI's code */
class MMEStackException : public std::runtime_error
{
public:
    MMEStackException(const std::string& what, int status_) : std::runtime_error(what), status(status_) {}
    int status;
};

/* stand-alone tensor descriptor with the accessors of MMESimTensorBase; never owns or copies the memory
 * (like the reference's wrapping constructor, sim_tensor.cpp:19-20) */
class Tensor
{
public:
    typedef std::array<unsigned, MME_HIP_MAX_TENSOR_DIMS> SizeArray;
    Tensor(const SizeArray& sizes, int dim, int type, void* data_, unsigned fpBias = 0, int infNanMode = MME_HIP_FULL_INF_NAN,
           const SizeArray* strides = nullptr)
        : m_sizes(sizes), m_dim(dim), m_type(type), m_fpBias(fpBias), m_infNanMode(infNanMode), m_data(data_)
    {
        for (int d = dim; d < MME_HIP_MAX_TENSOR_DIMS; d++) m_sizes[d] = 1;
        if (strides) m_strides = *strides;
        else
        {
            unsigned acc = 1;
            for (int d = 0; d < MME_HIP_MAX_TENSOR_DIMS; d++)
            {
                m_strides[d] = acc;
                acc *= m_sizes[d];
            }
        }
    }
    void*            data() const { return m_data; }
    const SizeArray& getSizes() const { return m_sizes; }
    const SizeArray& getStrides() const { return m_strides; }
    int              getDim() const { return m_dim; }
    int              getElementType() const { return m_type; }
    unsigned         getFpBias() const { return m_fpBias; }
    int              getInfNanMode() const { return m_infNanMode; }

private:
    SizeArray m_sizes, m_strides;
    int       m_dim, m_type;
    unsigned  m_fpBias;
    int       m_infNanMode;
    void*     m_data;
};

/* same members as the reference's ConvolutionParams */
struct ConvolutionParams
{
    constexpr static unsigned maxConvDim = 3;
    int                       dim = maxConvDim;
    union
    {
        int16_t  bf16;
        int32_t  f32;
        uint32_t int32 = 0;
    } paddingValue;
    std::array<int, maxConvDim + 1> padding;
    std::array<int, maxConvDim + 1> convStride;
    std::array<int, maxConvDim + 1> dilation;
    bool                            relu = false;
    ConvolutionParams()
    {
        dilation.fill(1);
        convStride.fill(1);
        padding.fill(0);
    }
};

/* stand-alone 2-d matrix with the accessors of the reference's Matrix (mme/mme_reference/mme_reference.h:60-104) that
 * doGemm reads: getElementType(), data(), getMatrix().getHeight() / getWidth().  Row-major height x width; owns a zeroed
 * buffer when no data pointer is given, otherwise copies or wraps the caller's (shouldCopyData), like the reference's
 * first constructor (mme_reference_impl.cpp:17-26). */
class Matrix
{
public:
    struct Shape
    {
        uint64_t height = 0, width = 0;
        uint64_t getHeight() const { return height; }
        uint64_t getWidth() const { return width; }
    };
    Matrix(int type, uint64_t height, uint64_t width, void* data_ = nullptr, bool shouldCopyData = true) : m_type(type)
    {
        m_shape.height = height;
        m_shape.width = width;
        const size_t es = (type == MME_HIP_FP8_143 || type == MME_HIP_FP8_152) ? 1 : ((type == MME_HIP_BF16 || type == MME_HIP_FP16 || type == MME_HIP_UFP16) ? 2 : 4);
        const size_t bytes = (size_t) (height * width) * es;
        if (data_ && !shouldCopyData) m_data = (unsigned char*) data_;
        else
        {
            m_owned.reset(new unsigned char[bytes ? bytes : 1]());
            if (data_ && bytes) std::memcpy(m_owned.get(), data_, bytes);
            m_data = m_owned.get();
        }
    }
    const Shape&         getMatrix() const { return m_shape; }
    int                  getElementType() const { return m_type; }
    unsigned char*       data() { return m_data; }
    const unsigned char* data() const { return m_data; }

private:
    int                              m_type;
    Shape                            m_shape;
    unsigned char*                   m_data = nullptr;
    std::unique_ptr<unsigned char[]> m_owned;
};

/* fused descale + relu + cast behind a device-resident contraction (mme_hip_epilogue) */
typedef mme_hip_epilogue Epilogue;

class Calculator
{
public:
    /* CPUCalculator::CPUCalculator, mme_reference.h:111-117 (chip: the reference's MmeCommon::ChipType value) */
    explicit Calculator(int chip, int max_tensor_dims = MME_HIP_MAX_TENSOR_DIMS, int max_conv_dims = MME_HIP_MAX_CONV_DIMS, unsigned seed = 0,
                        uint32_t lfsrNumRegs = 256, uint32_t* lfsr = nullptr, uint32_t polynomial = 0)
    {
        const int rc = mme_hip_create(&m_h, chip, max_tensor_dims, max_conv_dims, seed, lfsrNumRegs, lfsr, polynomial);
        if (rc != MME_HIP_OK) throw MMEStackException(mme_hip_last_error(nullptr), rc);
    }
    ~Calculator() { mme_hip_destroy(m_h); }
    Calculator(const Calculator&) = delete;
    Calculator& operator=(const Calculator&) = delete;

    /* mme_reference.h:122 */
    void limitNumOfThreads(unsigned numOfThreads) { check(mme_hip_limit_num_of_threads(m_h, numOfThreads)); }

    /* mme_reference.h:126-138, mme_reference_impl.cpp:541-596: output (M x N) = op(A) * op(B) on row-major matrices;
     * transposeA / transposeB say that the matrix handed in is the transpose of the factor.  The exponent biases and
     * inf/NaN modes of the operands are arguments here (a Matrix carries none).  M is the reference's Matrix or
     * MmeHip::Matrix: read through getElementType(), data(), getMatrix().getHeight() / getWidth(). */
    template<class M>
    void doGemm(M& output, const M& inputA, const M& inputB, bool transposeA, bool transposeB, int rm = MME_HIP_RM_NEAREST_EVEN,
                unsigned fpBiasA = 0, unsigned fpBiasB = 0, bool clipFp = false, bool clipFpInfIn = false,
                int infNanModeA = MME_HIP_FULL_INF_NAN, int infNanModeB = MME_HIP_FULL_INF_NAN, int* zeroPoints = nullptr)
    {
        no_zero_points(zeroPoints);
        const mme_hip_tensor o = pod_matrix(output, 0, MME_HIP_FULL_INF_NAN), a = pod_matrix(inputA, fpBiasA, infNanModeA),
                             b = pod_matrix(inputB, fpBiasB, infNanModeB);
        const int op = transposeA ? (transposeB ? MME_HIP_OP_ATBT : MME_HIP_OP_ATB) : (transposeB ? MME_HIP_OP_ABT : MME_HIP_OP_AB);
        check(mme_hip_batch_gemm(m_h, &o, &a, &b, op, rm, clipFp, clipFpInfIn));
    }

    /* mme_reference.h:140 (memcpy / transpose through the MME's DMA mode) and :180-187 (the integer path's requantisation):
     * not part of this library; they throw like any other unsupported request, so that a CPUCalculator built on this class
     * links without the reference's CPU implementation. */
    template<class T>
    void doDma(T&, const T&, int)
    {
        throw MMEStackException("doDma is not built in this library (memcpy / transpose are not contractions)", MME_HIP_EUNSUPPORTED);
    }
    template<class PT>
    void activationGemmlowp(PT, PT, PT, PT, bool, int, const void*)
    {
        throw MMEStackException("activationGemmlowp belongs to the integer path, which is not built in this library", MME_HIP_EUNSUPPORTED);
    }

    /* mme_reference.h:142-149.  zeroPoints belongs to the integer path and must be null. */
    template<class T>
    void doBatchGemm(T& outputTensor, const T& xTensor, const T& wTensor, int op, int rm = MME_HIP_RM_NEAREST_EVEN, bool clipFp = false,
                     bool clipFpInfIn = false, int* zeroPoints = nullptr)
    {
        no_zero_points(zeroPoints);
        const mme_hip_tensor o = pod(outputTensor), x = pod(xTensor), w = pod(wTensor);
        check(mme_hip_batch_gemm(m_h, &o, &x, &w, op, rm, clipFp, clipFpInfIn));
    }

    /* mme_reference.h:151-160.  The result is written into outputTensor's existing buffer. */
    template<class T, class P>
    void doConvolution(T& outputTensor, const T& xTensor, const T& wTensor, const T& yTensor, const P& params, int op,
                       int rm = MME_HIP_RM_NEAREST_EVEN, bool clipFp = false, bool clipFpInfIn = false, int* zeroPoints = nullptr)
    {
        no_zero_points(zeroPoints);
        const mme_hip_tensor      o = pod(outputTensor), x = pod(xTensor), w = pod(wTensor), y = pod(yTensor);
        const mme_hip_conv_params p = pod_conv(params);
        check(mme_hip_convolution(m_h, &o, &x, &w, &y, &p, op, rm, clipFp, clipFpInfIn));
    }

    /* mme_reference.h:162-172: tensors by (shared) pointer; res and bias are not read by the reference's float path
     * (mme_reference_impl.cpp:661-689) and must be null, actParams belongs to the integer path and must be null */
    template<class PT>
    void doActivation(PT output, const PT acc, const PT res, const PT bias, bool relu, int rm = MME_HIP_RM_NEAREST_EVEN,
                      const void* actParams = nullptr, bool clipFp = false, bool clipInfIn = false, bool flushDenorms = false,
                      bool stochasticFTZfp8 = false)
    {
        if (res || bias || actParams) throw MMEStackException("residual, bias and gemmlowp parameters belong to the integer path", MME_HIP_EUNSUPPORTED);
        const mme_hip_tensor o = pod(*output), a = pod(*acc);
        check(mme_hip_activation(m_h, &o, &a, relu, rm, clipFp, clipInfIn, flushDenorms, stochasticFTZfp8));
    }

    /* mme_reference.h:174-178 */
    template<class PT>
    void doMemoryWrite(PT memory, const PT mmeOut, int reductionOp = MME_HIP_REDUCTION_NONE, int reductionRm = 0, bool clipFp = false)
    {
        const mme_hip_tensor m = pod(*memory), o = pod(*mmeOut);
        check(mme_hip_memory_write(m_h, &m, &o, reductionOp, reductionRm, clipFp));
    }

    /* ---- device-resident forms: same descriptors holding device pointers; work is enqueued on stream() ------------ */
    template<class T>
    void doBatchGemmDev(T& outputTensor, const T& xTensor, const T& wTensor, int op, const Epilogue* epilogue = nullptr)
    {
        const mme_hip_tensor o = pod(outputTensor), x = pod(xTensor), w = pod(wTensor);
        check(mme_hip_batch_gemm_dev(m_h, &o, &x, &w, op, epilogue));
    }
    template<class T, class P>
    void doConvolutionDev(T& outputTensor, const T& xTensor, const T& wTensor, const T& yTensor, const P& params, int op,
                          const Epilogue* epilogue = nullptr)
    {
        const mme_hip_tensor      o = pod(outputTensor), x = pod(xTensor), w = pod(wTensor), y = pod(yTensor);
        const mme_hip_conv_params p = pod_conv(params);
        check(mme_hip_convolution_dev(m_h, &o, &x, &w, &y, &p, op, epilogue));
    }
    template<class T>
    void doActivationDev(T& output, const T& acc, bool relu, int rm = MME_HIP_RM_NEAREST_EVEN, bool clipFp = false, bool clipInfIn = false,
                         bool flushDenorms = false, bool stochasticFTZfp8 = false)
    {
        const mme_hip_tensor o = pod(output), a = pod(acc);
        check(mme_hip_activation_dev(m_h, &o, &a, relu, rm, clipFp, clipInfIn, flushDenorms, stochasticFTZfp8));
    }
    template<class T>
    void doMemoryWriteDev(T& memory, const T& mmeOut, int reductionOp = MME_HIP_REDUCTION_NONE, int reductionRm = 0, bool clipFp = false)
    {
        const mme_hip_tensor m = pod(memory), o = pod(mmeOut);
        check(mme_hip_memory_write_dev(m_h, &m, &o, reductionOp, reductionRm, clipFp));
    }
    void* stream() const { return mme_hip_stream(m_h); }
    void  setStream(void* hipStream) { check(mme_hip_set_stream(m_h, hipStream)); }
    void  synchronize() { check(mme_hip_synchronize(m_h)); }
    void  setFp8SpecialsPolicy(int policy) { check(mme_hip_set_fp8_specials_policy(m_h, policy)); }
    /* clipFp / clipFpInfIn for the device-resident contractions (read by the tf32 operand conversion only) */
    void  setOperandClip(bool clipFp, bool clipFpInfIn) { check(mme_hip_set_operand_clip(m_h, clipFp, clipFpInfIn)); }
    mme_hip_handle handle() const { return m_h; }

    /* Which kernel form a device-resident call would launch, without making it and without a device (mme_hip_plan_batch_gemm /
     * mme_hip_plan_convolution; no counterpart in the reference): the descriptors go through the same checks and planning as
     * the real call, their data pointers are not dereferenced.  Throws like the real call for a problem it would refuse. */
    struct Form
    {
        int largeTile;  /* 1 a large-tile kernel, 0 the general kernel, 2 the 3 x 3 forward kernel, -1 no contraction kernel */
        int tileRows;   /* 256 or 128 */
        int splitK;     /* slices of the reduction, 1: none */
        int wavefronts; /* per workgroup: 8 or 4 */
    };
    template<class T>
    static Form planBatchGemm(const T& outputTensor, const T& xTensor, const T& wTensor, int op, const Epilogue* epilogue = nullptr, int numCus = 256,
                              int fp8SpecialsPolicy = MME_HIP_FP8_SPECIALS_CHECK)
    {
        const mme_hip_tensor o = pod(outputTensor), x = pod(xTensor), w = pod(wTensor);
        int                  form[4];
        char                 error[512];
        const int            rc = mme_hip_plan_batch_gemm(&o, &x, &w, op, epilogue, numCus, fp8SpecialsPolicy, form, error, sizeof error);
        if (rc != MME_HIP_OK) throw MMEStackException(error, rc);
        return Form {form[0], form[1], form[2], form[3]};
    }
    template<class T, class P>
    static Form planConvolution(const T& outputTensor, const T& xTensor, const T& wTensor, const T& yTensor, const P& params, int op,
                                const Epilogue* epilogue = nullptr, int numCus = 256, int fp8SpecialsPolicy = MME_HIP_FP8_SPECIALS_CHECK)
    {
        const mme_hip_tensor      o = pod(outputTensor), x = pod(xTensor), w = pod(wTensor), y = pod(yTensor);
        const mme_hip_conv_params p = pod_conv(params);
        int                       form[4];
        char                      error[512];
        const int rc = mme_hip_plan_convolution(&o, &x, &w, &y, &p, op, epilogue, numCus, fp8SpecialsPolicy, form, error, sizeof error);
        if (rc != MME_HIP_OK) throw MMEStackException(error, rc);
        return Form {form[0], form[1], form[2], form[3]};
    }

private:
    template<class T>
    static mme_hip_tensor pod(const T& t)
    {
        mme_hip_tensor d;
        d.data = (void*) t.data();
        for (int i = 0; i < MME_HIP_MAX_TENSOR_DIMS; i++)
        {
            d.sizes[i] = (uint32_t) t.getSizes()[i];
            d.strides[i] = (uint32_t) t.getStrides()[i];
        }
        d.dim = t.getDim();
        d.dtype = (int32_t) t.getElementType();
        d.fp_bias = t.getFpBias();
        d.inf_nan_mode = (int32_t) t.getInfNanMode();
        return d;
    }
    template<class M>
    static mme_hip_tensor pod_matrix(const M& m, unsigned fpBias, int infNanMode)
    {
        mme_hip_tensor d;
        const uint64_t h = m.getMatrix().getHeight(), w = m.getMatrix().getWidth();
        if (h >= (1ull << 31) || w >= (1ull << 31) || h * w >= (1ull << 31)) throw MMEStackException("matrix: more than 2^31 elements", MME_HIP_EINVAL);
        d.data = (void*) m.data();
        for (int i = 0; i < MME_HIP_MAX_TENSOR_DIMS; i++)
        {
            d.sizes[i] = 1;
            d.strides[i] = (uint32_t) (h * w);
        }
        d.sizes[0] = (uint32_t) w;
        d.sizes[1] = (uint32_t) h;
        d.strides[0] = 1;
        d.strides[1] = (uint32_t) w;
        d.dim = 2;
        d.dtype = (int32_t) m.getElementType();
        d.fp_bias = fpBias;
        d.inf_nan_mode = infNanMode;
        return d;
    }
    template<class P>
    static mme_hip_conv_params pod_conv(const P& p)
    {
        mme_hip_conv_params c;
        c.dim = p.dim;
        c.padding_value = p.paddingValue.int32;
        for (int i = 0; i < MME_HIP_MAX_CONV_DIMS; i++)
        {
            c.padding[i] = p.padding[i];
            c.conv_stride[i] = p.convStride[i];
            c.dilation[i] = p.dilation[i];
        }
        c.relu = p.relu;
        return c;
    }
    static void no_zero_points(const int* zp)
    {
        if (zp) throw MMEStackException("zero points belong to the integer path", MME_HIP_EUNSUPPORTED);
    }
    void check(int rc) const
    {
        if (rc != MME_HIP_OK) throw MMEStackException(mme_hip_last_error(m_h), rc);
    }
    mme_hip_handle m_h = nullptr;
};

} // namespace MmeHip

#endif /* MME_HIP_CALCULATOR_H */
