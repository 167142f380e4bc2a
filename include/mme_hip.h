/*
 * mme_hip.h -- C ABI of the MI355X (gfx950) MME compute path.
 *
 * This is the drop-in boundary: a C++ class with the reference calculator's
 * surface (include/mme_hip_calculator.h) forwards every call to the entry
 * points below.  Signatures hold plain pointers, sizes and enum integers only.
 *
 * Each entry point cites the reference interface it replaces.  Paths are
 * relative to the reference tree (HabanaAI/Intel_Gaudi3_Software).
 *
 * Conventions
 *  - sizes[0] is the fastest (contiguous) dimension; strides are in elements
 *    (mme/mme_reference/sim_tensor_base.h:52-54,143-156).
 *  - dtype, op, rounding-mode and inf/nan-mode integers are the reference's enum
 *    values (mme/include/mme_common/mme_common_enum.h:25-102,191-197).
 *  - every function returns MME_HIP_OK (0) or a negative MME_HIP_E* code; the
 *    text of the last failure on a handle is mme_hip_last_error(h).  The C++
 *    wrapper turns a non-zero status into MmeCommon::MMEStackException, which
 *    is what MME_ASSERT does in the reference's release builds
 *    (mme/include/mme_assert.h:19-58).
 *  - "host" entry points take host pointers, stage through device memory and
 *    return with the result visible in host memory (the reference calculator is
 *    synchronous).  "_dev" entry points take device pointers and only enqueue
 *    work on the handle's stream; they allocate no device memory unless noted.
 *  - a handle is bound to one device and one HIP stream and is not re-entrant,
 *    like the reference object (per-call state in
 *    mme/mme_reference/mme_reference_impl.cpp:218-243).
 */
#ifndef MME_HIP_H
#define MME_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MME_HIP_MAX_TENSOR_DIMS 5 /* MME_MAX_TENSOR_DIMS, mme_common_enum.h:8 */
#define MME_HIP_MAX_CONV_DIMS 4   /* MME_MAX_CONV_DIMS,   mme_common_enum.h:9 */

/* status codes */
enum
{
    MME_HIP_OK = 0,
    MME_HIP_EINVAL = -1,      /* a reference MME_ASSERT condition failed            */
    MME_HIP_EUNSUPPORTED = -2,/* valid in the reference, not built in this library  */
    MME_HIP_EHIP = -3,        /* a HIP runtime call failed                          */
    MME_HIP_ENOMEM = -4
};

/* MmeCommon::ChipType (mme_common_enum.h:25-30). Only Gaudi3 numerics are built. */
enum
{
    MME_HIP_CHIP_GAUDI = 0,
    MME_HIP_CHIP_GAUDI2 = 1,
    MME_HIP_CHIP_GAUDI3 = 2
};

/* MmeCommon::EMmeDataType (mme_common_enum.h:32-61), float types of the path. */
enum
{
    MME_HIP_FP8_143 = 9,
    MME_HIP_FP8_152 = 10,
    MME_HIP_FP16 = 11, /* 1-5-10, configurable exponent bias (default 15) */
    MME_HIP_BF16 = 12,
    MME_HIP_FP32 = 13,
    MME_HIP_FP32_IEEE = 14,
    MME_HIP_TF32 = 15, /* operand type only: fp32 words, rounded to 10 mantissa bits on entry */
    MME_HIP_UFP16 = 17 /* unsigned fp16, 0-6-10, configurable exponent bias (default 31); e_types_nr is 16 */
};

/* MmeCommon::RoundingMode (mme_common_enum.h:65-80). */
enum
{
    MME_HIP_RM_NEAREST_EVEN = 0,
    MME_HIP_RM_TO_ZERO = 1,
    MME_HIP_RM_UP = 2,
    MME_HIP_RM_DOWN = 3,
    MME_HIP_RM_STOCHASTIC = 4,
    MME_HIP_RM_HALF_AWAY = 6,
    MME_HIP_RM_STOCHASTIC_AND_NEAREST = 7
};

/* MmeCommon::EMmeOpType (mme_common_enum.h:82-102). */
enum
{
    MME_HIP_OP_FWD = 0,
    MME_HIP_OP_DEDX = 1,
    MME_HIP_OP_DEDW = 2,
    MME_HIP_OP_DETERMINISTIC_DEDW = 3,
    MME_HIP_OP_TRANSPOSED_DEDX = 4,
    MME_HIP_OP_AB = 5,
    MME_HIP_OP_ABT = 6,
    MME_HIP_OP_ATB = 7,
    MME_HIP_OP_ATBT = 8
};

/* MmeCommon::InfNanMode (mme_common_enum.h:191-197). */
enum
{
    MME_HIP_FULL_INF_NAN = 0,
    MME_HIP_NO_INF_NAN = 1,
    MME_HIP_MINIMAL_INF_NAN = 2
};

/* MmeCommon::EMmeReductionOp (mme_common_enum.h:321-332). */
enum
{
    MME_HIP_REDUCTION_ADD = 0,
    MME_HIP_REDUCTION_SUB = 1,
    MME_HIP_REDUCTION_MIN = 2,
    MME_HIP_REDUCTION_MAX = 3,
    MME_HIP_REDUCTION_MAX_0 = 4,
    MME_HIP_REDUCTION_NONE = 5
};

/* MmeCommon::EMmeReductionRm (mme_common_enum.h:334-342). */
enum
{
    MME_HIP_REDUCTION_RM_NEAREST_EVEN = 0,
    MME_HIP_REDUCTION_RM_TO_ZERO = 1,
    MME_HIP_REDUCTION_RM_UP = 2,
    MME_HIP_REDUCTION_RM_DOWN = 3
};

/*
 * Tensor descriptor: the fields of MMESimTensorBase
 * (mme/mme_reference/sim_tensor_base.h:143-156) as a POD.
 * data is borrowed, never freed (sim_tensor.cpp:19-20).
 */
typedef struct mme_hip_tensor
{
    void*    data;
    uint32_t sizes[MME_HIP_MAX_TENSOR_DIMS];
    uint32_t strides[MME_HIP_MAX_TENSOR_DIMS]; /* elements; strides[0] must be 1 */
    int32_t  dim;
    int32_t  dtype;
    uint32_t fp_bias;      /* exponent bias of fp8 tensors (fpBias)              */
    int32_t  inf_nan_mode; /* InfNanMode of fp8 tensors                           */
} mme_hip_tensor;

/* ConvolutionParams (mme/mme_reference/convolution_params.h:7-29) as a POD. */
typedef struct mme_hip_conv_params
{
    int32_t  dim;              /* number of spatial dims, <= 3                   */
    uint32_t padding_value;    /* paddingValue.int32; forced to 0 for float types
                                  (mme_reference_impl.cpp:811-819)               */
    int32_t  padding[4];       /* indexed W, H, D, batch                         */
    int32_t  conv_stride[4];
    int32_t  dilation[4];
    int32_t  relu;             /* carried, unused by the contraction             */
} mme_hip_conv_params;

/*
 * Optional epilogue of the fused entry points.  The reference has no such
 * struct: it runs doBatchGemm/doConvolution into an fp32 tensor and then
 * doActivation (mme_verification/common/mme_test_manager.cpp:819-900); the
 * fused form is that same sequence with the power-of-two descale of the test
 * harness in between, done in registers instead of through an fp32 tensor:
 *     y = cast( relu?( acc * 2^scale_exp * 2^col_scale_exp[n] ) )
 * Each multiplication is an fp32 multiplication by an exact power of two.
 * With a stochastic rounding mode (4, 7) the conversion is the one of doActivation,
 * which runs over the output tensor's whole span in memory
 * (mme_reference_impl.cpp:1155, sim_tensor_base.cpp:177-194): the bytes between the
 * rows of an output with strided rows are then overwritten with the code of zero,
 * as they are when the reference converts a fresh accumulator tensor of that shape.
 * The other rounding modes leave those bytes untouched.
 */
typedef struct mme_hip_epilogue
{
    int32_t        scale_exp;      /* per-tensor exponent, |e| <= 126             */
    const int32_t* col_scale_exp;  /* per output channel (sizes[0] of out), device
                                      pointer in _dev calls, may be NULL          */
    int32_t        relu;
    int32_t        rounding_mode;  /* conversion rounding mode                    */
    int32_t        clip_fp;
    int32_t        clip_inf_in;
    int32_t        flush_denorms;
} mme_hip_epilogue;

typedef struct mme_hip_calc* mme_hip_handle;

/* ---- life cycle --------------------------------------------------------- */

/* Version string of the library ("mme-hip x.y gfx950"). */
const char* mme_hip_version(void);

/*
 * CPUCalculator::CPUCalculator(chip, max_tensor_dims, max_conv_dims, seed,
 * lfsrNumRegs, lfsr, polynomial) -- mme/mme_reference/mme_reference.h:111-117,
 * mme_reference_impl.cpp:129-200.  Fails with EINVAL when the dims differ from
 * 5 / 4 (:143-144) and EUNSUPPORTED for chips other than Gaudi3.
 * The handle uses the current HIP device and creates one stream on it.
 */
int mme_hip_create(mme_hip_handle* out,
                   int             chip,
                   int             max_tensor_dims,
                   int             max_conv_dims,
                   unsigned        seed,
                   uint32_t        lfsr_num_regs,
                   const uint32_t* lfsr,
                   uint32_t        polynomial);

/* CPUCalculator::~CPUCalculator -- mme_reference.h:118. */
void mme_hip_destroy(mme_hip_handle h);

/* Text of the last error on this handle (never NULL). h may be NULL for create errors. */
const char* mme_hip_last_error(mme_hip_handle h);

/* CPUCalculator::limitNumOfThreads -- mme_reference.h:122, impl :2002-2012.
 * Accepted and recorded; the GPU path has no host worker threads. */
int mme_hip_limit_num_of_threads(mme_hip_handle h, unsigned num_threads);

/* The handle's hipStream_t as void*.  _dev calls are enqueued on it. */
void* mme_hip_stream(mme_hip_handle h);

/* Use a caller-owned hipStream_t (NULL = the handle's own stream).  A handle's work spaces (split-k partial sums, decoded
 * operand copies, the flags and counters of the fp8 operand checks) are reused from call to call in stream order: the
 * caller orders the new stream behind what the handle enqueued on the previous one (or waits for it) before the next call.
 * Calls that may overlap in time belong on handles of their own. */
int mme_hip_set_stream(mme_hip_handle h, void* hip_stream);

/* hipStreamSynchronize on the handle's stream. */
int mme_hip_synchronize(mme_hip_handle h);

/*
 * Kernels whose wavefronts hand work to each other through counters in LDS (the 3x3 forward convolution) poll those counters
 * a bounded number of times; a wavefront that runs out of polls records that in a status word and goes on, so every kernel
 * ends, and mme_hip_synchronize (and the host-pointer entry points) then return MME_HIP_EHIP: the outputs since the last
 * synchronisation are not valid.  This sets the bound (default 2^22 polls of about 64 clocks).  No counterpart in the
 * reference; a host-side test uses a bound of zero to exercise the report.
 */
int mme_hip_set_wait_limit(mme_hip_handle h, unsigned polls);

/*
 * Diagnostics, no counterpart in the reference.  The device lowers its shader clock under load, and by how much depends on
 * the operand values (all-zero operands toggle nothing), so a kernel's distance from the published peak rate says little
 * without the clock it ran at.
 *
 * mme_hip_clock_probe(h, 1): from now on every workgroup of the large-tile contraction kernels notes the shader clock
 * counter and the constant 100 MHz counter when it starts and when it ends (up to 4096 workgroups per launch, 128 KiB of
 * device memory, allocated here); (h, 0) switches that off again.  mme_hip_clock_probe_read synchronises the stream and
 * reports, over the workgroups that ran since the last read: the clock (shader clocks per 100 MHz tick x 100), the mean and
 * the longest time a workgroup took, and their number.
 *
 * mme_hip_matrix_core_rate: `launches` launches of a loop of `iters` x 8 matrix instructions per wavefront (32x32x64 fp8
 * for MME_HIP_FP8_143, 32x32x16 for MME_HIP_BF16) on every compute unit, operands in registers, all zero or
 * (random_operands != 0) random and changing from instruction to instruction: the rate the matrix cores sustain on this
 * device with nothing else to do, and the clock they held.
 *
 * mme_hip_last_contraction_form: which form of the contraction kernels the latest doBatchGemm / doConvolution call of this
 * handle launched: large_tile 1 when a large-tile kernel took it (0: the general kernel; 2: the forward kernel for 3 x 3
 * filters over 64 -> 64 bf16 channels, whose other three figures are 0, 1, 8), the rows of its output tile (256 or
 * 128), the slices of the reduction (1: no split-k) and the wavefronts per workgroup (8, or 4 for the fp8 GEMM form with
 * 128 x 128 outputs per wavefront).  Lets a test state which kernel it is about.
 *
 * mme_hip_plan_batch_gemm / mme_hip_plan_convolution: the same four figures (form[0..3], in that order) for a call that is not
 * made: what mme_hip_batch_gemm_dev / mme_hip_convolution_dev would launch for these descriptors on a device with num_cus
 * compute units (<= 0: 256) under the given policy for fp8 special codes.  The call goes through the same checks and the same
 * planning code as the real one, launches and allocates nothing and needs no device or handle; the data pointers of the
 * descriptors are not dereferenced (their alignment matters: hand in the real ones, or any 16-byte aligned non-null value).
 * Returns what the real call would return for a refused problem, with its message in `error` (may be NULL); form[0] is -1 for
 * a problem that launches no contraction kernel (a zero-size common dimension).
 */
int mme_hip_clock_probe(mme_hip_handle h, int enable);
int mme_hip_last_contraction_form(mme_hip_handle h, int* large_tile, int* tile_rows, int* split_k, int* wavefronts);
int mme_hip_plan_batch_gemm(const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w, int op,
                            const mme_hip_epilogue* epilogue, int num_cus, int fp8_specials_policy, int form[4], char* error,
                            size_t error_bytes);
int mme_hip_plan_convolution(const mme_hip_tensor* out, const mme_hip_tensor* x, const mme_hip_tensor* w, const mme_hip_tensor* y,
                             const mme_hip_conv_params* params, int op, const mme_hip_epilogue* epilogue, int num_cus,
                             int fp8_specials_policy, int form[4], char* error, size_t error_bytes);
int mme_hip_clock_probe_read(mme_hip_handle h, double* shader_mhz, double* mean_us, double* max_us, int* workgroups);
int mme_hip_matrix_core_rate(mme_hip_handle h, int dtype, int random_operands, int iters, int launches, double* tflops, double* shader_mhz);

/*
 * clipFp / clipFpInfIn of the operand conversion, for the device-pointer contraction entry points (the host-pointer
 * ones take them per call).  On Gaudi3 only the tf32 flavour reads them: its operands are rounded from fp32 to tf32 on
 * entry and an overflow to infinity is clipped to the largest finite value when clip_fp is set (and, for an infinite
 * input, only when clip_fp_inf_in is set too) -- CPUCalculator::doBatchGemm / doConvolution arguments,
 * mme/mme_reference/mme_reference.h:127-150, passed on at mme_reference_impl.cpp:223-239 to
 * Gaudi3Tf32Fma (chip_fma/gaudi3_fma.h:88-105).  Default: both off.
 */
int mme_hip_set_operand_clip(mme_hip_handle h, int clip_fp, int clip_fp_inf_in);

/*
 * fp8 operands and the matrix cores.  gfx950's MFMA reads OCP e4m3 / e5m2.  Gaudi's fp8_152 in full inf/nan mode is
 * e5m2 up to the exponent bias, and fp8_143 in minimal inf/nan mode is e4m3; the bias becomes an exact power of two
 * on the accumulators.  In the other modes the codes with all exponent bits set mean something else to the hardware
 * (fp8_143 full mode: inf / NaN, fs_fma.cpp:6090-6100, but 256..448 for e4m3).
 *   MME_HIP_FP8_SPECIALS_CHECK (default): operands in such modes are scanned on the device; if a scan finds such a
 *     code the contraction runs on an exact bf16 decode of the operands instead (the whole contraction, enqueued behind
 *     the native kernel and predicated on a device flag; or, for large one-round fp8 GEMMs, the affected output tiles
 *     only, inside the native kernel's own launch; calls enqueued while the stream records a graph always take the
 *     predicated form, whose device flag survives replays on the safe side).  No host synchronisation.
 *   MME_HIP_FP8_SPECIALS_ASSUME_NONE: the caller guarantees that neither operand holds a code with all exponent bits set
 *     (e.g. the operands come out of a saturating quantiser, which never emits them); nothing is checked, and the
 *     output conversion does not look out for inf / NaN accumulators either.
 * No counterpart in the reference, which decodes every element in software.
 */
enum
{
    MME_HIP_FP8_SPECIALS_CHECK = 0,
    MME_HIP_FP8_SPECIALS_ASSUME_NONE = 1
};
int mme_hip_set_fp8_specials_policy(mme_hip_handle h, int policy);

/* ---- contraction: host pointers (reference-compatible, synchronous) ------ */

/*
 * CPUCalculator::doBatchGemm(out, x, w, op, rm, clipFp, clipFpInfIn, zeroPoints)
 * mme_reference.h:142-149, mme_reference_impl.cpp:445-539.
 * out must be fp32 (only {in,fp32} workers are registered, :188-196, :591).
 * rm is accepted and inert on the Gaudi3 float path (chip_fma/gaudi3_fma.cpp:40-60);
 * clip_fp / clip_fp_inf_in reach the tf32 operand conversion only (gaudi3_fma.h:43,79,96-98).
 * Operand types: bf16, fp32, tf32, fp16 / ufp16 (mixable), fp8_143 / fp8_152 (mixable).
 */
int mme_hip_batch_gemm(mme_hip_handle        h,
                       const mme_hip_tensor* out,
                       const mme_hip_tensor* x,
                       const mme_hip_tensor* w,
                       int                   op,
                       int                   rounding_mode,
                       int                   clip_fp,
                       int                   clip_fp_inf_in);

/*
 * CPUCalculator::doConvolution(out, x, w, y, params, op, rm, clipFp, clipFpInfIn, zp)
 * mme_reference.h:151-160, mme_reference_impl.cpp:598-659, 770-869.
 * Unlike the reference (:862-868) the result is always written into out->data.
 * rm reaches only the fp32 additions of dedx's col2im (im2col.h:70-75); this
 * library accumulates all taps of a dedx output in one fp32 MFMA accumulator.
 */
int mme_hip_convolution(mme_hip_handle             h,
                        const mme_hip_tensor*      out,
                        const mme_hip_tensor*      x,
                        const mme_hip_tensor*      w,
                        const mme_hip_tensor*      y,
                        const mme_hip_conv_params* params,
                        int                        op,
                        int                        rounding_mode,
                        int                        clip_fp,
                        int                        clip_fp_inf_in);

/*
 * CPUCalculator::doActivation(out, acc, res, bias, relu, rm, actParams, clipFp,
 * clipInfIn, flushDenorms, stochasticFTZfp8) -- mme_reference.h:162-172,
 * mme_reference_impl.cpp:661-689, 1143-1245.  res / bias / actParams are unused
 * by the reference's float path and have no parameter here.  relu modifies acc
 * in place like the reference (:683-686, 1132-1141).
 * The stochastic modes (rounding modes 4 and 7, stochastic_ftz_fp8) draw from the
 * calculator's LFSR registers exactly as the reference does (:1153-1240): element
 * i takes register i % 128 (fp8) or i % 64 (bf16), and the register steps once
 * after every use; the registers persist in the handle between calls.
 */
int mme_hip_activation(mme_hip_handle        h,
                       const mme_hip_tensor* out,
                       const mme_hip_tensor* acc,
                       int                   relu,
                       int                   rounding_mode,
                       int                   clip_fp,
                       int                   clip_inf_in,
                       int                   flush_denorms,
                       int                   stochastic_ftz_fp8);

/*
 * CPUCalculator::doMemoryWrite(memory, mmeOut, reductionOp, reductionRm, clipFp)
 * mme_reference.h:174-178, mme_reference_impl.cpp:718-768.  reduction_none is a
 * byte copy of memory's size.  add / sub / min / max / max_0 combine memory with
 * mmeOut element by element as the reference's executeOp does for fp32, bf16,
 * fp16 and fp8_152 tensors (fs_fma.cpp:2288-2955: an adder that rounds once in
 * reduction_rm and flushes denormal operands and results; fp16 and fp8_152 are
 * taken with exponent bias 15 and inf / NaN whatever the tensor's fields say,
 * fp8_152 sums are formed in fp16 and rounded a second time); the types the
 * reference rejects (fp8_143, ufp16) return EINVAL.
 */
int mme_hip_memory_write(mme_hip_handle        h,
                         const mme_hip_tensor* memory,
                         const mme_hip_tensor* mme_out,
                         int                   reduction_op,
                         int                   reduction_rm,
                         int                   clip_fp);

/* The same on device-resident tensors, asynchronous on the handle's stream (no
 * counterpart in the reference). */
int mme_hip_memory_write_dev(mme_hip_handle        h,
                             const mme_hip_tensor* memory,
                             const mme_hip_tensor* mme_out,
                             int                   reduction_op,
                             int                   reduction_rm,
                             int                   clip_fp);

/* ---- contraction: device pointers (asynchronous on the handle's stream) --- */

/*
 * doBatchGemm on device-resident tensors.  epilogue == NULL: out must be fp32
 * and receives the raw accumulators (reference semantics).  epilogue != NULL:
 * out may be fp32 / bf16 / fp16 / ufp16 / fp8_143 / fp8_152 and receives the fused
 * descale + relu + cast described at mme_hip_epilogue.
 */
int mme_hip_batch_gemm_dev(mme_hip_handle          h,
                           const mme_hip_tensor*   out,
                           const mme_hip_tensor*   x,
                           const mme_hip_tensor*   w,
                           int                     op,
                           const mme_hip_epilogue* epilogue);

/*
 * mme_hip_batch_gemm_dev for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid it).  No counterpart in the reference.  Same arguments, same kernels and bit-identical
 * results, but every work space the call needs (split-k partial sums, the decoded operand copies and the flag cell of the
 * fp8 / fp16 / tf32 / fp32 fall-backs) is taken from a static device array of MME_HIP_NOALLOC_SCRATCH_BYTES that each
 * device holds from the moment the library's code is loaded there until the process ends; the call never calls hipMalloc,
 * hipFree or an allocating library routine.  A problem whose work space does not fit returns MME_HIP_ENOMEM with the sizes
 * in mme_hip_last_error (large fp8 operands in an inf/NaN mode the hardware formats lack need decoded copies for the
 * fall-back: set MME_HIP_FP8_SPECIALS_ASSUME_NONE where that holds, or use mme_hip_batch_gemm_dev).  All handles of a
 * device share that device's array: calls that overlap in time on one device race on it, so serialise them (one stream,
 * or events between streams).  A stochastic rounding mode in the epilogue is served too (the LFSR jump table exists since
 * mme_hip_create; the fp32 intermediate comes out of the same array).
 *
 * Recording the other device-pointer entry points into a HIP graph: the recorded launches hold the addresses of the handle's
 * grow-only work spaces.  A work space must have its size before the recording starts (growing one on a recording stream
 * fails with the HIP error and leaves it as it was); once a handle has seen a recording stream it keeps every block it
 * outgrows until mme_hip_destroy instead of freeing it, so later larger calls do not invalidate a graph.  Destroy the graph
 * before the handle.
 */
#define MME_HIP_NOALLOC_SCRATCH_BYTES (32u << 20)
int mme_hip_batch_gemm_dev_noalloc(mme_hip_handle          h,
                                   const mme_hip_tensor*   out,
                                   const mme_hip_tensor*   x,
                                   const mme_hip_tensor*   w,
                                   int                     op,
                                   const mme_hip_epilogue* epilogue);

/* doConvolution on device-resident tensors; epilogue as above.  dedw with a
 * split reduction uses workspace from the handle (allocated on first use). */
int mme_hip_convolution_dev(mme_hip_handle             h,
                            const mme_hip_tensor*      out,
                            const mme_hip_tensor*      x,
                            const mme_hip_tensor*      w,
                            const mme_hip_tensor*      y,
                            const mme_hip_conv_params* params,
                            int                        op,
                            const mme_hip_epilogue*    epilogue);

/* doActivation on device-resident tensors (relu applied while casting; acc is
 * also updated in place when relu is set, like the reference). */
int mme_hip_activation_dev(mme_hip_handle        h,
                           const mme_hip_tensor* out,
                           const mme_hip_tensor* acc,
                           int                   relu,
                           int                   rounding_mode,
                           int                   clip_fp,
                           int                   clip_inf_in,
                           int                   flush_denorms,
                           int                   stochastic_ftz_fp8);

/* ---- elementwise cast / quantize / dequantize on flat device buffers ------ */

/*
 * n elements of fp32 -> out_dtype with the semantics of
 * convertToOutputDataType (mme_reference_impl.cpp:1143-1245): gaudi3::fp32_to_fp8
 * (coral-sim/src/gaudi3/fs_core/fs_fma.cpp:6731-7027), fp32_to_bf16 (:851-924),
 * fp32_to_fp32 (:1064-1088).  Before the cast each element is multiplied by
 * 2^scale_exp and, when col_scale_exp != NULL, by 2^col_scale_exp[i % n_cols]
 * (quantize-with-scale; both 0/NULL for a plain cast).  Deterministic rounding
 * modes only (0,1,2,3,6).
 */
int mme_hip_cast_from_fp32_dev(mme_hip_handle h,
                               void*          out,
                               int            out_dtype,
                               unsigned       out_fp_bias,
                               int            out_inf_nan_mode,
                               const float*   in,
                               size_t         n,
                               int            scale_exp,
                               const int32_t* col_scale_exp,
                               size_t         n_cols,
                               int            relu,
                               int            rounding_mode,
                               int            clip_fp,
                               int            clip_inf_in,
                               int            flush_denorms);

/*
 * n elements of in_dtype (fp8_143 / fp8_152 / bf16) -> fp32: gaudi3::fp8_to_fp32
 * (fs_fma.cpp:6066-6139) / bf16 << 16, then multiplied by 2^scale_exp and
 * 2^col_scale_exp[i % n_cols] (dequantize).
 */
int mme_hip_cast_to_fp32_dev(mme_hip_handle h,
                             float*         out,
                             const void*    in,
                             int            in_dtype,
                             unsigned       in_fp_bias,
                             int            in_inf_nan_mode,
                             size_t         n,
                             int            scale_exp,
                             const int32_t* col_scale_exp,
                             size_t         n_cols);

/*
 * max |x| over n fp32 elements (NaNs ignored), written as one float to
 * *out_absmax (device pointer).  Pre-pass of per-tensor scale selection; the
 * reference's harness computes it on the host (no reference function).
 */
int mme_hip_absmax_dev(mme_hip_handle h, float* out_absmax, const float* in, size_t n);

#ifdef __cplusplus
}
#endif
#endif /* MME_HIP_H */
