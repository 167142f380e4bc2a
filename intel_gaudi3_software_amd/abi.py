"""ctypes mirror of ``include/mme_hip.h``: PODs, enum values and the loader of ``libmme_hip.so``.

The enum integers are the reference's own (mme/include/mme_common/mme_common_enum.h:25-102,191-197), so a
descriptor built here can be handed unchanged to the reference calculator's ``MmeSimTensor`` constructor
(mme/mme_reference/sim_tensor.h:13-19).
"""
import ctypes as C
import os

import numpy as np

MAX_TENSOR_DIMS = 5
MAX_CONV_DIMS = 4

# status
OK, EINVAL, EUNSUPPORTED, EHIP, ENOMEM = 0, -1, -2, -3, -4
# ChipType
CHIP_GAUDI, CHIP_GAUDI2, CHIP_GAUDI3 = 0, 1, 2
# EMmeDataType
FP8_143, FP8_152, FP16, BF16, FP32, FP32_IEEE, TF32, UFP16 = 9, 10, 11, 12, 13, 14, 15, 17
# RoundingMode
RM_NEAREST_EVEN, RM_TO_ZERO, RM_UP, RM_DOWN, RM_STOCHASTIC, RM_HALF_AWAY, RM_STOCHASTIC_AND_NEAREST = 0, 1, 2, 3, 4, 6, 7
# EMmeOpType
OP_FWD, OP_DEDX, OP_DEDW, OP_DETERMINISTIC_DEDW, OP_TRANSPOSED_DEDX, OP_AB, OP_ABT, OP_ATB, OP_ATBT = range(9)
# InfNanMode
FULL_INF_NAN, NO_INF_NAN, MINIMAL_INF_NAN = 0, 1, 2
REDUCTION_ADD, REDUCTION_SUB, REDUCTION_MIN, REDUCTION_MAX, REDUCTION_MAX_0, REDUCTION_NONE = range(6)  # EMmeReductionOp
FP8_SPECIALS_CHECK, FP8_SPECIALS_ASSUME_NONE = 0, 1

DTYPE_SIZE = {FP8_143: 1, FP8_152: 1, FP16: 2, UFP16: 2, BF16: 2, FP32: 4, FP32_IEEE: 4, TF32: 4}
DTYPE_NUMPY = {FP8_143: np.uint8, FP8_152: np.uint8, BF16: np.uint16, FP16: np.uint16, UFP16: np.uint16, FP32: np.float32,
               FP32_IEEE: np.float32, TF32: np.uint32}
DTYPE_NAME = {FP8_143: "fp8_143", FP8_152: "fp8_152", BF16: "bf16", FP16: "fp16", UFP16: "ufp16", FP32: "fp32",
              FP32_IEEE: "fp32_ieee", TF32: "tf32"}


class Tensor(C.Structure):
    """``mme_hip_tensor``: the fields of MMESimTensorBase (mme/mme_reference/sim_tensor_base.h:143-156)."""
    _fields_ = [("data", C.c_void_p),
                ("sizes", C.c_uint32 * MAX_TENSOR_DIMS),
                ("strides", C.c_uint32 * MAX_TENSOR_DIMS),
                ("dim", C.c_int32),
                ("dtype", C.c_int32),
                ("fp_bias", C.c_uint32),
                ("inf_nan_mode", C.c_int32)]


class ConvParams(C.Structure):
    """``mme_hip_conv_params``: ConvolutionParams (mme/mme_reference/convolution_params.h:7-29)."""
    _fields_ = [("dim", C.c_int32),
                ("padding_value", C.c_uint32),
                ("padding", C.c_int32 * 4),
                ("conv_stride", C.c_int32 * 4),
                ("dilation", C.c_int32 * 4),
                ("relu", C.c_int32)]


class Epilogue(C.Structure):
    """``mme_hip_epilogue``: descale + relu + cast fused behind a contraction."""
    _fields_ = [("scale_exp", C.c_int32),
                ("col_scale_exp", C.c_void_p),
                ("relu", C.c_int32),
                ("rounding_mode", C.c_int32),
                ("clip_fp", C.c_int32),
                ("clip_inf_in", C.c_int32),
                ("flush_denorms", C.c_int32)]


def make_tensor(data_ptr, sizes, dtype, fp_bias=0, inf_nan_mode=FULL_INF_NAN, strides=None, dim=None):
    """Build a descriptor.  ``sizes[0]`` is the contiguous dimension; missing trailing sizes are 1; default strides
    are dense (setStridesAndGetTensorSize, mme/mme_reference/sim_tensor_base.cpp:351-374)."""
    sizes = list(sizes)
    nd = len(sizes) if dim is None else dim
    sizes = sizes + [1] * (MAX_TENSOR_DIMS - len(sizes))
    if strides is None:
        strides, acc = [], 1
        for s in sizes:
            strides.append(acc)
            acc *= s
    else:
        strides = list(strides) + [0] * (MAX_TENSOR_DIMS - len(strides))
        for d in range(len([s for s in strides if s]), MAX_TENSOR_DIMS):
            strides[d] = strides[d - 1] * sizes[d - 1]
    t = Tensor()
    t.data = data_ptr
    for d in range(MAX_TENSOR_DIMS):
        t.sizes[d] = sizes[d]
        t.strides[d] = strides[d]
    t.dim = nd
    t.dtype = dtype
    t.fp_bias = fp_bias
    t.inf_nan_mode = inf_nan_mode
    return t


def make_conv_params(dim=2, padding=(0, 0, 0), stride=(1, 1, 1), dilation=(1, 1, 1), relu=False):
    p = ConvParams()
    p.dim = dim
    p.padding_value = 0
    pad = list(padding) + [0] * (4 - len(padding))
    st = list(stride) + [1] * (4 - len(stride))
    di = list(dilation) + [1] * (4 - len(dilation))
    for i in range(4):
        p.padding[i] = pad[i]
        p.conv_stride[i] = st[i]
        p.dilation[i] = di[i]
    p.relu = int(relu)
    return p


_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmme_hip.so")
_lib = None

vp = C.c_void_p
_TP = C.POINTER(Tensor)


def load_library():
    """Load ``csrc/libmme_hip.so``.  There is no CPU fallback: a missing library is an error."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("%s is missing: build it with intel_gaudi3_software_amd.build.build_library() "
                           "(hipcc --offload-arch=gfx950)" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    L.mme_hip_version.restype = C.c_char_p
    L.mme_hip_create.argtypes = [C.POINTER(vp), C.c_int, C.c_int, C.c_int, C.c_uint, C.c_uint32, vp, C.c_uint32]
    L.mme_hip_destroy.argtypes = [vp]
    L.mme_hip_destroy.restype = None
    L.mme_hip_last_error.argtypes = [vp]
    L.mme_hip_last_error.restype = C.c_char_p
    L.mme_hip_limit_num_of_threads.argtypes = [vp, C.c_uint]
    L.mme_hip_stream.argtypes = [vp]
    L.mme_hip_stream.restype = vp
    L.mme_hip_set_stream.argtypes = [vp, vp]
    L.mme_hip_synchronize.argtypes = [vp]
    L.mme_hip_set_wait_limit.argtypes = [vp, C.c_uint]
    L.mme_hip_clock_probe.argtypes = [vp, C.c_int]
    L.mme_hip_clock_probe_read.argtypes = [vp, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_int)]
    L.mme_hip_last_contraction_form.argtypes = [vp] + [C.POINTER(C.c_int)] * 4
    L.mme_hip_plan_batch_gemm.argtypes = [_TP, _TP, _TP, C.c_int, C.POINTER(Epilogue), C.c_int, C.c_int, C.POINTER(C.c_int), C.c_char_p, C.c_size_t]
    L.mme_hip_plan_convolution.argtypes = [_TP, _TP, _TP, _TP, C.POINTER(ConvParams), C.c_int, C.POINTER(Epilogue), C.c_int, C.c_int, C.POINTER(C.c_int),
                                           C.c_char_p, C.c_size_t]
    L.mme_hip_matrix_core_rate.argtypes = [vp, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]
    L.mme_hip_set_fp8_specials_policy.argtypes = [vp, C.c_int]
    L.mme_hip_set_operand_clip.argtypes = [vp, C.c_int, C.c_int]
    L.mme_hip_batch_gemm.argtypes = [vp, _TP, _TP, _TP, C.c_int, C.c_int, C.c_int, C.c_int]
    L.mme_hip_convolution.argtypes = [vp, _TP, _TP, _TP, _TP, C.POINTER(ConvParams), C.c_int, C.c_int, C.c_int, C.c_int]
    L.mme_hip_activation.argtypes = [vp, _TP, _TP] + [C.c_int] * 6
    L.mme_hip_memory_write.argtypes = [vp, _TP, _TP, C.c_int, C.c_int, C.c_int]
    L.mme_hip_memory_write_dev.argtypes = [vp, _TP, _TP, C.c_int, C.c_int, C.c_int]
    L.mme_hip_batch_gemm_dev.argtypes = [vp, _TP, _TP, _TP, C.c_int, C.POINTER(Epilogue)]
    L.mme_hip_batch_gemm_dev_noalloc.argtypes = [vp, _TP, _TP, _TP, C.c_int, C.POINTER(Epilogue)]
    L.mme_hip_convolution_dev.argtypes = [vp, _TP, _TP, _TP, _TP, C.POINTER(ConvParams), C.c_int, C.POINTER(Epilogue)]
    L.mme_hip_activation_dev.argtypes = [vp, _TP, _TP] + [C.c_int] * 6
    L.mme_hip_cast_from_fp32_dev.argtypes = [vp, vp, C.c_int, C.c_uint, C.c_int, vp, C.c_size_t, C.c_int, vp,
                                             C.c_size_t] + [C.c_int] * 5
    L.mme_hip_cast_to_fp32_dev.argtypes = [vp, vp, vp, C.c_int, C.c_uint, C.c_int, C.c_size_t, C.c_int, vp, C.c_size_t]
    L.mme_hip_absmax_dev.argtypes = [vp, vp, vp, C.c_size_t]
    _lib = L
    return L


def _planned(rc, form, err):
    if rc != 0:
        raise ValueError("%s (status %d)" % (err.value.decode(), rc))
    return {"large_tile": form[0], "tile_rows": form[1], "split_k": form[2], "wavefronts": form[3]}


def plan_batch_gemm(out, x, w, op, epilogue=None, num_cus=256, fp8_specials_policy=FP8_SPECIALS_CHECK):
    """Which kernel form ``mme_hip_batch_gemm_dev`` would launch for these descriptors (``mme_hip_plan_batch_gemm``): nothing
    runs, no GPU is needed.  The descriptors' data pointers only matter through their alignment (``make_tensor(4096, ...)``
    will do).  Raises ValueError with the library's message for a problem the real call would refuse."""
    lib = load_library()
    form, err = (C.c_int * 4)(), C.create_string_buffer(512)
    rc = lib.mme_hip_plan_batch_gemm(C.byref(out), C.byref(x), C.byref(w), op, C.byref(epilogue) if epilogue is not None else None, num_cus,
                                     fp8_specials_policy, form, err, 512)
    return _planned(rc, form, err)


def plan_convolution(out, x, w, y, params, op, epilogue=None, num_cus=256, fp8_specials_policy=FP8_SPECIALS_CHECK):
    """The same for ``mme_hip_convolution_dev`` (``mme_hip_plan_convolution``)."""
    lib = load_library()
    form, err = (C.c_int * 4)(), C.create_string_buffer(512)
    rc = lib.mme_hip_plan_convolution(C.byref(out), C.byref(x), C.byref(w), C.byref(y), C.byref(params), op,
                                      C.byref(epilogue) if epilogue is not None else None, num_cus, fp8_specials_policy, form, err, 512)
    return _planned(rc, form, err)
