"""ctypes access to the CPU checkers (TEST INFRASTRUCTURE ONLY).

``oracle()`` loads ``oracle/libmme_oracle.so`` (the plain-C restatement, ``mme_oracle.c``) and ``ref()`` loads
``oracle/_ref/libmme_ref.so`` (the reference's own sources compiled by ``oracle/Makefile``; ``None`` when that
library has not been built).  Only tests, the smoke entry and the CPU-baseline leg of the benchmark import this
package; the product package never does.
"""
import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "libmme_oracle.so")
REF_SO = os.path.join(_HERE, "_ref", "libmme_ref.so")
REF_RMW_SO = os.path.join(_HERE, "_ref", "libmme_ref_rmw.so")

u8p, u16p, u32p, i32p, f32p = (C.POINTER(t) for t in (C.c_uint8, C.c_uint16, C.c_uint32, C.c_int32, C.c_float))
vp = C.c_void_p

_oracle = None
_ref = None


def build(with_ref=True):
    """Compile the checkers (gcc / g++ through oracle/Makefile).  The reference library is built only where the
    reference tree is present."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "oracle"])
    if with_ref and os.path.isdir(os.environ.get("MME_REFERENCE_ROOT", "/root/reference")):
        subprocess.check_call(["make", "-s", "-j8", "-C", _HERE, "ref",
                               "REF=" + os.environ.get("MME_REFERENCE_ROOT", "/root/reference")])
        # the drop-in demonstration links the MI355X library: built only where that has been built
        if os.path.exists(os.path.join(_HERE, "..", "intel_gaudi3_software_amd", "csrc", "libmme_hip.so")):
            subprocess.check_call(["make", "-s", "-j8", "-C", _HERE, "ref_dropin",
                                   "REF=" + os.environ.get("MME_REFERENCE_ROOT", "/root/reference")])


def oracle():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_SO):
            build(with_ref=False)
        L = C.CDLL(ORACLE_SO)
        L.orc_last_error.restype = C.c_char_p
        L.orc_fp8_to_fp32.restype = C.c_uint32
        L.orc_fp8_to_fp32.argtypes = [C.c_uint8] + [C.c_int] * 4
        L.orc_fp32_to_fp8.restype = C.c_uint8
        L.orc_fp32_to_fp8.argtypes = [C.c_uint32, C.c_int, C.c_int, C.c_int, C.c_int, C.c_uint32] + [C.c_int] * 5
        L.orc_fp32_to_bf16.restype = C.c_uint16
        L.orc_fp32_to_bf16.argtypes = [C.c_uint32, C.c_int, C.c_uint32, C.c_int, C.c_int, C.c_int]
        L.orc_fp32_to_fp32.restype = C.c_uint32
        L.orc_fp32_to_fp32.argtypes = [C.c_uint32] + [C.c_int] * 4
        L.orc_add_fp32.restype = C.c_uint32
        L.orc_add_fp32.argtypes = [C.c_uint32, C.c_uint32, C.c_int]
        L.orc_lfsr32.restype = C.c_uint32
        L.orc_lfsr32.argtypes = [C.c_uint32, C.c_uint32]
        L.orc_tree9.restype = C.c_uint32
        L.orc_tree9.argtypes = [u32p, u32p, C.c_int]
        L.orc_fma_vec_bf16.restype = C.c_uint32
        L.orc_fma_vec_bf16.argtypes = [vp, C.c_ssize_t, vp, C.c_ssize_t, C.c_size_t]
        L.orc_fma_vec_fp32.restype = C.c_uint32
        L.orc_fma_vec_fp32.argtypes = [vp, C.c_ssize_t, vp, C.c_ssize_t, C.c_size_t]
        L.orc_fma_vec_fp8.restype = C.c_uint32
        L.orc_fma_vec_fp8.argtypes = [vp, C.c_ssize_t, vp, vp, C.c_ssize_t, vp, C.c_size_t]
        L.orc_set_num_threads.argtypes = [C.c_int]
        L.orc_get_num_threads.restype = C.c_int
        L.orc_batch_gemm.argtypes = [vp, vp, vp, C.c_int]
        L.orc_convolution.argtypes = [vp, vp, vp, vp, vp, C.c_int, C.c_int]
        L.orc_activation.argtypes = [vp, vp] + [C.c_int] * 6 + [vp, C.c_uint32]
        L.orc_cast_from_fp32.argtypes = [vp, C.c_int, C.c_uint, C.c_int, vp, C.c_size_t, C.c_int, vp, C.c_size_t] + \
            [C.c_int] * 5
        L.orc_cast_to_fp32.argtypes = [vp, vp, C.c_int, C.c_uint, C.c_int, C.c_size_t, C.c_int, vp, C.c_size_t]
        L.orc_fp32_to_fp8_n.argtypes = [vp, vp, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_int, vp] + [C.c_int] * 5
        L.orc_fp8_to_fp32_n.argtypes = [vp, vp, C.c_size_t] + [C.c_int] * 4
        L.orc_fp32_to_bf16_n.argtypes = [vp, vp, C.c_size_t, C.c_int, vp, C.c_int, C.c_int, C.c_int]
        L.orc_fp32_to_fp32_n.argtypes = [vp, vp, C.c_size_t] + [C.c_int] * 4
        L.orc_add_fp32_n.argtypes = [vp, vp, vp, C.c_size_t, C.c_int]
        L.orc_tree9_n.argtypes = [vp, vp, vp, C.c_size_t, C.c_int]
        L.orc_memory_write.argtypes = [vp, vp, C.c_int, C.c_int, C.c_int]
        L.orc_cfp16_to_fp32.restype = C.c_uint32
        L.orc_cfp16_to_fp32.argtypes = [C.c_uint16, C.c_int, C.c_int, C.c_int]
        L.orc_fp32_to_cfp16.restype = C.c_uint16
        L.orc_fp32_to_cfp16.argtypes = [C.c_uint32, C.c_int, C.c_int, C.c_int, C.c_uint32] + [C.c_int] * 4
        L.orc_fp32_to_tf32.restype = C.c_uint32
        L.orc_fp32_to_tf32.argtypes = [C.c_uint32, C.c_int, C.c_int]
        L.orc_fma_vec_fp16.restype = C.c_uint32
        L.orc_fma_vec_fp16.argtypes = [vp, C.c_ssize_t, C.c_int, C.c_int, C.c_int, vp, C.c_ssize_t, C.c_int, C.c_int,
                                       C.c_int, C.c_size_t]
        L.orc_fma_vec_tf32.restype = C.c_uint32
        L.orc_fma_vec_tf32.argtypes = [vp, C.c_ssize_t, vp, C.c_ssize_t, C.c_size_t, C.c_int, C.c_int]
        L.orc_batch_gemm_clip.argtypes = [vp, vp, vp, C.c_int, C.c_int, C.c_int]
        L.orc_convolution_clip.argtypes = [vp, vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, C.c_int]
        L.orc_fp32_to_cfp16_n.argtypes = [vp, vp, C.c_size_t, C.c_int, C.c_int, C.c_int, vp] + [C.c_int] * 4
        L.orc_cfp16_to_fp32_n.argtypes = [vp, vp, C.c_size_t, C.c_int, C.c_int, C.c_int]
        L.orc_fp32_to_tf32_n.argtypes = [vp, vp, C.c_size_t, C.c_int, C.c_int]
        _oracle = L
    return _oracle


def ref():
    """The compiled reference, or None when oracle/_ref has not been built."""
    global _ref
    if _ref is None:
        if not os.path.exists(REF_SO):
            return None
        L = C.CDLL(REF_SO)
        L.ref_last_error.restype = C.c_char_p
        L.ref_set_num_threads.argtypes = [C.c_int]
        L.ref_batch_gemm.argtypes = [vp, vp, vp, C.c_int]
        L.ref_convolution.argtypes = [vp, vp, vp, vp, vp, C.c_int, C.c_int]
        L.ref_activation.argtypes = [vp, vp] + [C.c_int] * 6 + [vp, C.c_uint32, C.c_uint32]
        L.ref_fp32_to_fp8_n.argtypes = [vp, vp, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_int, vp] + [C.c_int] * 5
        L.ref_fp8_to_fp32_n.argtypes = [vp, vp, C.c_size_t] + [C.c_int] * 4
        L.ref_fp32_to_bf16_n.argtypes = [vp, vp, C.c_size_t, C.c_int, vp, C.c_int, C.c_int, C.c_int]
        L.ref_fp32_to_fp32_n.argtypes = [vp, vp, C.c_size_t] + [C.c_int] * 4
        L.ref_add_fp32_n.argtypes = [vp, vp, vp, C.c_size_t, C.c_int]
        L.ref_lfsr32.restype = C.c_uint32
        L.ref_lfsr32.argtypes = [C.c_uint32, C.c_uint32]
        L.ref_tree9_n.argtypes = [vp, vp, vp, C.c_size_t, C.c_int]
        L.ref_fma_vec.restype = C.c_uint32
        L.ref_fma_vec.argtypes = [vp, vp, C.c_uint, C.c_int, C.c_int, C.c_uint, C.c_uint, C.c_int, C.c_int]
        L.ref_compare_elements.argtypes = [vp, vp, vp, C.c_size_t, C.c_int, C.c_uint, C.c_int, C.c_uint]
        L.ref_compare_elements.restype = None
        L.ref_compare_tensors.argtypes = [vp, vp, C.c_uint, C.c_int, vp]
        if hasattr(L, "ref_compare_elements_partials"):
            L.ref_compare_elements_partials.argtypes = [vp, vp, vp, C.c_size_t, C.c_uint, C.c_int, C.c_uint, C.c_int, C.c_uint]
            L.ref_compare_elements_partials.restype = None
            L.ref_compare_tensors_partials.argtypes = [vp, vp, C.c_uint, C.c_uint, vp]
        L.ref_fma_vec_clip.restype = C.c_uint32
        L.ref_fma_vec_clip.argtypes = [vp, vp, C.c_uint, C.c_int, C.c_int, C.c_uint, C.c_uint] + [C.c_int] * 4
        L.ref_batch_gemm_clip.argtypes = [vp, vp, vp, C.c_int, C.c_int, C.c_int]
        L.ref_fp32_to_cfp16_n.argtypes = [vp, vp, C.c_size_t, C.c_int, C.c_int, C.c_int, vp] + [C.c_int] * 4
        L.ref_cfp16_to_fp32_n.argtypes = [vp, vp, C.c_size_t, C.c_int, C.c_int, C.c_int]
        L.ref_fp32_to_tf32_n.argtypes = [vp, vp, C.c_size_t, C.c_int, C.c_int]
        _ref = L
    return _ref


_ref_rmw = None


def ref_rmw():
    """The reference's memory-write reduction (executeOp), compiled at -O0 (see the Makefile), or None when not built."""
    global _ref_rmw
    if _ref_rmw is None:
        if not os.path.exists(REF_RMW_SO):
            return None
        L = C.CDLL(REF_RMW_SO)
        L.ref_memory_write_words.argtypes = [vp, vp, C.c_size_t] + [C.c_int] * 4
        L.ref_memory_write_words.restype = None
        _ref_rmw = L
    return _ref_rmw
