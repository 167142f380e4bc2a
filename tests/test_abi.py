"""The C ABI library: it loads, exports every symbol include/mme_hip.h declares, and its argument checks that need no
device behave like the reference's assertions.  (No compute call is made here.)"""
import ctypes as C
import os
import re

import pytest

from intel_gaudi3_software_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(abi.LIB_PATH):
        pytest.skip("libmme_hip.so has not been built (python -m intel_gaudi3_software_amd.build)")
    return abi.load_library()


def _declared():
    text = open(os.path.join(ROOT, "include", "mme_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mme_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_entry_points():
    names = _declared()
    for must in ("mme_hip_create", "mme_hip_destroy", "mme_hip_batch_gemm", "mme_hip_convolution", "mme_hip_activation",
                 "mme_hip_memory_write", "mme_hip_memory_write_dev", "mme_hip_batch_gemm_dev", "mme_hip_convolution_dev", "mme_hip_cast_from_fp32_dev",
                 "mme_hip_cast_to_fp32_dev"):
        assert must in names


def test_library_exports_every_declared_symbol(lib):
    missing = [n for n in _declared() if not hasattr(lib, n)]
    assert not missing, missing
    assert b"gfx950" in lib.mme_hip_version()


def test_create_rejects_wrong_static_dims_and_chips(lib):
    h = C.c_void_p()
    # "dynamic value different than static value" (mme_reference_impl.cpp:143-144): checked before any device is touched
    assert lib.mme_hip_create(C.byref(h), abi.CHIP_GAUDI3, 4, 4, 0, 256, None, 0) == abi.EINVAL
    assert b"static value" in lib.mme_hip_last_error(None)
    assert lib.mme_hip_create(C.byref(h), abi.CHIP_GAUDI2, 5, 4, 0, 256, None, 0) == abi.EUNSUPPORTED
    assert lib.mme_hip_create(C.byref(h), 17, 5, 4, 0, 256, None, 0) == abi.EINVAL
    assert not h.value


def test_pod_layout_matches_header():
    # mme_hip_tensor: pointer + 5 + 5 uint32 + 4 int32 ; conv params: 2 + 12 + 1 int32 ; epilogue
    assert C.sizeof(abi.Tensor) == 8 + 4 * 10 + 4 * 4
    assert C.sizeof(abi.ConvParams) == 4 * 15
    assert abi.Tensor.sizes.offset == 8 and abi.Tensor.strides.offset == 28 and abi.Tensor.dim.offset == 48
    assert C.sizeof(abi.Epilogue) == 40 and abi.Epilogue.col_scale_exp.offset == 8


def test_headers_compile_as_c_and_cpp(tmp_path):
    """include/mme_hip.h is plain C; include/mme_hip_calculator.h is C++17 and needs nothing but the C header."""
    import subprocess
    inc = os.path.join(ROOT, "include")
    c_src = tmp_path / "use_c.c"
    c_src.write_text('#include "mme_hip.h"\nint f(void) { mme_hip_tensor t; t.dim = 2; return t.dim + MME_HIP_OP_AB; }\n')
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-I" + inc, str(c_src)])
    cpp_src = tmp_path / "use_cpp.cpp"
    cpp_src.write_text('#include "mme_hip_calculator.h"\n'
                       'void f(MmeHip::Calculator& c, MmeHip::Tensor& o, const MmeHip::Tensor& a, const MmeHip::Tensor& b, const MmeHip::ConvolutionParams& p)\n'
                       '{ c.doBatchGemm(o, a, b, MME_HIP_OP_AB); c.doConvolution(o, a, b, o, p, MME_HIP_OP_FWD); c.doBatchGemmDev(o, a, b, MME_HIP_OP_ABT); }\n')
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Werror", "-fsyntax-only", "-I" + inc, str(cpp_src)])


def test_reference_side_stub_compiles_against_the_reference_headers():
    """include/reference_stub/mme_reference_hip.cpp defines every CPUCalculator method of mme/mme_reference/mme_reference.h:108-191
    on top of MmeHip::Calculator; with the reference tree present it must pass the compiler's front end against the
    reference's own headers (MmeSimTensor, Matrix, ConvolutionParams, the enums)."""
    import subprocess
    ref = os.environ.get("MME_REFERENCE_ROOT", "/root/reference")
    if not os.path.isdir(os.path.join(ref, "mme", "mme_reference")):
        pytest.skip("the reference tree is not present")
    inc = ["mme", "mme/include", "mme/mme_reference", "mme/src/mme_common", "mme/src", "3rd-parties", "3rd-parties/spdlog/include",
           "coral-sim/header/gaudi3/fs_core", "coral-sim/header/gaudi2/fs_core"]
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-w", "-I" + os.path.join(ROOT, "include")] + ["-I" + os.path.join(ref, i) for i in inc]
    subprocess.check_call(cmd + [os.path.join(ROOT, "include", "reference_stub", "mme_reference_hip.cpp")])
    # every public method of the class is defined by the stub
    text = open(os.path.join(ROOT, "include", "reference_stub", "mme_reference_hip.cpp")).read()
    for m in ("CPUCalculator::CPUCalculator", "CPUCalculator::~CPUCalculator", "limitNumOfThreads", "doGemm", "doDma", "doBatchGemm", "doConvolution",
              "doActivation", "doMemoryWrite", "activationGemmlowp"):
        assert m in text
