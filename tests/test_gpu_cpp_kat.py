"""The C++ surface (include/mme_hip_calculator.h): the reference's own known-answer unit tests
(mme/tests/unit_tests/mme_unit_test.cpp:67-172, 394-519) restated against MmeHip::Calculator in tests/cpp/kat_calculator.cpp,
built by intel_gaudi3_software_amd.build.build_cpp_tests() and run here as a child process; and the drop-in demonstration
oracle/_ref/dropin_reference_types (tests/cpp/dropin_reference_types.cpp over the reference's own MmeSimTensor / Matrix /
CPUCalculator headers and the stub of include/reference_stub, the genuine calculator beside it under another name)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "kat_calculator")


@pytest.mark.gpu
def test_cpp_known_answers():
    assert os.path.exists(EXE), "tests/cpp/kat_calculator has not been built (python -m intel_gaudi3_software_amd.build)"
    r = subprocess.run([EXE], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=120)
    text = r.stdout.decode(errors="replace")
    print(text)
    assert r.returncode == 0, text
    assert text.count("ok    ") == 12 and "FAILED" not in text


@pytest.mark.gpu
def test_reference_classes_over_the_stub():
    """The reference's own tensor classes and CPUCalculator interface with the stub's methods behind them, compared in one
    program with the genuine reference calculator on the same tensor objects.  The program is built from the reference
    tree (oracle/Makefile, target ref_dropin); where it has not been built the test has nothing to run."""
    exe = os.path.join(ROOT, "oracle", "_ref", "dropin_reference_types")
    if not os.path.exists(exe):
        pytest.skip("oracle/_ref/dropin_reference_types has not been built (needs the reference tree: make -C oracle ref_dropin)")
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=300)
    text = r.stdout.decode(errors="replace")
    print(text)
    assert r.returncode == 0, text
    assert text.count("\nok ") + text.startswith("ok ") == 9 and "FAILED" not in text and "all ok" in text
