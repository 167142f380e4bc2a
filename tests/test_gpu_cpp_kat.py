"""The C++ surface (include/mme_hip_calculator.h): the reference's own known-answer unit tests
(mme/tests/unit_tests/mme_unit_test.cpp:67-172, 394-519) restated against MmeHip::Calculator in tests/cpp/kat_calculator.cpp,
built by intel_gaudi3_software_amd.build.build_cpp_tests() and run here as a child process."""
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
