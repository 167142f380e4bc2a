import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    import oracle
    return oracle.oracle()


@pytest.fixture(scope="session")
def ref():
    import oracle
    lib = oracle.ref()
    if lib is None:
        pytest.skip("oracle/_ref/libmme_ref.so is not built (needs the reference tree)")
    return lib


@pytest.fixture(scope="session")
def calc():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from intel_gaudi3_software_amd import HipCalculator
    c = HipCalculator()
    yield c
    c.close()
