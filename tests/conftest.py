import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle_mod():
    import oracle

    oracle.build()
    return oracle


@pytest.fixture(scope="session")
def blas():
    """The tensor-level API; fails (never skips) if the HIP library is missing."""
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import hpcdeepneuralnetworks_amd as pkg

    pkg._lib.lib()  # raises if libhpcdnn.so has not been built
    return pkg.blas
