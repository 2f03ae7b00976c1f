import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def hip():
    """The HIP kernel table; GPU tests fail (not skip) when it cannot be created."""
    import torch

    assert torch.cuda.is_available(), "GPU test selected but no GPU is visible"
    from pfeife_amd.hip import HipKernels

    return HipKernels()


@pytest.fixture(scope="session")
def oracle():
    from oracle.kernels_oracle import OracleKernels

    return OracleKernels("cpu")
