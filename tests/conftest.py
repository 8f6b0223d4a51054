import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs the HIP kernels)")


@pytest.fixture(scope="session")
def dev():
    """The HIP device; GPU tests fail (not skip) when the kernel library is missing."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    from areal_amd import _lib

    _lib.load()  # raises if libareal_hip.so has not been built
    return torch.device("cuda:0")
