import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "cuda-mace_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def cabi():
    """The ctypes binding of the HIP library; GPU tests call the kernels through it."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from cuda_mace import _cabi

    return _cabi
