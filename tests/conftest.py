import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def dev():
    """cuda:0 with the kernel library initialised; GPU tests fail loudly without it."""
    import torch
    assert torch.cuda.is_available(), "GPU tests need a visible MI355X"
    from nnabla_amd import kernels
    kernels.init(0)
    return torch.device("cuda:0")
