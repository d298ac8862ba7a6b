import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU checker (test infrastructure)."""
    from oracle import oracle as o
    o.lib()
    return o


@pytest.fixture(scope="session")
def hgemm_lib():
    """The shipped library through its C ABI; built beforehand, never built inside a test."""
    import cuda_hgemm_amd
    return cuda_hgemm_amd.library()


@pytest.fixture(scope="session")
def vendor_lib():
    import cuda_hgemm_amd
    return cuda_hgemm_amd.vendor_library()


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("a GPU test was selected but no GPU is visible")
    return torch.device("cuda:0")
