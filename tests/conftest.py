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
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this process")
    return torch.device("cuda:0")


@pytest.fixture
def gemm_override():
    """Forces a tile shape on wc_batched_gemm / a choice between the two shifted-operand kernels
    through the library's test hook, and restores the defaults afterwards."""
    from pytorch_winoconv_amd import _lib
    lib = _lib.load()

    def force(config=-1, rows_mode=1):
        _lib.check(lib.wc_test_gemm_override(config, rows_mode))
    yield force
    _lib.check(lib.wc_test_gemm_override(-1, 1))
