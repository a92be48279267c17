import os
import sys

import pytest

# the library's test hook (wc_test_gemm_override) works only in a process that opts in before its first call
os.environ.setdefault("WINOCONV_TEST_HOOKS", "1")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    # the tests load what is built; only a tree in which nothing has been built yet is built here
    from pytorch_winoconv_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()


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

    from pytorch_winoconv_amd import engine

    def force(config=-1, rows_mode=1):
        _lib.check(lib.wc_test_gemm_override(config, rows_mode))
        engine._SETUPS.clear()              # workspace sizes are kept per problem, and some settings change them
    yield force
    _lib.check(lib.wc_test_gemm_override(-1, 1))
    engine._SETUPS.clear()


@pytest.fixture(params=["compiled", "ctypes"])
def host_layer(request, monkeypatch):
    """Runs a test once through the compiled host layer (the pybind11 module MakePytorchBackend) and once
    through the ctypes binding of the same C ABI."""
    from pytorch_winoconv_amd import engine
    if request.param == "compiled" and engine._ext is None:
        pytest.fail("the compiled host layer MakePytorchBackend is not built (pytorch_winoconv_amd.build())")
    monkeypatch.setattr(engine, "USE_EXT", request.param == "compiled")
    return request.param
