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
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def ref(orc):
    r = orc.ref()
    if r is None:
        pytest.skip("oracle/_ref is not built (the reference tree is absent)")
    return r


@pytest.fixture(scope="session", autouse=True)
def _torch_runtime_first():
    """Tests use torch as plumbing (graph construction, device buffers) next to the library.
    PyTorch wheels carry their own HIP runtime; initialising it before libcoral_search.so
    touches the device keeps both on one runtime instance whatever order the tests run in."""
    try:
        import torch
        if torch.cuda.is_available():
            torch.cuda.init()
    except ImportError:
        pass
    yield
