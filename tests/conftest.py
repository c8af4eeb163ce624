import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def lib():
    """The built C-ABI library; built once on demand when missing (CPU cross-compile)."""
    from chatlearn_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from chatlearn_amd.build import build
        build(verbose=False)
    return _lib.lib()


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from chatlearn_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail("libclgrpo.so missing on a GPU box: the HIP path cannot run")
    return torch.device("cuda:0")
