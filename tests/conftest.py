import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session", autouse=True)
def _built_libraries():
    """Tests load what is built; they build only when nothing is there."""
    from d2conv3d_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from d2conv3d_amd.build import build_library
        build_library()
    from oracle import cpu
    cpu.build()
    yield


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
