import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def mlk():
    """The product package with its HIP library loaded; GPU tests only."""
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import muxi_native_layout_kernels_amd as pkg
    from muxi_native_layout_kernels_amd import _lib
    _lib.load()
    return pkg
