import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    """cuda:0 with the native library loaded; fails (never skips) when either is missing."""
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from flaggems_amd import _C

    _C.lib()  # raises if libfg_mi355.so is not built
    return torch.device("cuda:0")
