import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


# FG_INTERPRETED=1: the GPU parity tests run on the CPU, kernels executed by the interpreter of tests/emu/ (see
# tests/emu/session.py; tests/test_interpreted_suite.py starts such runs).  The HIP stand-in has to be bound before
# torch is imported, hence here, at the top of the first file pytest loads.
INTERPRETED = os.environ.get("FG_INTERPRETED") == "1"
if INTERPRETED:
    sys.path.insert(0, os.path.join(ROOT, "tests", "emu"))
    import session as _interp_session
    sys.path.pop(0)
    _interp_session.install()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_terminal_summary(terminalreporter):
    if INTERPRETED:
        terminalreporter.write_line("interpreted kernel launches: %d" % _interp_session.DEVICE.total_launches)


@pytest.fixture(autouse=INTERPRETED)
def _interpreter_between_tests():
    yield
    if INTERPRETED:
        err = _interp_session.between_tests()
        assert err is None, "the interpreter refused a launch:\n%s" % err


@pytest.fixture(scope="session")
def gpu():
    """cuda:0 with the native library loaded; fails (never skips) when either is missing."""
    import torch

    if INTERPRETED:
        return torch.device("cpu")
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from flaggems_amd import _C

    _C.lib()  # raises if libfg_mi355.so is not built
    return torch.device("cuda:0")


class _FgEnv:
    """Sets or removes FG_* switches and has the library read them again (it reads the environment
    once, not per call)."""

    def __init__(self):
        self._saved = {}

    def _reload(self):
        from flaggems_amd import _C

        _C.lib().fg_reload_options()

    def setenv(self, name, value):
        self._saved.setdefault(name, os.environ.get(name))
        os.environ[name] = value
        self._reload()

    def delenv(self, name, raising=False):
        self._saved.setdefault(name, os.environ.get(name))
        os.environ.pop(name, None)
        self._reload()

    def restore(self):
        for name, old in self._saved.items():
            if old is None:
                os.environ.pop(name, None)
            else:
                os.environ[name] = old
        self._reload()


@pytest.fixture
def fg_env():
    env = _FgEnv()
    yield env
    env.restore()
