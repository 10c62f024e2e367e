import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


class _Options:
    """Option switches of the library (moe_a2a_set_option) for one test; all back to 0 afterwards."""

    def __init__(self):
        from kernel_amd import _lib

        self._lib_mod = _lib
        self._lib = _lib.load()
        self._touched = set()

    def set(self, name, value):
        opt = getattr(self._lib_mod, "OPT_" + name)
        self._touched.add(opt)
        rc = self._lib.moe_a2a_set_option(opt, int(value))
        assert rc >= 0, rc

    def reset(self):
        for opt in self._touched:
            self._lib.moe_a2a_set_option(opt, 0)


@pytest.fixture
def options():
    o = _Options()
    yield o
    o.reset()
