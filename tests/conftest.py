import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (gfx950) and the built HIP kernel library")


@pytest.fixture
def emu_ops():
    """Routes the engine's operations to the CPU stand-in for the duration of a test."""
    from spyinfer_amd.kernels import ops
    from tests.emu_ops import EmuOps
    ops.install_test_double(EmuOps())
    yield
    ops.install_test_double(None)


@pytest.fixture(autouse=True)
def poisoned_cache_pool(monkeypatch):
    """Every cache pool that a test's engine makes is filled with NaN instead of zeros.  A slot is always written
    before it is read, so a correct engine never shows it; a read of a slot that was never written (a wrong page, a
    key beyond a request's length that is not masked) turns the logits into NaN instead of passing as a zero."""
    from spyinfer_amd.cache.storage import CacheStorage
    real = CacheStorage.__init__

    def init(self, *args, **kwargs):
        real(self, *args, **kwargs)
        self.fill(float("nan"))
    monkeypatch.setattr(CacheStorage, "__init__", init)
