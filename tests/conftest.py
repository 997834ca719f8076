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
