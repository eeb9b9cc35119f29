import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    """Initialises libmjt.so on device 0 for the GPU parity tests."""
    from jittor_amd import _lib
    _lib.init(0)
    yield _lib
    _lib.sync()


@pytest.fixture(scope="module")
def compile_only():
    """libmjt.so in compile-only mode: kernels are specialised and compiled
    for gfx950, nothing is launched (no GPU needed)."""
    from jittor_amd import _lib
    _lib.init(-1)
    yield _lib
    _lib.shutdown()
