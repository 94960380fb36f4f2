import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_sessionstart(session):
    """The tests load the library that is built; it is built here only if there is none."""
    import __graft_entry__

    __graft_entry__.ensure_built()


def _gpu_count():
    try:
        from appy_amd.backends.hip import runtime as rt

        return rt.device_count()
    except Exception:
        return 0


@pytest.fixture(scope="session")
def gpu():
    """Skips when no GPU is visible; GPU tests must never fall back to a CPU path."""
    n = _gpu_count()
    if n < 1:
        pytest.skip("no GPU visible")
    return n
