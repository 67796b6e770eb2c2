import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 device (runs the HIP kernels through the C ABI)")


@pytest.fixture(scope="session")
def be():
    """One backend for the whole GPU session (one process on the card)."""
    import moe4all_amd as m

    backend = m.Backend(0)
    yield backend
    backend.close()
