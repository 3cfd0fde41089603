import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def backend():
    """One HIP backend for the whole GPU session (one process, one device)."""
    import splash_amd
    b = splash_amd.Backend(0)
    yield b
    b.close()
