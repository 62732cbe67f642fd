import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950); runs on the GPU box only")


@pytest.fixture(scope="session")
def gpu():
    """Initialise the HIP library on device 0; a missing GPU or library is an error, not a skip."""
    from shrike_amd import runtime
    runtime.init(0)
    return runtime
