import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def device():
    """The HIP library initialised on device 0. Fails (never skips) when the
    library or the device is missing, so a GPU run cannot pass on a fallback."""
    from webgpt_amd import blocks
    dev = blocks.Device(0)
    blocks.initializeOperations(dev)
    yield dev
    blocks.destroyOperations()
