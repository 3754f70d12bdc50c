import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def hip():
    """Loads librai_hip.so and initialises device 0; fails loudly if either is missing."""
    from rai_amd import _lib, hip as hipmod

    _lib.load()
    assert hipmod.device_count() >= 1, "no HIP device visible"
    _lib.call("rai_hip_init", 0)
    return hipmod
