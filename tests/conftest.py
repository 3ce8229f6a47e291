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
    """The loaded C-ABI library; GPU tests fail loudly if it is missing or finds no device."""
    from bidmat_amd import hip_abi, device
    lib = hip_abi.load()
    assert device.device_available(), "libbidmathip.so loaded but no HIP device is visible"
    return lib
