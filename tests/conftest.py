import os
import sys

import pytest

# several tests steer the kernel generators through HELIUM_HIP_* overrides, which are only honoured in tuning mode
os.environ.setdefault("HELIUM_HIP_TUNING", "1")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu():
    """Initialises device 0 through the C ABI; GPU tests fail loudly if that is impossible."""
    from helium_amd import device

    device.init(0)
    return device
