import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def fk():
    """The product binding.  GPU tests fail loudly if the HIP library or device is missing."""
    import fusekit_amd.native as native

    if not native.has_device():
        pytest.fail("GPU test selected but no HIP device is visible: " + native.lib.fk_last_error().decode())
    return native
