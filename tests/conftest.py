import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    config.addinivalue_line("markers", "sanitizer: builds and runs the host-side C++ under -fsanitize=thread / address (CPU only)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as _oracle
    _oracle.lib()
    return _oracle


@pytest.fixture(scope="session")
def gpu():
    """Initialise the device through the C ABI.  No fallback: a missing library or device is a failure."""
    from backup_1_amd import capi
    capi.init()
    return capi
