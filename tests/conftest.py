import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs through libxsmi355.so)")


@pytest.fixture(scope="session")
def gpu():
    """Initialises the library on device 0; a missing library or device is a failure, not a skip."""
    from xshinnosuke_amd import backend
    backend.init(0)
    return backend
