import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    """Initialise the library on device 0; a missing library or GPU is an error, not a skip."""
    from ancora_cutile_amd import _lib
    _lib.init(0)
    return _lib
