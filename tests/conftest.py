import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oxh():
    """The shipped library, initialised on device 0.  GPU tests only."""
    from oxidize_amd import _lib
    lib = _lib.lib()
    _lib.check(lib.oxh_init(0))
    return lib
