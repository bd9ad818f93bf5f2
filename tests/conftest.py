import os
import sys

import pytest

# the tests compare implementations of one operator through the library's diagnostic switches, which take
# effect only in a process that asks for them before the library's first call
os.environ.setdefault("FASTMEM_DEBUG_HOOKS", "1")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def lib():
    """The C-ABI library; GPU tests call through it."""
    from fast_memory_amd import _lib
    return _lib.load()
