import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (test infrastructure; built on demand with gcc)."""
    from oracle import yko
    yko.lib()
    return yko


@pytest.fixture(scope="session")
def native():
    """The product library through its ctypes binding; fails loudly if it is not built."""
    from yasakani_amd import native as n
    n.lib()
    return n
