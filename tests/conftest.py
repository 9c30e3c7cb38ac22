import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs through the native HIP library)")


@pytest.fixture(scope="session")
def orc():
    from oracle.cpu import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def dn():
    """The native library, bound to device 0.  GPU tests only."""
    from darknet_amd import api, lib
    L = lib.load()
    api.set_gpu(0)
    return L
