import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    import oracle
    oracle.lib()
    oracle.set_threads(min(16, oracle.max_threads()))
    return oracle


@pytest.fixture(scope="session")
def hip():
    """numpy-level facade over the C-ABI of libsliced_hip.so on device 0."""
    from sliced_amd import numpy_api
    numpy_api.init(0)
    return numpy_api
