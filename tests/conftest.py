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


# Direct GPU-versus-oracle deviations that the full-size parity tests record, printed as one table
# at the end of the run (and asserted against their ceilings where they are recorded).
_DEVIATIONS = []


@pytest.fixture(scope="session")
def deviations():
    def record(config, what, value, ceiling):
        _DEVIATIONS.append((config, what, float(value), float(ceiling)))
        print("deviation  %-34s %-44s %.3e  (ceiling %.1e)" % (config, what, value, ceiling), flush=True)
        assert value <= ceiling, (config, what, value, ceiling)
    return record


def pytest_terminal_summary(terminalreporter):
    if not _DEVIATIONS:
        return
    terminalreporter.write_line("direct GPU-vs-oracle deviations (worst element per case)")
    for config, what, value, ceiling in _DEVIATIONS:
        terminalreporter.write_line("  %-34s %-44s %.3e  (ceiling %.1e)" % (config, what, value, ceiling))
