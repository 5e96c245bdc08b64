import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (test infrastructure), using a few host threads for speed.

    Thread count never changes results: threads only split independent rows/heads."""
    import oracle

    oracle.lib()
    oracle.set_threads(min(8, os.cpu_count() or 1))
    return oracle
