import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _reset_dispatch_mode():
    # same per-test reset as the reference's conftest.py:4-7
    import sten_amd
    sten_amd.set_dispatch_failure("warn")
    yield
