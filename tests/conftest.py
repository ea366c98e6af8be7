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
    from oracle import oracle as o
    o.build()
    return o


@pytest.fixture(scope="session")
def ctx():
    """HIP-backed Context; fails (not skips) when the library or the GPU is missing."""
    import metaltile_amd as m
    return m.Context(0)


@pytest.fixture(scope="session")
def runner():
    import metaltile_amd as m
    return m.GpuRunner(0)
