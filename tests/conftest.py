import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
for extra in (os.path.dirname(os.path.abspath(__file__)), os.path.join(ROOT, "oracle")):   # util.py; the oracle's loader
    if extra not in sys.path:
        sys.path.insert(0, extra)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle_lib
    return oracle_lib.load()


@pytest.fixture(scope="session")
def backend():
    """One handle for the whole GPU session (a fresh process = a fresh HIP context)."""
    from ml_dataflow_amd import Backend
    be = Backend(device_id=0, num_streams=8)
    yield be
    be.close()
