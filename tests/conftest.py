import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle_lib():
    import oracle
    oracle.build()
    return oracle


@pytest.fixture(scope="session")
def gpu():
    """Initialises device 0 through the C ABI; fails (never skips) when the library or the GPU is missing."""
    from thor_amd import runtime
    n = runtime.device_count()
    assert n >= 1, "no HIP device visible: GPU tests must run on the MI355X box"
    runtime.set_device(0)
    return runtime
