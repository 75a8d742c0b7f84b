import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu():
    """The GPU tests must run the HIP path: no device (or no native library) is a failure, not a skip."""
    from cinn_amd import runtime
    n = runtime.device_count()
    assert n > 0, "a test marked gpu ran without a visible GPU"
    return n


@pytest.fixture
def rng():
    return np.random.default_rng(1234)
