import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; runs the HIP path through the C ABI")


@pytest.fixture(scope="session")
def H():
    """The CPU oracle device module (oracle/hostref.py)."""
    from oracle import hostref
    hostref.load()
    return hostref


@pytest.fixture(scope="session")
def G():
    """The HIP device module; fails (never skips) when the library is missing."""
    from deepnet_amd import hip, native
    native.load()
    native.check(native.load().dnh_init(0))
    return hip


@pytest.fixture
def rng():
    return np.random.default_rng(123)
