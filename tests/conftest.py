import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def O():
    """The CPU checker (oracle/oracle.py)."""
    import oracle
    return oracle


@pytest.fixture(scope="session")
def D():
    """The product: ctypes mirror of the C++ front-end; fails loudly when the native libraries are missing."""
    import dali_amd
    return dali_amd


@pytest.fixture(scope="session")
def gpu(D):
    """Initialises the device through the C ABI; a GPU test without a device is an error, not a skip."""
    from dali_amd._native import hip, hip_check
    hip_check(hip.dali_hip_init(0), "dali_hip_init")
    return hip


@pytest.fixture()
def rng():
    return np.random.RandomState(1234)


def golden(name):
    import json
    with open(os.path.join(ROOT, "tests", "golden", name)) as f:
        return json.load(f)
