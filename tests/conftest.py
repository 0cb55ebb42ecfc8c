import importlib
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    import rmi_oracle

    return rmi_oracle


@pytest.fixture(scope="session")
def rmi():
    """The product package (its directory name is not a Python identifier)."""
    return importlib.import_module("rust-model-inference_amd")


@pytest.fixture(scope="session")
def hip(rmi):
    """The loaded C-ABI library wrapper, initialised on device 0 (GPU tests only)."""
    rmi.init(0)
    return rmi


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
