import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def fw():
    """The ctypes binding of libflowwalker_hip.so (package directory has a hyphen in its name)."""
    return importlib.import_module("flowwalker-artifact_amd")


@pytest.fixture(scope="session")
def gpu(fw):
    """The binding, after checking that a device is visible.  GPU tests fail (not skip) without one."""
    assert fw.device_count() > 0, "no HIP device visible: GPU tests need a real MI355X"
    return fw
