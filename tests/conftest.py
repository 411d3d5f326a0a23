import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950); run with -m gpu")


@pytest.fixture(scope="session")
def wkf():
    """The ctypes binding of the in-tree library (fails loudly when it is not built)."""
    from helpers import load_package
    return load_package()


@pytest.fixture(scope="session")
def planner(wkf):
    """A device with no GPU behind it: kernels are generated and compiled, never run."""
    return wkf.Device.planner()


@pytest.fixture(scope="session")
def gpu(wkf):
    """The real device.  No skip and no fallback: a GPU test without a GPU is an error.
    WKF_TEST_PLAN_ONLY=1 swaps in a plan-only device: every test then stops (skipped) right after
    its kernels are generated and compiled, which fills the in-tree kernel cache on a machine with
    no GPU; it never produces a pass."""
    if os.environ.get("WKF_TEST_PLAN_ONLY") == "1":
        return wkf.Device.planner()
    return wkf.Device.new(0)
