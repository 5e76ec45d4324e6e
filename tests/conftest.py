import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "autodiff-ir-rust_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def hip_device():
    """The product device.  Fails loudly (no fallback) when the library or the GPU is missing."""
    from adhip import HipDevice
    return HipDevice(0)


@pytest.fixture()
def oracle_device():
    from oracle.interp import OracleDevice
    return OracleDevice()
