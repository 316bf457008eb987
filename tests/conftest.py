import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def hip():
    """The product library on a real device.  GPU tests never fall back: a
    missing library or device is a failure, not a skip."""
    from vtl_amd import capi
    assert os.path.exists(capi.LIB_PATH), "libvtlhip.so is not built"
    n = capi.device_count()
    assert n > 0, "no HIP device visible: GPU tests need a GPU"
    capi.call("vtl_hip_set_device", 0)
    return capi
