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


class _Knobs:
    """Environment switches of the library for one test: the library reads its
    VTL_HIP_* switches once, so every change here is followed by
    vtl_hip_reload_env()."""

    def __init__(self, monkeypatch):
        self._mp = monkeypatch

    def _reload(self):
        from vtl_amd import capi
        capi.call("vtl_hip_reload_env")

    def setenv(self, name, value):
        self._mp.setenv(name, value)
        self._reload()

    def delenv(self, name, raising=True):
        self._mp.delenv(name, raising=raising)
        self._reload()


@pytest.fixture
def knobs(monkeypatch):
    k = _Knobs(monkeypatch)
    yield k
    monkeypatch.undo()
    k._reload()
