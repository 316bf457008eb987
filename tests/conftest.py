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


GUARD_BYTES = 4096
GUARD_BYTE = 0xA5


@pytest.fixture
def guard_bands(monkeypatch):
    """Every device buffer the test allocates through HipStorage (inputs, outputs, scales)
    sits between two patterned guard bands of 4 KiB, checked when the buffer is released and
    again at the end of the test: a kernel that writes before or past its output is caught,
    which exactly-sized allocations would let pass unseen.  The contract guarded is the
    reference's: a device call returns a status and never touches memory it was not given
    (storage/cuda_d_cuda.v:69-77)."""
    import ctypes as C
    import weakref

    import numpy as np

    from vtl_amd import capi
    from vtl_amd.storage import _SUPPORTED, HipParams, HipStorage

    live = {}          # id(storage) -> (weakref, base pointer, payload bytes)
    damaged = []

    def check(base, nbytes, what):
        for name, off in (("before", 0), ("after", GUARD_BYTES + nbytes)):
            band = np.empty(GUARD_BYTES, np.uint8)
            capi.call("vtl_hip_memcpy_d2h", band.ctypes.data, base + off, GUARD_BYTES)
            bad = np.flatnonzero(band != GUARD_BYTE)
            if bad.size:
                damaged.append(f"{what}: {bad.size} guard bytes {name} the buffer overwritten, first at offset "
                               f"{int(bad[0]) - (GUARD_BYTES if off == 0 else 0)} relative to its "
                               f"{'start' if off == 0 else 'end'}")

    def empty(count, dtype, params=None):
        params = params or HipParams()
        dt = np.dtype(dtype)
        if dt.type not in _SUPPORTED:
            raise TypeError(f"HipStorage: unsupported element type {dt}")
        capi.call("vtl_hip_set_device", params.device_id)
        nbytes = int(count) * dt.itemsize
        if not nbytes:
            return HipStorage(0, 0, int(count), dt, params.device_id)
        base = C.c_void_p(0)
        capi.call("vtl_hip_malloc", C.byref(base), nbytes + 2 * GUARD_BYTES)
        capi.call("vtl_hip_memset", base.value, GUARD_BYTE, GUARD_BYTES)
        capi.call("vtl_hip_memset", base.value + GUARD_BYTES + nbytes, GUARD_BYTE, GUARD_BYTES)
        st = HipStorage(base.value + GUARD_BYTES, nbytes, int(count), dt, params.device_id)
        live[id(st)] = (weakref.ref(st), base.value, nbytes)
        return st

    def release(self):
        rec = live.pop(id(self), None)
        if rec is None or not self.ptr:
            if self.ptr and rec is None:
                capi.call("vtl_hip_free", self.ptr)
            self.ptr = 0
            return
        _, base, nbytes = rec
        capi.call("vtl_hip_sync")
        check(base, nbytes, f"{self.dtype}[{self.count}]")
        capi.call("vtl_hip_free", base)
        self.ptr = 0

    def finalize(self):    # never hand an interior pointer to vtl_hip_free
        rec = live.pop(id(self), None)
        if rec is not None and getattr(self, "ptr", 0):
            capi._lib.vtl_hip_free(rec[1])
            self.ptr = 0

    monkeypatch.setattr(HipStorage, "empty", staticmethod(empty))
    monkeypatch.setattr(HipStorage, "release", release)
    monkeypatch.setattr(HipStorage, "__del__", finalize)
    yield damaged      # the list of findings so far (a test of the guard itself reads and clears it)
    capi.call("vtl_hip_sync")
    for key, (ref, base, nbytes) in list(live.items()):
        st = ref()
        check(base, nbytes, "buffer still allocated at the end of the test")
        capi.call("vtl_hip_free", base)
        if st is not None:
            st.ptr = 0
        live.pop(key, None)
    assert not damaged, "; ".join(damaged[:5])
