"""Device storage: the Python mirror of the V file `storage/hip_d_hip.v`.

Follows `CudaStorage[T]` (storage/cuda_d_cuda.v:19-107): a raw device pointer
with byte size and element count, created from host memory with a blocking
copy, copied back with `cpu()` / `to_array()`, and released explicitly
(nothing frees on garbage collection in the reference; here `__del__` is a
safety net only).  A numpy array stands in for `CpuStorage[T]`.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import capi


@dataclass
class HipParams:
    """`@[params] HipParams{device_id int = 0}` (cf. CudaParams, storage/cuda_d_cuda.v:9-11)."""
    device_id: int = 0


_SUPPORTED = (np.float32, np.int8, np.int32, np.float64, np.uint8)


class HipStorage:
    """`HipStorage[T]{ptr voidptr; size int; count int; device_id int}`."""

    def __init__(self, ptr: int, size: int, count: int, dtype, device_id: int = 0):
        self.ptr = ptr
        self.size = size      # bytes
        self.count = count    # elements
        self.dtype = np.dtype(dtype)
        self.device_id = device_id

    # -- construction ------------------------------------------------------
    @staticmethod
    def empty(count: int, dtype, params: HipParams | None = None) -> "HipStorage":
        params = params or HipParams()
        dt = np.dtype(dtype)
        if dt.type not in _SUPPORTED:
            raise TypeError(f"HipStorage: unsupported element type {dt}")
        capi.call("vtl_hip_set_device", params.device_id)
        nbytes = int(count) * dt.itemsize
        ptr = C.c_void_p(0)
        if nbytes:
            capi.call("vtl_hip_malloc", C.byref(ptr), nbytes)
        return HipStorage(ptr.value or 0, nbytes, int(count), dt, params.device_id)

    @staticmethod
    def from_cpu(arr: np.ndarray, params: HipParams | None = None) -> "HipStorage":
        """`(cpu &CpuStorage[T]) hip(params) !&HipStorage[T]` (storage/cuda_d_cuda.v:32-55)."""
        flat = np.ascontiguousarray(arr).reshape(-1)
        st = HipStorage.empty(flat.size, flat.dtype, params)
        if st.size:
            capi.call("vtl_hip_memcpy_h2d", st.ptr, flat.ctypes.data, st.size)
        return st

    def hip(self, params: HipParams | None = None) -> "HipStorage":
        """Identity, for chaining (storage/cuda_d_cuda.v:62-65)."""
        return self

    # -- transfer back -------------------------------------------------------
    def cpu(self) -> np.ndarray:
        """`.cpu() !&CpuStorage[T]` (storage/cuda_d_cuda.v:68-81)."""
        if self.count and not self.ptr:
            raise capi.VtlHipError("HipStorage.cpu", capi.ERR_INVALID_ARG, "null pointer")
        out = np.empty(self.count, self.dtype)
        if self.size:
            capi.call("vtl_hip_memcpy_d2h", out.ctypes.data, self.ptr, self.size)
        return out

    def to_array(self) -> np.ndarray:
        """`.to_array() ![]T` (storage/cuda_d_cuda.v:84-95)."""
        return self.cpu()

    def release(self) -> None:
        """`.release()` (storage/cuda_d_cuda.v:98-102)."""
        if self.ptr:
            capi.call("vtl_hip_free", self.ptr)
            self.ptr = 0

    def __del__(self):  # safety net; the reference relies on explicit release()
        try:
            if getattr(self, "ptr", 0) and capi._lib is not None:
                capi._lib.vtl_hip_free(self.ptr)
                self.ptr = 0
        except Exception:
            pass


def hip_available() -> bool:
    """True when the library loads and reports at least one device."""
    try:
        return capi.device_count() > 0
    except (OSError, FileNotFoundError):
        return False
