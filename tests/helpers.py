"""Shared helpers of the GPU parity tests."""
import json
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np

import oracle
from vtl_amd import capi
from vtl_amd.storage import HipStorage
from vtl_amd.tensor import HipTensor

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "kat_vectors.json")))
CPU_THREADS = min(16, os.cpu_count() or 1)


def f32_list(vs):
    return np.array([np.float32(float(v)) if isinstance(v, str) else np.float32(v) for v in vs], np.float32)


def rel_err(got: np.ndarray, ref: np.ndarray) -> float:
    """Relative error with the denominator guarded against cancellation:
    max |got - ref| / max(|ref|, 1e-6 * max|ref|)."""
    ref64 = ref.astype(np.float64)
    den = np.maximum(np.abs(ref64), 1e-6 * max(np.abs(ref64).max(), 1e-30))
    return float((np.abs(got.astype(np.float64) - ref64) / den).max())


def dev(a: np.ndarray) -> HipTensor:
    return HipTensor.from_host(a)


def quantize_with_scale_mt(x: np.ndarray, scale: np.ndarray, per_row: bool) -> np.ndarray:
    """Oracle quantize-with-scale, split over host threads (ctypes drops the GIL)."""
    x = np.ascontiguousarray(x, np.float32)
    rows = x.shape[0]
    if rows < 2 * CPU_THREADS:
        return oracle.quantize_with_scale(x, scale, per_row)
    out = np.empty(x.shape, np.int8)
    bounds = np.linspace(0, rows, CPU_THREADS + 1).astype(int)

    def work(i):
        lo, hi = bounds[i], bounds[i + 1]
        if hi > lo:
            out[lo:hi] = oracle.quantize_with_scale(x[lo:hi], scale[lo:hi] if per_row else scale, per_row)
    with ThreadPoolExecutor(CPU_THREADS) as ex:
        list(ex.map(work, range(CPU_THREADS)))
    return out


def raw_device_buffer(nbytes: int) -> HipStorage:
    return HipStorage.empty(nbytes, np.uint8)


def h2d(ptr: int, a: np.ndarray) -> None:
    a = np.ascontiguousarray(a)
    capi.call("vtl_hip_memcpy_h2d", ptr, a.ctypes.data, a.nbytes)


def d2h(ptr: int, shape, dtype) -> np.ndarray:
    out = np.empty(shape, dtype)
    capi.call("vtl_hip_memcpy_d2h", out.ctypes.data, ptr, out.nbytes)
    return out
