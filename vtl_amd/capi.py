"""ctypes binding of libvtlhip.so: one Python function per C-ABI entry point.

This is the same surface the V binding declares with `fn C.vtl_hip_*`; see
include/vtl_hip.h for the contract of every call.  There is no CPU fallback
here: if the library is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libvtlhip.so")

OK = 0
ERR_INVALID_ARG = 1
ERR_NO_DEVICE = 2
ERR_RUNTIME = 3
ERR_OUT_OF_MEMORY = 4
ERR_UNSUPPORTED = 5

_i64, _ci, _vp, _sz = C.c_int64, C.c_int, C.c_void_p, C.c_size_t
_pp = C.POINTER(C.c_void_p)

# name -> (restype, argtypes); kept in step with include/vtl_hip.h
SIGNATURES = {
    "vtl_hip_device_count": (_ci, [C.POINTER(_ci)]),
    "vtl_hip_set_device": (_ci, [_ci]),
    "vtl_hip_device_info": (_ci, [C.c_char_p, _sz, C.POINTER(_ci), C.POINTER(_ci)]),
    "vtl_hip_malloc": (_ci, [_pp, _sz]),
    "vtl_hip_free": (_ci, [_vp]),
    "vtl_hip_memcpy_h2d": (_ci, [_vp, _vp, _sz]),
    "vtl_hip_memcpy_d2h": (_ci, [_vp, _vp, _sz]),
    "vtl_hip_memcpy_d2d": (_ci, [_vp, _vp, _sz]),
    "vtl_hip_memset": (_ci, [_vp, _ci, _sz]),
    "vtl_hip_sync": (_ci, []),
    "vtl_hip_set_stream": (_ci, [_vp]),
    "vtl_hip_get_stream": (_ci, [_pp]),
    "vtl_hip_event_create": (_ci, [_pp]),
    "vtl_hip_event_destroy": (_ci, [_vp]),
    "vtl_hip_event_record": (_ci, [_vp]),
    "vtl_hip_event_elapsed_ms": (_ci, [_vp, _vp, C.POINTER(C.c_float)]),
    "vtl_hip_absmax_f32": (_ci, [_vp, _i64, _i64, _ci, _vp]),
    "vtl_hip_quantize_f32_i8": (_ci, [_vp, _i64, _i64, _ci, _vp, _vp]),
    "vtl_hip_quantize_with_scale_f32_i8": (_ci, [_vp, _vp, _i64, _i64, _ci, _vp]),
    "vtl_hip_dequantize_i8_f32": (_ci, [_vp, _vp, _i64, _i64, _ci, _vp]),
    "vtl_hip_gemm_i8_i32": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci]),
    "vtl_hip_linear_i8_f32": (_ci, [_vp, _vp, _ci, _vp, _vp, _ci, _vp, _vp, _ci, _ci, _ci, _ci]),
    "vtl_hip_linear_i8_requant": (_ci, [_vp, _vp, _ci, _vp, _vp, _ci, _vp, _ci, _vp, _vp, _vp, _ci, _ci, _ci]),
    "vtl_hip_gemm_tile_choice": (_ci, [_ci, _ci, _ci, _ci, C.POINTER(_ci), C.POINTER(_ci), C.POINTER(_ci),
                                       C.POINTER(_ci)]),
    "vtl_hip_linear_f32_dynquant_workspace": (_sz, [_ci, _ci]),
    "vtl_hip_linear_f32_dynquant": (_ci, [_vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp, _sz]),
    "vtl_hip_linear_f32_dynquant_noalloc": (_ci, [_vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci]),
    "vtl_hip_matmul_f32": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci]),
    "vtl_hip_matmul_f64": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci]),
    "vtl_hip_linear_f32": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci]),
    "vtl_hip_linear_f64": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci]),
    "vtl_hip_colsum_f32": (_ci, [_vp, _i64, _i64, _vp]),
    "vtl_hip_colsum_f64": (_ci, [_vp, _i64, _i64, _vp]),
    "vtl_hip_linear_backward_f32": (_ci, [_vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci]),
    "vtl_hip_linear_backward_f64": (_ci, [_vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci]),
    "vtl_hip_relu_f32": (_ci, [_vp, _i64]),
    "vtl_hip_relu_f64": (_ci, [_vp, _i64]),
    "vtl_hip_gemv_f32": (_ci, [_vp, _vp, _vp, _i64, _i64]),
    "vtl_hip_gemv_f64": (_ci, [_vp, _vp, _vp, _i64, _i64]),
    "vtl_hip_sigmoid_f32": (_ci, [_vp, _vp, _i64]),
    "vtl_hip_sigmoid_f64": (_ci, [_vp, _vp, _i64]),
    "vtl_hip_strerror": (C.c_char_p, [_ci]),
    "vtl_hip_last_error": (C.c_char_p, []),
    "vtl_hip_version": (C.c_char_p, []),
    "vtl_hip_reload_env": (_ci, []),
}


class VtlHipError(RuntimeError):
    """A C-ABI call returned a non-zero status (the V side wraps it in `error(...)`)."""

    def __init__(self, fn: str, status: int, detail: str = ""):
        self.fn = fn
        self.status = status
        msg = f"{fn} failed with status {status}"
        if detail:
            msg += f": {detail}"
        super().__init__(msg)


_lib = None


def lib() -> C.CDLL:
    """Load libvtlhip.so (built beforehand by vtl_amd.build); never falls back."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with `python -m vtl_amd.build` (needs hipcc)")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def call(name: str, *args) -> None:
    """Call an int-returning entry point and raise VtlHipError on failure."""
    L = lib()
    st = getattr(L, name)(*args)
    if st != OK:
        detail = L.vtl_hip_strerror(st).decode()
        last = L.vtl_hip_last_error().decode()
        if st in (ERR_RUNTIME, ERR_OUT_OF_MEMORY, ERR_NO_DEVICE) and last:
            detail += " [" + last + "]"
        raise VtlHipError(name, st, detail)


def status(name: str, *args) -> int:
    """Call an entry point and return its raw status (for error-path tests)."""
    return int(getattr(lib(), name)(*args))


def device_count() -> int:
    n = _ci(0)
    st = lib().vtl_hip_device_count(C.byref(n))
    return int(n.value) if st == OK else 0


def device_info():
    name = C.create_string_buffer(256)
    cu, mhz = _ci(0), _ci(0)
    call("vtl_hip_device_info", name, 256, C.byref(cu), C.byref(mhz))
    return name.value.decode(), int(cu.value), int(mhz.value)


def version() -> str:
    return lib().vtl_hip_version().decode()
