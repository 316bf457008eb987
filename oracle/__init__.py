"""ctypes loader for the CPU oracle (libvtloracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of bench.py, never by the product package.  The arithmetic
is documented in vtl_oracle.h / vtl_oracle.c next to this file.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libvtloracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile libvtloracle.so with gcc (make)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "libvtloracle.so"], check=True,
                   stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return _LIB_PATH


_NATIVE_PATH = os.path.join(_HERE, "_native", "libvtloracle_native.so")
_flags = "-O3 -march=x86-64-v3 -ffp-contract=off -fopenmp (oracle/Makefile)"


def use_native_build() -> str:
    """For the CPU-baseline leg of bench.py: compile the same source for the CPU
    of THIS machine (gcc -O3 -march=native -ffp-contract=off -fopenmp, about a
    second) and make later calls use it.  The shipped library is built for a
    generic x86-64-v3 target because it travels between machines.  Returns the
    flags in use; keeps the shipped build when gcc is missing or fails."""
    global _lib, _flags
    os.makedirs(os.path.dirname(_NATIVE_PATH), exist_ok=True)
    cmd = ["gcc", "-O3", "-march=native", "-ffp-contract=off", "-fno-fast-math", "-fopenmp", "-fPIC", "-std=c11",
           "-shared", "-o", _NATIVE_PATH, os.path.join(_HERE, "vtl_oracle.c"), "-lm"]
    try:
        subprocess.run(cmd, check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=120)
    except (OSError, subprocess.SubprocessError):
        return _flags
    _lib = None
    lib(_NATIVE_PATH)
    _flags = "-O3 -march=native -ffp-contract=off -fopenmp (built on this host)"
    return _flags


def build_flags() -> str:
    return _flags


def lib(path: str | None = None) -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if path is None and not os.path.exists(_LIB_PATH):
        build()
    L = C.CDLL(path or _LIB_PATH)
    i64, ci, vp, f32 = C.c_int64, C.c_int, C.c_void_p, C.c_float
    sig = {
        "vtl_ref_absmax_f32": (None, [vp, i64, i64, ci, vp]),
        "vtl_ref_scale_from_absmax": (f32, [f32]),
        "vtl_ref_quantize_one": (C.c_int8, [f32, f32]),
        "vtl_ref_quantize_f32_i8": (None, [vp, i64, i64, ci, vp, vp]),
        "vtl_ref_quantize_with_scale": (None, [vp, vp, i64, i64, ci, vp]),
        "vtl_ref_dequantize_i8_f32": (None, [vp, vp, i64, i64, ci, vp]),
        "vtl_ref_gemm_i8_i32": (None, [vp, vp, vp, i64, i64, i64, ci]),
        "vtl_ref_epilogue_f32": (None, [vp, vp, ci, vp, ci, vp, vp, i64, i64, ci]),
        "vtl_ref_linear_i8_f32": (None, [vp, vp, ci, vp, vp, ci, vp, vp, i64, i64, i64, ci, ci]),
        "vtl_ref_linear_f32_dynquant": (None, [vp, vp, vp, vp, vp, i64, i64, i64, ci, ci]),
        "vtl_ref_relu_f32": (None, [vp, i64]),
        "vtl_ref_linear_f32_via_f64": (None, [vp, vp, vp, vp, i64, i64, i64]),
        "vtl_ref_matmul_f32": (None, [vp, vp, vp, i64, i64, i64, ci, ci, ci]),
        "vtl_ref_matmul_f64": (None, [vp, vp, vp, i64, i64, i64, ci, ci, ci]),
        "vtl_ref_colsum_f32": (None, [vp, i64, i64, vp]),
        "vtl_ref_colsum_f64": (None, [vp, i64, i64, vp]),
        "vtl_ref_linear_backward_f32": (None, [vp, vp, vp, vp, vp, vp, i64, i64, i64, ci]),
        "vtl_ref_linear_backward_f64": (None, [vp, vp, vp, vp, vp, vp, i64, i64, i64, ci]),
        "vtl_ref_gemv_f32": (None, [vp, vp, vp, i64, i64]),
        "vtl_ref_gemv_f64": (None, [vp, vp, vp, i64, i64]),
        "vtl_ref_sigmoid_f32": (None, [vp, vp, i64]),
        "vtl_ref_sigmoid_f64": (None, [vp, vp, i64]),
        "vtl_ref_relu_f64": (None, [vp, i64]),
        "vtl_ref_quantize_f32_i8_mt": (None, [vp, i64, i64, ci, vp, vp, ci]),
        "vtl_ref_dequantize_i8_f32_mt": (None, [vp, vp, i64, i64, ci, vp, ci]),
        "vtl_ref_max_threads": (ci, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def _p(a):
    return None if a is None else a.ctypes.data


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


def max_threads() -> int:
    return int(lib().vtl_ref_max_threads())


def absmax(x: np.ndarray, per_row: bool) -> np.ndarray:
    x = _c(x, np.float32)
    rows, cols = x.shape
    out = np.empty(rows if per_row else 1, np.float32)
    lib().vtl_ref_absmax_f32(_p(x), rows, cols, int(per_row), _p(out))
    return out


def scale_from_absmax(a: float) -> np.float32:
    return np.float32(lib().vtl_ref_scale_from_absmax(C.c_float(float(a))))


def quantize_one(x: float, scale: float) -> int:
    return int(lib().vtl_ref_quantize_one(C.c_float(float(x)), C.c_float(float(scale))))


def quantize(x: np.ndarray, per_row: bool, threads: int = 1):
    x = _c(x, np.float32)
    rows, cols = x.shape
    q = np.empty((rows, cols), np.int8)
    s = np.empty(rows if per_row else 1, np.float32)
    lib().vtl_ref_quantize_f32_i8_mt(_p(x), rows, cols, int(per_row), _p(q), _p(s), threads)
    return q, s


def quantize_with_scale(x: np.ndarray, scale: np.ndarray, per_row: bool) -> np.ndarray:
    x = _c(x, np.float32)
    scale = _c(scale, np.float32)
    rows, cols = x.shape
    assert scale.size == (rows if per_row else 1)
    q = np.empty((rows, cols), np.int8)
    lib().vtl_ref_quantize_with_scale(_p(x), _p(scale), rows, cols, int(per_row), _p(q))
    return q


def dequantize(q: np.ndarray, scale: np.ndarray, per_row: bool, threads: int = 1) -> np.ndarray:
    q = _c(q, np.int8)
    scale = _c(scale, np.float32)
    rows, cols = q.shape
    assert scale.size == (rows if per_row else 1)
    x = np.empty((rows, cols), np.float32)
    lib().vtl_ref_dequantize_i8_f32_mt(_p(q), _p(scale), rows, cols, int(per_row), _p(x), threads)
    return x


def gemm_i8_i32(A: np.ndarray, Bt: np.ndarray, threads: int = 1) -> np.ndarray:
    A = _c(A, np.int8)
    Bt = _c(Bt, np.int8)
    M, K = A.shape
    N, K2 = Bt.shape
    assert K == K2
    Cm = np.empty((M, N), np.int32)
    lib().vtl_ref_gemm_i8_i32(_p(A), _p(Bt), _p(Cm), M, N, K, threads)
    return Cm


def epilogue(acc, sa, sw, bias, relu=False) -> np.ndarray:
    acc = _c(acc, np.int32)
    M, N = acc.shape
    sa = _c(np.atleast_1d(sa), np.float32)
    sw = _c(np.atleast_1d(sw), np.float32)
    assert sa.size in (1, M) and sw.size in (1, N)
    b = None if bias is None else _c(bias, np.float32).reshape(-1)
    assert b is None or b.size == N
    Y = np.empty((M, N), np.float32)
    lib().vtl_ref_epilogue_f32(_p(acc), _p(sa), int(sa.size == M),
                               _p(sw), int(sw.size == N), _p(b), _p(Y), M, N, int(relu))
    return Y


def linear_i8_f32(A, sa, Wq, sw, bias, relu=False, threads: int = 1) -> np.ndarray:
    A = _c(A, np.int8)
    Wq = _c(Wq, np.int8)
    M, K = A.shape
    N, K2 = Wq.shape
    assert K == K2
    sa = _c(np.atleast_1d(sa), np.float32)
    sw = _c(np.atleast_1d(sw), np.float32)
    assert sa.size in (1, M) and sw.size in (1, N)
    b = None if bias is None else _c(bias, np.float32).reshape(-1)
    Y = np.empty((M, N), np.float32)
    lib().vtl_ref_linear_i8_f32(_p(A), _p(sa), int(sa.size == M), _p(Wq), _p(sw), int(sw.size == N),
                                _p(b), _p(Y), M, N, K, int(relu), threads)
    return Y


def linear_i8_requant(A, sa, Wq, sw, bias, relu=False, threads: int = 1):
    """The int8 linear followed by per-row quantization of its f32 output: the
    hand-off between two int8 layers.  Composition of linear_i8_f32 and quantize."""
    y = linear_i8_f32(A, sa, Wq, sw, bias, relu=relu, threads=threads)
    q, s = quantize(y, True, threads=threads)
    return q, s, y


def linear_f32_dynquant(X, Wq, sw, bias, relu=False, threads: int = 1) -> np.ndarray:
    X = _c(X, np.float32)
    Wq = _c(Wq, np.int8)
    M, K = X.shape
    N, K2 = Wq.shape
    assert K == K2
    sw = _c(sw, np.float32)
    assert sw.size == N
    b = None if bias is None else _c(bias, np.float32).reshape(-1)
    Y = np.empty((M, N), np.float32)
    lib().vtl_ref_linear_f32_dynquant(_p(X), _p(Wq), _p(sw), _p(b), _p(Y), M, N, K, int(relu), threads)
    return Y


def relu(x: np.ndarray) -> np.ndarray:
    y = np.array(x, dtype=np.float32, copy=True, order="C")
    lib().vtl_ref_relu_f32(_p(y), y.size)
    return y


def linear_f32_via_f64(X, W, bias) -> np.ndarray:
    X = _c(X, np.float32)
    W = _c(W, np.float32)
    M, K = X.shape
    N, K2 = W.shape
    assert K == K2
    b = None if bias is None else _c(bias, np.float32).reshape(-1)
    Y = np.empty((M, N), np.float32)
    lib().vtl_ref_linear_f32_via_f64(_p(X), _p(W), _p(b), _p(Y), M, N, K)
    return Y


def _suffix(dtype) -> str:
    dt = np.dtype(dtype)
    if dt == np.float32:
        return "f32"
    if dt == np.float64:
        return "f64"
    raise TypeError(f"matmul oracle covers float32 and float64, not {dt}")


def matmul(a: np.ndarray, b: np.ndarray, trans_a: bool = False, trans_b: bool = False,
           threads: int = 1) -> np.ndarray:
    """op(a) . op(b) through f64, rounded once to the operands' dtype."""
    sfx = _suffix(a.dtype)
    a = _c(a, a.dtype)
    b = _c(b, a.dtype)
    M, K = (a.shape[1], a.shape[0]) if trans_a else a.shape
    K2, N = (b.shape[1], b.shape[0]) if trans_b else b.shape
    assert K == K2, (a.shape, b.shape, trans_a, trans_b)
    c = np.empty((M, N), a.dtype)
    getattr(lib(), f"vtl_ref_matmul_{sfx}")(_p(a), _p(b), _p(c), M, N, K, int(trans_a), int(trans_b),
                                            threads)
    return c


def colsum(x: np.ndarray) -> np.ndarray:
    sfx = _suffix(x.dtype)
    x = _c(x, x.dtype)
    out = np.empty(x.shape[1], x.dtype)
    getattr(lib(), f"vtl_ref_colsum_{sfx}")(_p(x), x.shape[0], x.shape[1], _p(out))
    return out


def linear_backward(grad: np.ndarray, x: np.ndarray, w: np.ndarray, threads: int = 1):
    """(dx[M,K], dw[N,K], db[N]) of y = x.W^T + b for the upstream gradient grad[M,N]."""
    sfx = _suffix(grad.dtype)
    dt = grad.dtype
    grad, x, w = _c(grad, dt), _c(x, dt), _c(w, dt)
    M, N = grad.shape
    K = x.shape[1]
    assert x.shape == (M, K) and w.shape == (N, K)
    dx, dw, db = np.empty((M, K), dt), np.empty((N, K), dt), np.empty(N, dt)
    getattr(lib(), f"vtl_ref_linear_backward_{sfx}")(_p(grad), _p(x), _p(w), _p(dx), _p(dw), _p(db),
                                                     M, N, K, threads)
    return dx, dw, db


def gemv(a: np.ndarray, x: np.ndarray) -> np.ndarray:
    sfx = _suffix(a.dtype)
    a, x = _c(a, a.dtype), _c(x, a.dtype)
    assert a.ndim == 2 and x.shape == (a.shape[1],)
    y = np.empty(a.shape[0], a.dtype)
    getattr(lib(), f"vtl_ref_gemv_{sfx}")(_p(a), _p(x), _p(y), a.shape[0], a.shape[1])
    return y


def sigmoid(x: np.ndarray) -> np.ndarray:
    sfx = _suffix(x.dtype)
    x = _c(x, x.dtype)
    y = np.empty_like(x)
    getattr(lib(), f"vtl_ref_sigmoid_{sfx}")(_p(x), _p(y), x.size)
    return y


def relu_f64(x: np.ndarray) -> np.ndarray:
    y = np.array(x, dtype=np.float64, copy=True, order="C")
    lib().vtl_ref_relu_f64(_p(y), y.size)
    return y
