"""A seeded sweep of ragged shapes through the C ABI: quantize / dequantize with
both scale modes and every alignment of the column count, the int8 linear with
every combination of scale modes, bias and ReLU, and the f64-accumulating
matmul in its four layouts.  The shapes are drawn once from fixed seeds, so the
set is the same in every run."""
import numpy as np
import pytest

import oracle
from helpers import CPU_THREADS, dev
from vtl_amd import capi
from vtl_amd.tensor import HipTensor, matmul_hip

pytestmark = pytest.mark.gpu


def test_quantize_dequantize_ragged_shapes(hip):
    rng = np.random.default_rng(51)
    for case in range(60):
        rows = int(rng.integers(1, 70))
        cols = int(rng.choice([1, 2, 3, 5, 31, 64, 100, 255, 256, 257, 1000, 1023, 1024, 1028, 4097, 5000, 70001]))
        per_row = bool(rng.integers(0, 2))
        x = (rng.standard_normal((rows, cols)) * 10.0 ** rng.integers(-3, 4)).astype(np.float32)
        if case % 7 == 0:
            x[rng.integers(0, rows), rng.integers(0, cols)] = np.nan
        if case % 11 == 0:
            x[rng.integers(0, rows)] = 0.0
        print("quantize", case, rows, cols, per_row, flush=True)
        X = dev(x)
        Q, S = X.quantize_i8(0 if per_row else -1)
        qr, sr = oracle.quantize(x, per_row)
        assert np.array_equal(Q.cpu(), qr), (rows, cols, per_row)
        assert np.array_equal(S.cpu().reshape(-1), sr.reshape(-1)), (rows, cols, per_row)
        D = Q.dequantize(S, 0 if per_row else -1)
        assert np.array_equal(D.cpu(), oracle.dequantize(qr, sr, per_row))
        for t in (X, Q, S, D):
            t.release()


def test_int8_linear_ragged_shapes(hip):
    rng = np.random.default_rng(52)
    for case in range(70):
        m = int(rng.integers(1, 300))
        n = int(rng.integers(1, 300))
        k = int(rng.choice([16, 32, 48, 112, 128, 144, 256, 272, 384, 512, 1000, 1024, 1040, 2048, 7, 33, 100]))
        sa_rows, sw_cols = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        relu, with_bias = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        a = rng.integers(-127, 128, (m, k), dtype=np.int8)
        w = rng.integers(-127, 128, (n, k), dtype=np.int8)
        sa = rng.uniform(0.5, 1.5, m if sa_rows else 1).astype(np.float32)
        sw = rng.uniform(0.5, 1.5, n if sw_cols else 1).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32) if with_bias else None
        print("linear", case, m, n, k, sa_rows, sw_cols, relu, with_bias, flush=True)
        A, W, SA, SW = dev(a), dev(w), dev(sa), dev(sw)
        B = dev(bias) if with_bias else None
        Y, Ci = HipTensor.empty([m, n], np.float32), HipTensor.empty([m, n], np.int32)
        capi.call("vtl_hip_gemm_i8_i32", A.ptr, W.ptr, Ci.ptr, m, n, k)
        acc = oracle.gemm_i8_i32(a, w, threads=CPU_THREADS)
        assert np.array_equal(Ci.cpu(), acc), (m, n, k)
        capi.call("vtl_hip_linear_i8_f32", A.ptr, SA.ptr, int(sa_rows), W.ptr, SW.ptr, int(sw_cols),
                  B.ptr if with_bias else None, Y.ptr, m, n, k, int(relu))
        sa_full = sa if sa_rows else np.full(m, sa[0], np.float32)
        sw_full = sw if sw_cols else np.full(n, sw[0], np.float32)
        assert np.array_equal(Y.cpu(), oracle.epilogue(acc, sa_full, sw_full, bias, relu=relu)), (m, n, k)
        for t in (A, W, SA, SW, Y, Ci) + ((B,) if with_bias else ()):
            t.release()


def test_matmul_ragged_shapes(hip):
    rng = np.random.default_rng(53)
    for case in range(40):
        m, n, k = (int(v) for v in rng.integers(1, 200, 3))
        ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        dt = np.float32 if case % 2 == 0 else np.float64
        # integer-valued operands: the result is exact in any order of summation
        a = rng.integers(-8, 9, (k, m) if ta else (m, k)).astype(dt)
        b = rng.integers(-8, 9, (n, k) if tb else (k, n)).astype(dt)
        print("matmul", case, m, n, k, ta, tb, dt.__name__, flush=True)
        A, B = dev(a), dev(b)
        C = matmul_hip(A, B, ta, tb)
        want = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
        assert np.array_equal(C.cpu(), want.astype(dt)), (m, n, k, ta, tb)
        for t in (A, B, C):
            t.release()
