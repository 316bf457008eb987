"""Seeded random shapes through every int8 entry point, against the oracle.

The fixed-shape parity tests pin the boundaries the kernels were written
around; these draw shapes blindly (any K, odd included, any M and N across the
routing thresholds) so that a boundary nobody listed is still crossed.  Same
bar: int32 sums, int8 codes and f32 outputs bit-equal to the oracle's.
"""
import numpy as np
import pytest

import oracle
from helpers import CPU_THREADS, dev
from vtl_amd.tensor import HipTensor, gemm_i8_hip, linear_i8_hip, linear_f32_dynquant_hip

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("guard_bands")]


def _draw_shape(rng):
    """M, N, K spread over decades; half of the K are multiples of 16."""
    m = int(rng.choice([1, 2, 3, 5, 8, 9, 31, 32, 33, 64, 100, 129, 256, 300]))
    if rng.random() < 0.4:
        m = int(rng.integers(1, 301))
    n = int(np.exp(rng.uniform(0, np.log(20000)))) if rng.random() < 0.3 else int(rng.integers(1, 20001))
    k = int(np.exp(rng.uniform(0, np.log(9000)))) if rng.random() < 0.3 else int(rng.integers(1, 9001))
    if rng.random() < 0.5:
        k = max(16, k & ~15)
    while m * n * k > 1.5e9:          # keeps the CPU oracle to a fraction of a second per case
        n = max(1, n // 2)
    return m, n, k


@pytest.mark.parametrize("block", range(8))
def test_random_shapes_int8_matmul_and_linear(hip, block):
    rng = np.random.Generator(np.random.Philox(1000 + block))
    for _ in range(25):
        m, n, k = _draw_shape(rng)
        a = rng.integers(-127, 128, (m, k), dtype=np.int8)
        bt = rng.integers(-127, 128, (n, k), dtype=np.int8)
        sa = (rng.uniform(0.5, 1.5, m) / 127).astype(np.float32)
        sb = (rng.uniform(0.5, 1.5, n) / 127).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32)
        ref = oracle.gemm_i8_i32(a, bt, threads=CPU_THREADS)
        A, B, SA, SB, BI = dev(a), dev(bt), dev(sa), dev(sb), dev(bias)
        Cm = HipTensor.empty([m, n], np.int32)
        gemm_i8_hip(Cm, A, B)
        assert np.array_equal(Cm.cpu(), ref), (m, n, k)
        relu = bool(rng.integers(0, 2))
        y = linear_i8_hip(A, SA, B, SB, BI, relu=relu)
        assert np.array_equal(y.cpu(), oracle.epilogue(ref, sa, sb, bias, relu=relu)), (m, n, k)
        for h in (A, B, SA, SB, BI, Cm, y):
            h.release()


@pytest.mark.parametrize("block", range(4))
def test_random_shapes_linear_with_quantization_on_the_fly(hip, block):
    rng = np.random.Generator(np.random.Philox(2000 + block))
    for _ in range(25):
        m, n, k = _draw_shape(rng)
        x = (rng.standard_normal((m, k)) * np.exp(rng.uniform(-20, 20, (m, 1)))).astype(np.float32)
        w = rng.integers(-127, 128, (n, k), dtype=np.int8)
        sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32) if rng.random() < 0.7 else None
        relu = bool(rng.integers(0, 2))
        X, W, SW = dev(x), dev(w), dev(sw)
        BI = dev(bias) if bias is not None else None
        y = linear_f32_dynquant_hip(X, W, SW, BI, relu=relu)
        want = oracle.linear_f32_dynquant(x, w, sw, bias, relu=relu, threads=CPU_THREADS)
        assert np.array_equal(y.cpu(), want), (m, n, k)
        for h in (X, W, SW, BI, y):
            if h is not None:
                h.release()


@pytest.mark.parametrize("block", range(3))
def test_random_decode_shapes_quantized_inside_the_launch(hip, block):
    """2 to 32 tokens, hundreds to thousands of weight rows, K any multiple of 256 up to 8192:
    the shapes around the launch whose first workgroups quantize the tokens for the others.  Row magnitudes
    spread over 17 decades, zero rows, staging buffers that come and go between calls (so a
    later call finds other codes at an address an earlier one used)."""
    rng = np.random.Generator(np.random.Philox(2500 + block))
    for _ in range(16):
        m = int(rng.integers(2, 33))
        n = int(rng.integers(2048, 20001)) if rng.random() < 0.6 else int(rng.integers(128, 2048))
        k = 256 * int(rng.integers(1, 33))
        while m * n * k > 1.5e9:
            n = max(2048, n // 2)
            k = max(256, (k // 2) & ~255)
        x = (rng.standard_normal((m, k)) * np.exp(rng.uniform(-20, 20, (m, 1)))).astype(np.float32)
        if rng.random() < 0.4:
            x[int(rng.integers(0, m))] = 0.0
        w = rng.integers(-127, 128, (n, k), dtype=np.int8)
        sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32) if rng.random() < 0.7 else None
        relu = bool(rng.integers(0, 2))
        X, W, SW = dev(x), dev(w), dev(sw)
        BI = dev(bias) if bias is not None else None
        want = oracle.linear_f32_dynquant(x, w, sw, bias, relu=relu, threads=CPU_THREADS)
        for _rep in range(2):
            y = linear_f32_dynquant_hip(X, W, SW, BI, relu=relu)
            assert np.array_equal(y.cpu(), want), (m, n, k)
            y.release()
        for h in (X, W, SW, BI):
            if h is not None:
                h.release()


@pytest.mark.parametrize("block", range(4))
def test_random_shapes_quantize_dequantize_absmax(hip, block):
    """Row counts and row lengths drawn blindly (odd lengths, single rows and columns,
    rows from a few bytes to hundreds of KiB), per row and per tensor, magnitudes
    spread over 40 decades from row to row."""
    rng = np.random.Generator(np.random.Philox(3000 + block))
    for _ in range(20):
        cols = int(np.exp(rng.uniform(0, np.log(200000))))
        rows = int(np.exp(rng.uniform(0, np.log(20000))))
        while rows * cols > 3_000_000:
            rows = max(1, rows // 2)
        x = (rng.standard_normal((rows, cols)) * np.exp(rng.uniform(-46, 46, (rows, 1)))).astype(np.float32)
        x[rng.random((rows, cols)) < 0.002] *= 20
        flat = x.reshape(-1)
        flat[: min(4, flat.size)] = np.array([0.5, 1.5, -2.5, 3.5], np.float32)[: min(4, flat.size)]
        if rows > 3:
            x[rows // 2] = 0.0                      # an all-zero row: scale 0
        t = dev(x)
        for axis in (0, -1):
            per_row = axis == 0
            am = t.absmax(axis)
            assert np.array_equal(am.cpu(), oracle.absmax(x, per_row)), (rows, cols, axis)
            q, s = t.quantize_i8(axis)
            qr, sr = oracle.quantize(x, per_row, threads=CPU_THREADS)
            assert np.array_equal(s.cpu(), sr), (rows, cols, axis)
            assert np.array_equal(q.cpu(), qr), (rows, cols, axis)
            d = q.dequantize(s, axis)
            assert np.array_equal(d.cpu(), oracle.dequantize(qr, sr, per_row), equal_nan=True), (rows, cols, axis)
            for h in (am, q, s, d):
                h.release()
        t.release()
