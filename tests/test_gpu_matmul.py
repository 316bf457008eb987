"""Device matmul with f64 accumulation (la.matmul la/la.v:38-55, gate_matmul
autograd/gates_blas.v:6-23), the unquantized Linear forward and
LinearGate.backward (nn/gates/layers/linear.v:57-79) against the CPU oracle.

Bar: the device sums the same f64 products in another order, so the f64 sums
agree to ~1e-16 relative and the results rounded to f32 agree except where a
sum lies that close to a rounding boundary: at most one unit in the last
place, on a tiny fraction of elements (far inside the 1e-5 relative tolerance
of the f32 outputs of this path).  Integer-valued operands make every order
exact, and there the comparison is bit for bit at full size."""
import numpy as np
import pytest

import oracle
from helpers import CPU_THREADS, dev
from vtl_amd import capi
from vtl_amd.layers import (linear_backward_hip_f32, linear_forward_hip_exact, matmul_gate_backward_hip,
                            matmul_hip_host)
from vtl_amd.tensor import colsum_hip, linear_backward_hip, linear_hip, matmul_hip

pytestmark = pytest.mark.gpu


def ulp_diff(a, b):
    it = np.int32 if a.dtype == np.float32 else np.int64
    return np.abs(a.view(it).astype(np.int64) - b.view(it).astype(np.int64))


def assert_close_to_oracle(got, want, abs_products=None):
    assert got.shape == want.shape and got.dtype == want.dtype
    if got.dtype == np.float32:
        d = ulp_diff(got, want)
        assert d.max() <= 1, f"max ulp distance {d.max()}"
        assert (d > 0).mean() < 1e-3, f"{(d > 0).mean():.2e} of the elements differ"
    else:
        # f64 results: 2^-52 per operation over the K-term sum of |a||b|
        assert np.all(np.abs(got - want) <= 1e-13 * abs_products)


def run_matmul(A, B, ta, tb):
    a, b = dev(A), dev(B)
    c = matmul_hip(a, b, ta, tb)
    out = c.cpu()
    for t in (a, b, c):
        t.release()
    return out


SHAPES = [(1, 1, 1), (2, 3, 4), (2, 2, 2), (17, 33, 65), (64, 256, 784), (128, 128, 16), (130, 70, 250),
          (256, 1024, 96), (1, 512, 300), (300, 1, 77), (513, 255, 1030)]


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_matmul_shapes_and_layouts(hip, dt, ta, tb):
    rng = np.random.default_rng(21)
    for (M, N, K) in SHAPES:
        A = rng.standard_normal((K, M) if ta else (M, K)).astype(dt)
        B = rng.standard_normal((N, K) if tb else (K, N)).astype(dt)
        print("matmul", dt.__name__, ta, tb, M, N, K, flush=True)
        got = run_matmul(A, B, ta, tb)
        want = oracle.matmul(A, B, ta, tb, threads=CPU_THREADS)
        absprod = None
        if dt == np.float64:
            absprod = np.abs(A.T if ta else A) @ np.abs(B.T if tb else B)
        assert_close_to_oracle(got, want, absprod)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_split_k_paths(hip, dt, knobs):
    """Few output tiles and a long K slice K over the grid; forced slice counts cover
    ragged K, edge tiles and the unsplit fallback."""
    rng = np.random.default_rng(27)
    cases = [(256, 4096, 11008, False, False, None), (256, 1024, 4096, False, True, None),
             (64, 64, 2048, True, False, None), (100, 70, 1000, False, True, "3"), (128, 192, 4096, True, True, "5"),
             (33, 65, 777, False, False, "16"), (64, 128, 96, False, True, "4")]
    for (M, N, K, ta, tb, force) in cases:
        if force is None:
            knobs.delenv("VTL_HIP_MATMUL_SPLITS", raising=False)
        else:
            knobs.setenv("VTL_HIP_MATMUL_SPLITS", force)
        A = rng.standard_normal((K, M) if ta else (M, K)).astype(dt)
        B = rng.standard_normal((N, K) if tb else (K, N)).astype(dt)
        print("split-K", dt.__name__, M, N, K, ta, tb, force, flush=True)
        got = run_matmul(A, B, ta, tb)
        want = oracle.matmul(A, B, ta, tb, threads=CPU_THREADS)
        absprod = np.abs(A.T if ta else A).astype(np.float64) @ np.abs(B.T if tb else B).astype(np.float64)
        assert_close_to_oracle(got, want, absprod)
        # integer-valued operands: bit for bit whatever the slicing
        Ai, Bi = np.rint(A * 4).astype(dt), np.rint(B * 4).astype(dt)
        exact = (Ai.T if ta else Ai).astype(np.float64) @ (Bi.T if tb else Bi).astype(np.float64)
        assert np.array_equal(run_matmul(Ai, Bi, ta, tb), exact.astype(dt))
    # the Linear form keeps bias and ReLU after the sliced sum
    knobs.delenv("VTL_HIP_MATMUL_SPLITS", raising=False)
    x = rng.standard_normal((128, 4096)).astype(dt)
    w = (rng.standard_normal((256, 4096)) * 0.05).astype(dt)
    b = rng.standard_normal(256).astype(dt)
    xd, wd, bd = dev(x), dev(w), dev(b.reshape(1, -1))
    y = linear_hip(xd, wd, bd, relu=True)
    ref = oracle.matmul(x, w, False, True) + b
    assert_close_to_oracle(y.cpu(), np.where(ref < 0, dt(0), ref).astype(dt),
                           np.abs(x).astype(np.float64) @ np.abs(w.T).astype(np.float64) + np.abs(b))
    for t in (xd, wd, bd, y):
        t.release()


@pytest.mark.parametrize("tile", ["64", "128"])
def test_forced_tile_sizes(hip, tile, knobs):
    """VTL_HIP_MATMUL_TILE forces the 64x64 or the 128x128 tile kernel: whole and ragged
    tiles, all four layouts, both give the oracle's result (integers bit for bit)."""
    knobs.setenv("VTL_HIP_MATMUL_TILE", tile)
    rng = np.random.default_rng(int(tile))
    for (M, N, K, ta, tb) in [(256, 384, 128, False, True), (300, 200, 96, True, False), (129, 65, 260, True, True),
                              (1, 1, 1, False, False), (640, 512, 64, False, False)]:
        A = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
        B = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
        got = run_matmul(A, B, ta, tb)
        want = oracle.matmul(A, B, ta, tb, threads=CPU_THREADS)
        absprod = np.abs(A.T if ta else A).astype(np.float64) @ np.abs(B.T if tb else B).astype(np.float64)
        assert_close_to_oracle(got, want, absprod)
        Ai, Bi = np.rint(A * 4).astype(np.float32), np.rint(B * 4).astype(np.float32)
        exact = (Ai.T if ta else Ai).astype(np.float64) @ (Bi.T if tb else Bi).astype(np.float64)
        assert np.array_equal(run_matmul(Ai, Bi, ta, tb), exact.astype(np.float32))


def test_reference_literals(hip):
    # la/la_test.v:30-37
    a = np.array([[1.0, 0], [0.0, 1]])
    b = np.array([[4.0, 1], [2.0, 2]])
    assert np.array_equal(matmul_hip_host(a, b), b)
    assert np.array_equal(matmul_hip_host(a.astype(np.float32), b.astype(np.float32)), b.astype(np.float32))
    # la/la_test.v:39-57: rank-3 and vector operands are refused
    with pytest.raises(ValueError):
        matmul_hip_host(np.zeros((2, 2, 4)), np.zeros((2, 4, 2)))
    with pytest.raises(ValueError):
        matmul_hip_host(a, np.array([1.0, 2]))
    with pytest.raises(ValueError, match="Invalid shapes for matrix multiplication"):
        matmul_hip_host(np.zeros((2, 3)), np.zeros((2, 3)))
    # benchmarks/vs_numpy/matmul_bench.v:28-33 at its largest size, against exact integers
    n = 512
    i, j = np.indices((n, n))
    ai, bi = (i + j) % 7, (i * j) % 5
    got = matmul_hip_host(ai * 0.01, bi * 0.02)
    want_int = ai.astype(np.int64) @ bi.astype(np.int64)
    assert np.all(np.abs(got - want_int * 2e-4) <= 1e-12 * np.maximum(want_int, 1))


@pytest.mark.parametrize("M,N,K,ta,tb", [(4096, 4096, 4096, False, True), (4096, 4096, 4096, False, False),
                                         (2048, 4096, 1024, True, False), (1000, 1500, 2100, True, True),
                                         (256, 11008, 4096, False, True)])
def test_integer_valued_operands_exact_at_full_size(hip, M, N, K, ta, tb):
    """Operands in [-8, 8]: every partial sum is an integer below 2^24, so any
    summation order gives the same f32 and f64; numpy's f64 BLAS supplies it."""
    rng = np.random.default_rng(22)
    Ai = rng.integers(-8, 9, (K, M) if ta else (M, K)).astype(np.float64)
    Bi = rng.integers(-8, 9, (N, K) if tb else (K, N)).astype(np.float64)
    want = (Ai.T if ta else Ai) @ (Bi.T if tb else Bi)
    assert np.abs(want).max() < 2 ** 24
    print("exact f32", M, N, K, ta, tb, flush=True)
    got32 = run_matmul(Ai.astype(np.float32), Bi.astype(np.float32), ta, tb)
    assert np.array_equal(got32, want.astype(np.float32))
    if M * N <= 2048 * 4096:
        print("exact f64", M, N, K, ta, tb, flush=True)
        assert np.array_equal(run_matmul(Ai, Bi, ta, tb), want)


def test_full_size_random_against_oracle_rows(hip):
    """4096^3 f32 with normal operands; the oracle restates a band of rows."""
    rng = np.random.default_rng(23)
    M = N = K = 4096
    A = rng.standard_normal((M, K)).astype(np.float32)
    W = rng.standard_normal((N, K)).astype(np.float32)
    got = run_matmul(A, W, False, True)
    rows = np.r_[0:24, 2040:2056, 4072:4096]
    want = oracle.matmul(A[rows], W, False, True, threads=CPU_THREADS)
    assert_close_to_oracle(got[rows], want)
    # linearity in the first operand holds exactly for a power-of-two factor
    got2 = run_matmul(A * np.float32(0.25), W, False, True)
    assert np.array_equal(got2, got * np.float32(0.25))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_linear_forward_with_bias_and_relu(hip, dt):
    rng = np.random.default_rng(24)
    for (M, N, K) in [(1, 2, 3), (64, 256, 784), (33, 130, 257), (256, 1024, 512)]:
        x = rng.standard_normal((M, K)).astype(dt)
        w = (rng.standard_normal((N, K)) * 0.05).astype(dt)
        b = rng.standard_normal(N).astype(dt)
        if dt == np.float32:
            want = oracle.linear_f32_via_f64(x, w, b)
        else:
            want = oracle.matmul(x, w, False, True) + b
        absprod = np.abs(x).astype(np.float64) @ np.abs(w.T).astype(np.float64) + np.abs(b)
        assert_close_to_oracle(linear_forward_hip_exact(x, w, b), want, absprod)
        xd, wd, bd = dev(x), dev(w), dev(b.reshape(1, -1))
        y = linear_hip(xd, wd, bd, relu=True)
        assert_close_to_oracle(y.cpu(), np.where(want < 0, dt(0), want).astype(dt), absprod)
        y0 = linear_hip(xd, wd, None)
        want0 = oracle.matmul(x, w, False, True)
        assert_close_to_oracle(y0.cpu(), want0, absprod)
        for t in (xd, wd, bd, y, y0):
            t.release()
    # autograd_cuda/device_session_test.v:34-47 literals, CPU reference within 1e-9
    x = np.array([[1.0, 2.0, 3.0]])
    w = np.array([[0.1, 0.2, 0.3], [0.4, 0.5, 0.6]])
    b = np.array([[0.01, 0.02]])
    assert np.all(np.abs(linear_forward_hip_exact(x, w, b) - [[1.41, 3.22]]) < 1e-9)


@pytest.mark.parametrize("rows,cols", [(0, 5), (1, 1), (7, 3), (256, 4096), (300, 1001), (65536, 256),
                                       (100000, 4), (5000, 130), (64, 11008)])
@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_column_sums(hip, dt, rows, cols):
    rng = np.random.default_rng(25)
    x = rng.standard_normal((rows, cols)).astype(dt)
    xd = dev(x) if rows else None
    if rows == 0:
        from vtl_amd.tensor import HipTensor
        out = HipTensor.empty([1, cols], dt)
        capi.call("vtl_hip_colsum_f32" if dt == np.float32 else "vtl_hip_colsum_f64", None, 0, cols, out.ptr)
        assert not out.cpu().any()
        out.release()
        return
    s = colsum_hip(xd)
    got = s.cpu().reshape(-1)
    want = oracle.colsum(x)
    assert_close_to_oracle(got, want, np.abs(x).sum(axis=0))
    xd.release()
    s.release()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_linear_backward_against_oracle(hip, dt):
    rng = np.random.default_rng(26)
    for (M, N, K) in [(1, 2, 3), (64, 256, 784), (37, 130, 65), (256, 1024, 4096), (512, 4096, 1024)]:
        g = rng.standard_normal((M, N)).astype(dt)
        x = rng.standard_normal((M, K)).astype(dt)
        w = (rng.standard_normal((N, K)) * 0.05).astype(dt)
        print("backward", dt.__name__, M, N, K, flush=True)
        want = oracle.linear_backward(g, x, w, threads=CPU_THREADS)
        gd, xd, wd = dev(g), dev(x), dev(w)
        outs = linear_backward_hip(gd, xd, wd)
        g64, x64, w64 = np.abs(g).astype(np.float64), np.abs(x).astype(np.float64), np.abs(w).astype(np.float64)
        bounds = (g64 @ w64, g64.T @ x64, g64.sum(axis=0))
        for got_t, want_a, bnd in zip(outs, want, bounds):
            assert_close_to_oracle(got_t.cpu().reshape(want_a.shape), want_a, bnd)
        # gradients that are not required are not computed
        only_dw = linear_backward_hip(gd, xd, wd, need_dx=False, need_db=False)
        assert only_dw[0] is None and only_dw[2] is None
        assert np.array_equal(only_dw[1].cpu(), outs[1].cpu())
        for t in (gd, xd, wd, *outs, only_dw[1]):
            t.release()


def test_linear_backward_host_entry(hip, monkeypatch):
    # operands of autograd_cuda/device_session_test.v:52-60; gradients worked by hand
    g = np.array([[1.0, 0.5]], np.float32)
    x = np.array([[1.0, 2.0, 3.0]], np.float32)
    w = np.array([[0.1, 0.2, 0.3], [0.4, 0.5, 0.6]], np.float32)
    monkeypatch.delenv("VTL_HIP_BACKWARD", raising=False)
    with pytest.raises(RuntimeError, match="VTL_HIP_BACKWARD"):
        linear_backward_hip_f32(g, x, w, True)
    monkeypatch.setenv("VTL_USE_HIP", "1")
    monkeypatch.setenv("VTL_HIP_BACKWARD", "1")
    d_in, d_w, d_b = linear_backward_hip_f32(g, x, w, True)
    assert d_in.shape == (1, 3) and d_w.shape == (2, 3) and d_b.shape == (1, 2)
    assert np.allclose(d_in, [[0.3, 0.45, 0.6]], rtol=1e-6)
    assert np.array_equal(d_w, [[1, 2, 3], [0.5, 1, 1.5]]) and np.array_equal(d_b, [[1, 0.5]])
    # the reference's CUDA test asks for 1e-6 agreement with the CPU gradients (device_session_test.v:62-80)
    want = oracle.linear_backward(g.astype(np.float64), x.astype(np.float64), w.astype(np.float64))
    got = linear_backward_hip_f32(g.astype(np.float64), x.astype(np.float64), w.astype(np.float64), True)
    for a, b in zip(got, want):
        assert np.all(np.abs(a.reshape(b.shape) - b) < 1e-6)
    _, _, zeros = linear_backward_hip_f32(g, x, w, False)
    assert zeros.shape == (1, 2) and not zeros.any()


def test_argument_errors(hip):
    from helpers import raw_device_buffer
    buf = raw_device_buffer(4096)
    p = buf.ptr
    assert capi.status("vtl_hip_matmul_f32", p, p, p, -1, 2, 2, 0, 0) == capi.ERR_INVALID_ARG
    assert capi.status("vtl_hip_matmul_f32", None, p, p, 2, 2, 2, 0, 0) == capi.ERR_INVALID_ARG
    assert capi.status("vtl_hip_matmul_f64", p, p, None, 2, 2, 2, 0, 0) == capi.ERR_INVALID_ARG
    assert capi.status("vtl_hip_matmul_f32", p, p, p, 0, 5, 3, 0, 0) == capi.OK
    assert capi.status("vtl_hip_colsum_f32", None, 4, 4, p) == capi.ERR_INVALID_ARG
    assert capi.status("vtl_hip_linear_backward_f32", None, p, p, p, p, p, 2, 2, 2) == capi.ERR_INVALID_ARG
    assert capi.status("vtl_hip_linear_backward_f32", p, p, None, p, None, None, 2, 2, 2) == capi.ERR_INVALID_ARG
    # K == 0: zeros (plus the bias for the Linear form)
    capi.call("vtl_hip_memset", p, 0xFF, 4096)
    capi.call("vtl_hip_matmul_f32", None, None, p, 3, 4, 0, 0, 0)
    from helpers import d2h
    assert not d2h(p, 12, np.float32).any()
    buf.release()


def test_matmul_gate_backward(hip, monkeypatch):
    """MatMulGate.backward (autograd/gates_blas.v:43-48): dA = g . B^T, dB = A^T . g."""
    monkeypatch.setenv("VTL_USE_HIP", "1")
    monkeypatch.setenv("VTL_HIP_BACKWARD", "1")
    rng = np.random.default_rng(28)
    for dt in (np.float32, np.float64):
        a = rng.standard_normal((37, 53)).astype(dt)
        b = rng.standard_normal((53, 29)).astype(dt)
        g = rng.standard_normal((37, 29)).astype(dt)
        da, db = matmul_gate_backward_hip(g, a, b)
        want_a = oracle.matmul(g, np.ascontiguousarray(b.T))
        want_b = oracle.matmul(np.ascontiguousarray(a.T), g)
        absa = np.abs(g).astype(np.float64) @ np.abs(b.T).astype(np.float64)
        absb = np.abs(a.T).astype(np.float64) @ np.abs(g).astype(np.float64)
        assert_close_to_oracle(da, want_a, absa)
        assert_close_to_oracle(db, want_b, absb)
    with pytest.raises(ValueError, match="Invalid shapes"):
        matmul_gate_backward_hip(np.zeros((3, 3)), np.zeros((3, 4)), np.zeros((5, 3)))
