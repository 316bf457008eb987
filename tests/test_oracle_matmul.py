"""Pins of the oracle's f64-accumulating matmul, column sum and Linear backward
(la.matmul la/la.v:38-55, LinearGate.backward nn/gates/layers/linear.v:57-79)
by checks that do not retype its formula: the reference's own test literals,
numpy's f64 matmul on explicitly transposed copies, integer-valued operands
whose sums are exact in any order, math.fsum, and finite differences."""
import math

import numpy as np
import pytest

import oracle


def ulp_diff(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Distance in units of the last place between same-sign finite floats."""
    it = np.int32 if a.dtype == np.float32 else np.int64
    return np.abs(a.view(it).astype(np.int64) - b.view(it).astype(np.int64))


def test_identity_times_b_is_b():
    # la/la_test.v:30-37
    a = np.array([[1.0, 0], [0.0, 1]])
    b = np.array([[4.0, 1], [2.0, 2]])
    for dt in (np.float32, np.float64):
        assert np.array_equal(oracle.matmul(a.astype(dt), b.astype(dt)), b.astype(dt))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_matmul_against_numpy_f64(dt, ta, tb):
    rng = np.random.default_rng(11)
    M, N, K = 37, 29, 83
    A = rng.standard_normal((K, M) if ta else (M, K)).astype(dt)
    B = rng.standard_normal((N, K) if tb else (K, N)).astype(dt)
    got = oracle.matmul(A, B, ta, tb)
    opa = (A.T if ta else A).astype(np.float64)
    opb = (B.T if tb else B).astype(np.float64)
    want = (opa @ opb)
    assert got.shape == (M, N) and got.dtype == dt
    if dt == np.float32:
        # numpy's BLAS sums in another order: the f64 sums differ by ~1e-16 relative, so
        # the two roundings to f32 may disagree by one unit in the last place, rarely
        d = ulp_diff(got, want.astype(np.float32))
        assert d.max() <= 1 and (d > 0).mean() < 0.01
    else:
        bound = 1e-15 * (np.abs(opa) @ np.abs(opb)) * K
        assert np.all(np.abs(got - want) <= bound)


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_matmul_integer_valued_operands_are_exact(ta, tb):
    rng = np.random.default_rng(12)
    M, N, K = 45, 51, 260
    Ai = rng.integers(-16, 17, (K, M) if ta else (M, K))
    Bi = rng.integers(-16, 17, (N, K) if tb else (K, N))
    want = (Ai.T if ta else Ai).astype(np.int64) @ (Bi.T if tb else Bi).astype(np.int64)
    for dt in (np.float32, np.float64):
        got = oracle.matmul(Ai.astype(dt), Bi.astype(dt), ta, tb)
        assert np.array_equal(got.astype(np.int64), want)
        assert np.array_equal(oracle.matmul(Ai.astype(dt), Bi.astype(dt), ta, tb, threads=4), got)


def test_matmul_bench_literals_closed_form():
    # benchmarks/vs_numpy/matmul_bench.v:28-33: a[i,j] = ((i+j)%7)*0.01, b[i,j] = ((i*j)%5)*0.02
    n = 128
    i, j = np.indices((n, n))
    ai, bi = (i + j) % 7, (i * j) % 5
    got = oracle.matmul(ai * 0.01, bi * 0.02)
    want_int = ai.astype(np.int64) @ bi.astype(np.int64)      # exact
    assert np.all(np.abs(got - want_int * 2e-4) <= 1e-12 * np.maximum(want_int, 1))


def test_forward_literals_of_the_device_session_test():
    # autograd_cuda/device_session_test.v:34-36: x = [1,2,3], W = [[.1,.2,.3],[.4,.5,.6]]
    x = np.array([[1.0, 2.0, 3.0]])
    w = np.array([[0.1, 0.2, 0.3], [0.4, 0.5, 0.6]])
    y = oracle.matmul(x, w, False, True)
    assert np.allclose(y, [[1.4, 3.2]], rtol=0, atol=1e-15)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_colsum_against_fsum(dt):
    rng = np.random.default_rng(13)
    x = (rng.standard_normal((301, 17)) * 10.0 ** rng.integers(-3, 4, (301, 17))).astype(dt)
    got = oracle.colsum(x)
    for c in range(x.shape[1]):
        exact = math.fsum(float(v) for v in x[:, c])
        if dt == np.float32:
            assert ulp_diff(got[c:c + 1], np.array([exact], np.float32)).max() <= 1
        else:
            assert abs(got[c] - exact) <= 1e-13 * np.abs(x[:, c]).sum()


def test_linear_backward_hand_worked():
    # operands of autograd_cuda/device_session_test.v:52-60, gradients by hand:
    # dx = g.W = [1*.1+.5*.4, 1*.2+.5*.5, 1*.3+.5*.6]; dw = g^T.x; db = g
    g = np.array([[1.0, 0.5]])
    x = np.array([[1.0, 2.0, 3.0]])
    w = np.array([[0.1, 0.2, 0.3], [0.4, 0.5, 0.6]])
    dx, dw, db = oracle.linear_backward(g, x, w)
    assert dx.shape == (1, 3) and dw.shape == (2, 3) and db.shape == (2,)
    assert np.allclose(dx, [[0.3, 0.45, 0.6]], rtol=0, atol=1e-15)
    assert np.array_equal(dw, [[1.0, 2.0, 3.0], [0.5, 1.0, 1.5]])
    assert np.array_equal(db, [1.0, 0.5])
    dx32, dw32, db32 = oracle.linear_backward(g.astype(np.float32), x.astype(np.float32), w.astype(np.float32))
    assert np.allclose(dx32, dx, rtol=1e-6) and np.array_equal(dw32, dw) and np.array_equal(db32, db)


def test_linear_backward_matches_finite_differences():
    rng = np.random.default_rng(14)
    M, N, K = 5, 4, 6
    x, w, b = rng.standard_normal((M, K)), rng.standard_normal((N, K)), rng.standard_normal(N)
    g = rng.standard_normal((M, N))

    def loss(x_, w_, b_):
        return float((g * (x_ @ w_.T + b_)).sum())

    dx, dw, db = oracle.linear_backward(g, x, w)
    h = 1e-6
    for (arr, grad_arr, which) in ((x, dx, 0), (w, dw, 1), (b, db, 2)):
        num = np.zeros_like(arr)
        for idx in np.ndindex(arr.shape):
            p, m = arr.copy(), arr.copy()
            p[idx] += h
            m[idx] -= h
            args_p = [x, w, b]
            args_m = [x, w, b]
            args_p[which], args_m[which] = p, m
            num[idx] = (loss(*args_p) - loss(*args_m)) / (2 * h)
        assert np.allclose(grad_arr, num, rtol=1e-6, atol=1e-7)


def test_empty_contraction_gives_zeros():
    for dt in (np.float32, np.float64):
        c = oracle.matmul(np.zeros((3, 0), dt), np.zeros((0, 4), dt))
        assert c.shape == (3, 4) and not c.any()
        assert not oracle.colsum(np.zeros((0, 5), dt)).any()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_gemv_against_numpy_and_exact_integers(dt):
    rng = np.random.default_rng(15)
    a, x = rng.standard_normal((37, 301)).astype(dt), rng.standard_normal(301).astype(dt)
    got = oracle.gemv(a, x)
    want = a.astype(np.float64) @ x.astype(np.float64)
    if dt == np.float32:
        assert ulp_diff(got, want.astype(np.float32)).max() <= 1
    else:
        assert np.all(np.abs(got - want) <= 1e-13 * (np.abs(a) @ np.abs(x)))
    ai, xi = rng.integers(-9, 10, (50, 777)), rng.integers(-9, 10, 777)
    assert np.array_equal(oracle.gemv(ai.astype(dt), xi.astype(dt)).astype(np.int64), ai @ xi)


def test_sigmoid_closed_forms_and_numpy():
    for dt in (np.float32, np.float64):
        assert oracle.sigmoid(np.zeros(3, dt))[0] == dt(0.5)
        x = np.linspace(-30, 30, 2001).astype(dt)
        s = oracle.sigmoid(x)
        assert s.dtype == dt and np.all((s >= 0) & (s <= 1)) and np.all(np.diff(s) >= 0)
        # sigmoid(x) + sigmoid(-x) = 1 up to the roundings of the two quotients
        assert np.all(np.abs(s + oracle.sigmoid(-x) - 1) <= 4 * np.finfo(dt).eps)
        # the same three operations with numpy's exp (both exps are correct to <= 1 ulp of f64)
        e = np.exp(-x.astype(np.float64)).astype(dt)
        want = dt(1) / (dt(1) + e)
        # one ulp of difference between the two exps can grow to two in the f64 quotient
        assert ulp_diff(s, want.astype(dt)).max() <= (1 if dt == np.float32 else 2)
        big = oracle.sigmoid(np.array([1000.0, -1000.0, 90.0, -90.0], dt))
        assert big[0] == 1 and big[1] == 0 and big[2] == 1 and 0 <= big[3] < 1e-38
    # literals: sigmoid(1) = 0.7310585786300049, sigmoid(-2) = 0.11920292202211755
    s = oracle.sigmoid(np.array([1.0, -2.0]))
    assert abs(s[0] - 0.7310585786300049) < 2e-16 and abs(s[1] - 0.11920292202211755) < 2e-17


def test_relu_f64_closed_form():
    x = np.array([-1.5, -0.0, 0.0, 2.5, -np.inf, np.inf, np.nan])
    y = oracle.relu_f64(x)
    assert np.array_equal(y[:6], [0.0, -0.0, 0.0, 2.5, 0.0, np.inf]) and np.isnan(y[6])
    assert np.signbit(y[1]) and not np.signbit(y[0])
