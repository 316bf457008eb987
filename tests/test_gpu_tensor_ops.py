"""Generic device-tensor operations (gemv, ReLU, sigmoid; the reference's
CudaTensor counterparts tensor_cuda_d_cuda.v:182-270) against the CPU oracle.

Bar: ReLU bit for bit.  gemv sums the same f64 products in another order: at
most one unit in the last place after the rounding to f32, 1e-13 of the sum of
|a||x| for f64.  sigmoid uses the device's f64 exp, correct to about an ulp like
the C library's: at most one ulp (f32) / four ulp (f64) apart."""
import numpy as np
import pytest

import oracle
from helpers import dev
from vtl_amd import capi
from vtl_amd.tensor import HipTensor, gemv_hip

pytestmark = pytest.mark.gpu


def ulp_diff(a, b):
    it = np.int32 if a.dtype == np.float32 else np.int64
    return np.abs(a.view(it).astype(np.int64) - b.view(it).astype(np.int64))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("rows,cols", [(1, 1), (3, 5), (64, 784), (4096, 4096), (10, 100000), (100000, 7),
                                       (2047, 2049), (5, 2048), (0, 8)])
def test_gemv(hip, dt, rows, cols):
    rng = np.random.default_rng(41)
    a = rng.standard_normal((rows, cols)).astype(dt)
    x = rng.standard_normal(cols).astype(dt)
    if rows == 0:
        assert capi.status("vtl_hip_gemv_f32", None, None, None, 0, cols) == capi.OK
        return
    A, X, Y = dev(a), dev(x), HipTensor.empty([rows], dt)
    gemv_hip(Y, A, X)
    got, want = Y.cpu(), oracle.gemv(a, x)
    if dt == np.float32:
        d = ulp_diff(got, want)
        assert d.max() <= 1 and (d > 0).mean() < 1e-2
    else:
        assert np.all(np.abs(got - want) <= 1e-13 * (np.abs(a) @ np.abs(x)))
    # integer-valued operands: exact whatever the order
    ai, xi = np.rint(a * 3).astype(dt), np.rint(x * 3).astype(dt)
    Ai, Xi = dev(ai), dev(xi)
    gemv_hip(Y, Ai, Xi)
    assert np.array_equal(Y.cpu(), (ai.astype(np.float64) @ xi.astype(np.float64)).astype(dt))
    with pytest.raises(ValueError):
        gemv_hip(Y, A, Y) if rows != cols else gemv_hip(A, A, X)
    for t in (A, X, Y, Ai, Xi):
        t.release()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_sigmoid_and_relu(hip, dt):
    rng = np.random.default_rng(42)
    x = (rng.standard_normal((513, 1027)) * 6).astype(dt)
    x.reshape(-1)[:12] = [0, -0.0, 1, -1, 100, -100, 800, -800, 1e-30, -1e-30, np.inf, -np.inf]
    X = dev(x)
    S = X.sigmoid_hip()
    got, want = S.cpu(), oracle.sigmoid(x)
    assert S.shape == X.shape and got.dtype == dt
    d = ulp_diff(got, want)
    assert d.max() <= (1 if dt == np.float32 else 4), d.max()
    assert got.reshape(-1)[0] == dt(0.5) and got.reshape(-1)[10] == 1 and got.reshape(-1)[11] == 0
    R = X.relu_hip()
    want_r = oracle.relu(x) if dt == np.float32 else oracle.relu_f64(x)
    assert np.array_equal(R.cpu(), want_r) and np.array_equal(X.cpu(), x)        # the input is untouched
    assert np.array_equal(np.signbit(R.cpu()), np.signbit(want_r))
    X.relu_()
    assert np.array_equal(X.cpu(), want_r)
    nan = dev(np.array([np.nan, -1.0], dt))
    assert np.isnan(nan.relu_hip().cpu()[0]) and np.isnan(nan.sigmoid_hip().cpu()[0])
    for t in (X, S, R, nan):
        t.release()
    assert capi.status("vtl_hip_sigmoid_f32", None, None, 4) == capi.ERR_INVALID_ARG
    assert capi.status("vtl_hip_sigmoid_f64", None, None, 0) == capi.OK
    assert capi.status("vtl_hip_relu_f64", None, -1) == capi.ERR_INVALID_ARG


def test_activation_hooks_host_round_trip(hip, monkeypatch):
    from vtl_amd import relu_forward_hip_f32, sigmoid_forward_hip_f32
    x = (np.random.default_rng(43).standard_normal((7, 33)) * 4).astype(np.float32)
    monkeypatch.delenv("VTL_USE_HIP", raising=False)
    with pytest.raises(RuntimeError, match="VTL_USE_HIP"):
        relu_forward_hip_f32(x)
    monkeypatch.setenv("VTL_USE_HIP", "1")
    assert np.array_equal(relu_forward_hip_f32(x), oracle.relu(x))
    assert ulp_diff(sigmoid_forward_hip_f32(x), oracle.sigmoid(x)).max() <= 1
    assert relu_forward_hip_f32(np.zeros((0, 4), np.float32)).shape == (0, 4)
    with pytest.raises(TypeError):
        relu_forward_hip_f32(np.zeros(4, np.int32))
