"""Tensors with more than 2^31 elements: every kernel indexes with 64 bits.
The inputs are a random block repeated many times plus a few planted values
at the far end, so the oracle only has to restate one block and the planted
rows; the whole device result is compared."""
import numpy as np
import pytest

import oracle
from helpers import CPU_THREADS, d2h, dev, raw_device_buffer
from vtl_amd import capi
from vtl_amd.tensor import HipTensor, linear_i8_hip

pytestmark = pytest.mark.gpu

BLOCK_ROWS, REPS, EXTRA, COLS = 4096, 256, 3, 2052      # (4096 * 256 + 3) * 2052 = 2 151 683 100 > 2^31


def _big_input():
    rng = np.random.default_rng(31)
    block = rng.standard_normal((BLOCK_ROWS, COLS)).astype(np.float32)
    rows = BLOCK_ROWS * REPS + EXTRA
    x = np.empty((rows, COLS), np.float32)
    x[: BLOCK_ROWS * REPS].reshape(REPS, BLOCK_ROWS, COLS)[:] = block
    x[BLOCK_ROWS * REPS:] = block[:EXTRA]
    x[-1, -1] = np.float32(1000.0)          # the very last element carries the tensor's absmax
    x[-2, 0] = np.float32(-77.0)
    return block, x


def test_quantize_dequantize_beyond_2_31_elements(hip):
    block, x = _big_input()
    rows = x.shape[0]
    assert x.size > 2 ** 31
    print("upload", x.nbytes >> 20, "MiB", flush=True)
    X = dev(x)
    tail = x[BLOCK_ROWS * REPS:]

    # one scale per row: rows are independent, so the block's codes repeat
    print("per-row quantize", flush=True)
    Q, S = X.quantize_i8(0)
    q, s = Q.cpu(), S.cpu().reshape(-1)
    qb, sb = oracle.quantize(block, True, threads=CPU_THREADS)
    qt, st = oracle.quantize(tail, True)
    assert np.array_equal(s[: BLOCK_ROWS * REPS].reshape(REPS, BLOCK_ROWS), np.broadcast_to(sb, (REPS, BLOCK_ROWS)))
    assert np.array_equal(q[: BLOCK_ROWS * REPS].reshape(REPS, BLOCK_ROWS, COLS),
                          np.broadcast_to(qb, (REPS, BLOCK_ROWS, COLS)))
    assert np.array_equal(q[BLOCK_ROWS * REPS:], qt) and np.array_equal(s[BLOCK_ROWS * REPS:], st)
    assert q[-1, -1] == 127 and s[-1] == np.float32(1000.0) / np.float32(127.0)

    print("per-row dequantize", flush=True)
    D = Q.dequantize(S, 0)
    d = D.cpu()
    db = oracle.dequantize(qb, sb, True)
    assert np.array_equal(d[: BLOCK_ROWS * REPS].reshape(REPS, BLOCK_ROWS, COLS),
                          np.broadcast_to(db, (REPS, BLOCK_ROWS, COLS)))
    assert np.array_equal(d[BLOCK_ROWS * REPS:], oracle.dequantize(qt, st, True))
    for h in (Q, S, D):
        h.release()
    del q, d

    # one scale for the tensor: the planted last element sets it
    print("per-tensor quantize", flush=True)
    A = X.absmax(-1)
    assert A.cpu()[0] == np.float32(1000.0)
    Q, S = X.quantize_i8(-1)
    scale = S.cpu().reshape(-1)
    assert scale[0] == np.float32(1000.0) / np.float32(127.0)
    q = Q.cpu()
    qb = oracle.quantize_with_scale(block, scale, False)
    assert np.array_equal(q[: BLOCK_ROWS * REPS].reshape(REPS, BLOCK_ROWS, COLS),
                          np.broadcast_to(qb, (REPS, BLOCK_ROWS, COLS)))
    assert np.array_equal(q[BLOCK_ROWS * REPS:], oracle.quantize_with_scale(tail, scale, False))
    assert q[-1, -1] == 127 and q[-2, 0] == -10      # -77 / (1000/127) = -9.779 -> -10
    for h in (X, A, Q, S):
        h.release()


def test_linear_output_beyond_2_31_elements(hip):
    """[46400, 128] x [46400, 128]^T: 2.15e9 outputs; sampled row bands against the oracle."""
    m = n = 46400
    k = 128
    rng = np.random.default_rng(32)
    a = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sa = rng.uniform(0.5, 1.5, m).astype(np.float32)
    sw = rng.uniform(0.5, 1.5, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    assert m * n > 2 ** 31
    A, W, SA, SW, B = dev(a), dev(w), dev(sa), dev(sw), dev(bias)
    print("linear", m, n, k, flush=True)
    Y = linear_i8_hip(A, SA, W, SW, B, relu=True)
    rows = np.r_[0:8, 23195:23205, m - 8:m]
    for r0 in (0, 23195, m - 8):
        band = slice(r0, r0 + 8)
        got = np.empty((8, n), np.float32)
        capi.call("vtl_hip_memcpy_d2h", got.ctypes.data, Y.ptr + r0 * n * 4, got.nbytes)
        want = oracle.linear_i8_f32(a[band], sa[band], w, sw, bias, relu=True, threads=CPU_THREADS)
        assert np.array_equal(got, want), f"rows {r0}..{r0 + 8}"
    C = HipTensor.empty([m, n], np.int32)
    capi.call("vtl_hip_gemm_i8_i32", A.ptr, W.ptr, C.ptr, m, n, k)
    got = np.empty((8, n), np.int32)
    capi.call("vtl_hip_memcpy_d2h", got.ctypes.data, C.ptr + (m - 8) * n * 4, got.nbytes)
    assert np.array_equal(got, oracle.gemm_i8_i32(a[m - 8:], w, threads=CPU_THREADS))
    del rows
    for h in (A, W, SA, SW, B, Y, C):
        h.release()


@pytest.mark.parametrize("keep_f32", [False, True])
def test_requantizing_linear_beyond_2_31_elements(hip, keep_f32):
    """[140000, 64] x [16384, 64]^T handed on as codes: 2.29e9 outputs.  Without the f32 rows
    the int32 sums go through 9 GB of library scratch and the row kernel; with them the
    library takes the two-pass route through the caller's Y.  Sampled row bands against
    the oracle."""
    from vtl_amd.tensor import linear_i8_requant_hip
    m, n, k = 140000, 16384, 64
    rng = np.random.default_rng(33)
    a = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sa = rng.uniform(0.5, 1.5, m).astype(np.float32)
    sw = rng.uniform(0.5, 1.5, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    assert m * n > 2 ** 31
    A, W, SA, SW, B = dev(a), dev(w), dev(sa), dev(sw), dev(bias)
    print("requant", m, n, k, keep_f32, flush=True)
    out = linear_i8_requant_hip(A, SA, W, SW, B, relu=True, keep_f32=keep_f32)
    yq, sy = out[0], out[1]
    scales = sy.cpu()
    for r0 in (0, 70001, m - 8):
        band = slice(r0, r0 + 8)
        got = np.empty((8, n), np.int8)
        capi.call("vtl_hip_memcpy_d2h", got.ctypes.data, yq.ptr + r0 * n, got.nbytes)
        q_ref, s_ref, y_ref = oracle.linear_i8_requant(a[band], sa[band], w, sw, bias, relu=True, threads=CPU_THREADS)
        assert np.array_equal(got, q_ref) and np.array_equal(scales[band], s_ref), f"rows {r0}..{r0 + 8}"
        if keep_f32:
            gy = np.empty((8, n), np.float32)
            capi.call("vtl_hip_memcpy_d2h", gy.ctypes.data, out[2].ptr + r0 * n * 4, gy.nbytes)
            assert np.array_equal(gy, y_ref)
    for h in (A, W, SA, SW, B) + tuple(out):
        h.release()


def test_wide_output_beyond_2_32_elements(hip, knobs):
    """Maximum sizes: 260 x 16.9 M outputs (4.4e9 elements, 17.6 GB of f32).  Element offsets past
    2^32 must be formed in 64 bits: whole rows from either side of every tile-row boundary are
    compared with the oracle, and the one tile shape that cannot address such a row length
    (256 rows x N >= 2^32) is refused rather than run."""
    m, n, k = 260, (1 << 24) + 123000, 32
    rng = np.random.default_rng(2024)
    a = rng.integers(-127, 128, (m, k), dtype=np.int8)
    bt = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sa = rng.uniform(0.01, 0.02, m).astype(np.float32)
    sb = rng.uniform(0.01, 0.02, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    A, B, dsa, dsb, dbias = dev(a), dev(bt), dev(sa), dev(sb), dev(bias)
    rows = [0, 31, 32, 127, 128, 255, 256, 259]
    ref = oracle.gemm_i8_i32(a[rows], bt, threads=CPU_THREADS)
    want = oracle.epilogue(ref, sa[rows], sb, bias, relu=True)

    out = raw_device_buffer(m * n * 4)
    capi.call("vtl_hip_gemm_i8_i32", A.ptr, B.ptr, out.ptr, m, n, k)
    for i, r in enumerate(rows):
        assert np.array_equal(d2h(out.ptr + r * n * 4, (n,), np.int32), ref[i]), r
    capi.call("vtl_hip_linear_i8_f32", A.ptr, dsa.ptr, 1, B.ptr, dsb.ptr, 1, dbias.ptr, out.ptr, m, n, k, 1)
    for i, r in enumerate(rows):
        assert np.array_equal(d2h(out.ptr + r * n * 4, (n,), np.float32), want[i]), r

    knobs.setenv("VTL_HIP_GEMM_CONFIG", "7,1")     # 256 x 256 tiles: 255 * N + 255 >= 2^32
    assert capi.status("vtl_hip_gemm_i8_i32", A.ptr, B.ptr, out.ptr, m, n, k) == capi.ERR_UNSUPPORTED
    knobs.setenv("VTL_HIP_GEMM_CONFIG", "5,1")     # 128 x 128 tiles still can
    capi.call("vtl_hip_gemm_i8_i32", A.ptr, B.ptr, out.ptr, m, n, k)
    for i, r in enumerate(rows):
        assert np.array_equal(d2h(out.ptr + r * n * 4, (n,), np.int32), ref[i]), r
    knobs.delenv("VTL_HIP_GEMM_CONFIG")
    for h in (A, B, dsa, dsb, dbias):
        h.release()
    out.release()
