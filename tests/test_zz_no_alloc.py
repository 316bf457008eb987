"""The entry point that allocates nothing, vtl_hip_linear_f32_dynquant_noalloc,
against vtl_hip_linear_f32_dynquant through the C ABI: same bits, on calls in
a row that share the device's static scratch, the later ones smaller."""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import CPU_THREADS, dev
from vtl_amd import capi
from vtl_amd.tensor import HipTensor

pytestmark = pytest.mark.gpu


def _both(x, wq, sw, bias, relu):
    """(existing entry point, no-alloc entry point) on the same device buffers."""
    m, k = x.shape
    n = wq.shape[0]
    X, W, SW = dev(x), dev(wq), dev(sw)
    B = dev(bias) if bias is not None else None
    out = []
    for name, tail in (("vtl_hip_linear_f32_dynquant", (None, 0)), ("vtl_hip_linear_f32_dynquant_noalloc", ())):
        Y = HipTensor.from_host(np.full((m, n), np.float32(-777.0)))
        capi.call(name, X.ptr, W.ptr, SW.ptr, B.ptr if B else None, Y.ptr, m, n, k, 1 if relu else 0, *tail)
        out.append(Y.cpu())
        Y.release()
    for h in (X, W, SW) + ((B,) if B else ()):
        h.release()
    return out


def test_noalloc_matches_existing_entry_point_on_calls_in_a_row(hip):
    rng = np.random.Generator(np.random.Philox(77))
    # a K split (16 MiB of int32 partial sums + 2.8 MB of codes in the scratch), then a smaller
    # call without a split, then a K that needs the operands repacked, then a single token
    shapes = [(256, 4096, 11008, True, True), (64, 1024, 4096, False, True), (48, 300, 1000, True, False),
              (1, 2048, 4096, False, True)]
    for m, n, k, relu, with_bias in shapes:
        x = rng.standard_normal((m, k), dtype=np.float32)
        wq = rng.integers(-127, 128, (n, k), dtype=np.int8)
        sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32) if with_bias else None
        old, new = _both(x, wq, sw, bias, relu)
        assert np.array_equal(new, old), (m, n, k)
        want = oracle.linear_f32_dynquant(x, wq, sw, bias, relu=relu, threads=CPU_THREADS)
        assert np.array_equal(new, want), (m, n, k)


def test_noalloc_rejects_what_does_not_fit(hip):
    # 2048 x 8192 activations: 16 MiB of codes fit, but the 8 x 8 tiles of this product are split
    # over K and their int32 partial sums do not
    m, n, k = 2048, 2048, 16384
    X = HipTensor.empty([m, k], np.float32)
    W = HipTensor.empty([n, k], np.int8)
    SW = HipTensor.empty([n], np.float32)
    Y = HipTensor.from_host(np.full((m, n), np.float32(5.0)))
    capi.call("vtl_hip_memset", X.ptr, 0, m * k * 4)
    capi.call("vtl_hip_memset", W.ptr, 0, n * k)
    capi.call("vtl_hip_memset", SW.ptr, 0, n * 4)
    st = capi.status("vtl_hip_linear_f32_dynquant_noalloc", X.ptr, W.ptr, SW.ptr, None, Y.ptr, m, n, k, 0)
    capi.call("vtl_hip_sync")
    if st == capi.OK:          # no K split chosen for this shape: everything fitted
        assert not Y.cpu().any()
    else:
        assert st == capi.ERR_UNSUPPORTED
        assert b"static scratch" in capi.lib().vtl_hip_last_error()
        assert np.all(Y.cpu() == np.float32(5.0))
    # a staging need beyond the array on its own: 40 MiB of codes
    m2, k2 = 4096, 10240
    X2 = HipTensor.empty([m2, k2], np.float32)
    W2 = HipTensor.empty([64, k2], np.int8)
    Y2 = HipTensor.empty([m2, 64], np.float32)
    st = capi.status("vtl_hip_linear_f32_dynquant_noalloc", X2.ptr, W2.ptr, SW.ptr, None, Y2.ptr, m2, 64, k2, 0)
    assert st == capi.ERR_UNSUPPORTED and b"static scratch" in capi.lib().vtl_hip_last_error()
    capi.call("vtl_hip_sync")
    for h in (X, W, SW, Y, X2, W2, Y2):
        h.release()
