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


_FRESH_PROCESS = r"""
import ctypes as C, json, os, sys
import numpy as np
sys.path.insert(0, sys.argv[1])
from vtl_amd import capi
from vtl_amd.tensor import HipTensor
capi.call("vtl_hip_set_device", 0)
hiprt = C.CDLL("libamdhip64.so")
def free_bytes():
    free, total = C.c_size_t(), C.c_size_t()
    assert hiprt.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value
d = np.load(sys.argv[2])
x, wq, sw = d["x"], d["wq"], d["sw"]
m, k = x.shape
n = wq.shape[0]
X, W, SW = HipTensor.from_host(x), HipTensor.from_host(wq), HipTensor.from_host(sw)
Y = HipTensor.from_host(np.full((m, n), np.float32(-3.0)))
Y2 = HipTensor.from_host(np.full((64, n), np.float32(-3.0)))
capi.call("vtl_hip_sync")
readings = [free_bytes()]
capi.call("vtl_hip_linear_f32_dynquant_noalloc", X.ptr, W.ptr, SW.ptr, None, Y.ptr, m, n, k, 0)
capi.call("vtl_hip_sync")
readings.append(free_bytes())
capi.call("vtl_hip_linear_f32_dynquant_noalloc", X.ptr, W.ptr, SW.ptr, None, Y2.ptr, 64, n, k, 0)
capi.call("vtl_hip_sync")
readings.append(free_bytes())
np.savez(sys.argv[3], y=Y.cpu(), y2=Y2.cpu())
# the same call through the entry point that may allocate: the library's own buffer appears now
capi.call("vtl_hip_linear_f32_dynquant", X.ptr, W.ptr, SW.ptr, None, Y.ptr, m, n, k, 0, None, 0)
capi.call("vtl_hip_sync")
readings.append(free_bytes())
print(json.dumps(readings))
"""


def test_noalloc_leaves_device_memory_alone_in_a_fresh_process(hip, tmp_path, monkeypatch):
    """The property the entry point is named for, checked where it can be seen: in a process
    whose library has staged nothing yet, so that its own growing buffers do not exist and a
    call that bypassed the static array would have to allocate them (32 MiB at least).
    Forced onto 128x128 tiles with K cut in two, 768 x 4096 x 2048 needs 24 MiB of int32
    partial sums and 1.5 MiB of codes, which fit the 32 MiB array.  The library's buffers are
    32 MiB or more each and this call would need two of them, so across the process's first
    call the device's free memory may drop by what the HIP runtime sets up at a first launch
    (a few MiB, measured 4) but by nothing like 32 MiB; across a second, smaller call it
    must not move at all; and the same call through vtl_hip_linear_f32_dynquant must take
    64 MiB, which shows that the readings would have caught an allocation."""
    import json
    import os
    import subprocess
    import sys
    rng = np.random.Generator(np.random.Philox(78))
    m, n, k = 768, 4096, 2048
    x = rng.standard_normal((m, k), dtype=np.float32)
    wq = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
    np.savez(tmp_path / "in.npz", x=x, wq=wq, sw=sw)
    env = dict(os.environ, VTL_HIP_GEMM_CONFIG="5,2")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-c", _FRESH_PROCESS, root, str(tmp_path / "in.npz"),
                          str(tmp_path / "out.npz")], env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                         text=True, timeout=110)
    assert res.returncode == 0, res.stderr[-2000:]
    before, after_first, after_second, after_allocating = json.loads(res.stdout.strip().splitlines()[-1])
    assert 0 <= before - after_first < (16 << 20)
    assert after_second == after_first
    assert after_allocating <= after_second - (64 << 20)
    out = np.load(tmp_path / "out.npz")
    want = oracle.linear_f32_dynquant(x, wq, sw, None, threads=CPU_THREADS)
    assert np.array_equal(out["y"], want) and np.array_equal(out["y2"], want[:64])


def test_noalloc_rejects_what_does_not_fit(hip, knobs):
    # 2048 x 16384 activations: 32 MiB of codes alone fill the array, and with the product
    # forced onto 256x256 tiles with K cut in four the int32 partial sums (64 MiB) cannot fit
    knobs.setenv("VTL_HIP_GEMM_CONFIG", "7,4")
    m, n, k = 1024, 2048, 16384
    X = HipTensor.empty([m, k], np.float32)
    W = HipTensor.empty([n, k], np.int8)
    SW = HipTensor.empty([n], np.float32)
    Y = HipTensor.from_host(np.full((m, n), np.float32(5.0)))
    capi.call("vtl_hip_memset", X.ptr, 0, m * k * 4)
    capi.call("vtl_hip_memset", W.ptr, 0, n * k)
    capi.call("vtl_hip_memset", SW.ptr, 0, n * 4)
    st = capi.status("vtl_hip_linear_f32_dynquant_noalloc", X.ptr, W.ptr, SW.ptr, None, Y.ptr, m, n, k, 0)
    capi.call("vtl_hip_sync")
    # 16 MiB of codes fit; 4 planes of 1024 x 2048 int32 (32 MiB) on top of them do not
    assert st == capi.ERR_UNSUPPORTED
    assert b"static scratch" in capi.lib().vtl_hip_last_error()
    assert np.all(Y.cpu() == np.float32(5.0))
    knobs.delenv("VTL_HIP_GEMM_CONFIG")
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
