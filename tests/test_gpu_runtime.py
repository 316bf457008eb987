"""Device, memory, transfer, stream and timing entry points on a real device
(the calls HipStorage makes where CudaStorage calls cudaMalloc / cudaMemcpy /
cudaFree, storage/cuda_d_cuda.v:32-102)."""
import ctypes as C
import os

import numpy as np
import pytest

from helpers import d2h, h2d, raw_device_buffer
from vtl_amd import capi
from vtl_amd.storage import HipParams, HipStorage
from vtl_amd.tensor import HipTensor

pytestmark = pytest.mark.gpu


def test_device_queries(hip):
    assert capi.device_count() >= 1
    name, cus, mhz = capi.device_info()
    assert "gfx950" in name and cus == 256 and mhz > 1000
    assert capi.status("vtl_hip_set_device", capi.device_count() + 3) == capi.ERR_NO_DEVICE
    assert capi.status("vtl_hip_set_device", -1) == capi.ERR_NO_DEVICE
    with pytest.raises(capi.VtlHipError) as ei:
        HipStorage.empty(4, np.float32, HipParams(device_id=99))
    assert ei.value.status == capi.ERR_NO_DEVICE


def test_storage_round_trip_and_release(hip):
    rng = np.random.default_rng(0)
    for dtype in (np.float32, np.int8, np.int32):
        a = (rng.standard_normal(1000) * 50).astype(dtype)
        st = HipStorage.from_cpu(a)
        assert st.count == 1000 and st.size == a.nbytes and st.ptr
        assert st.hip() is st
        assert np.array_equal(st.cpu(), a) and np.array_equal(st.to_array(), a)
        st.release()
        assert st.ptr == 0
        st.release()                                  # releasing twice is harmless
    empty = HipStorage.from_cpu(np.zeros(0, np.float32))
    assert empty.count == 0 and empty.cpu().size == 0
    t = HipTensor.from_host(np.arange(12, dtype=np.float32).reshape(3, 4))
    assert t.shape == [3, 4] and t.strides == [4, 1] and t.hip() is t
    assert np.array_equal(t.cpu(), np.arange(12, dtype=np.float32).reshape(3, 4))
    t.release()


def test_memset_and_device_to_device_copy(hip):
    n = 1 << 20
    a, b = raw_device_buffer(n + 64), raw_device_buffer(n + 64)
    capi.call("vtl_hip_memset", a.ptr, 0x5A, n)
    capi.call("vtl_hip_memcpy_d2d", b.ptr, a.ptr, n)          # 16-byte aligned: the library's copy kernel
    assert np.all(d2h(b.ptr, n, np.uint8) == 0x5A)
    src = np.arange(1001, dtype=np.uint8)
    h2d(a.ptr + 3, src)
    capi.call("vtl_hip_memcpy_d2d", b.ptr + 5, a.ptr + 3, src.size)   # unaligned, odd size: runtime copy
    capi.call("vtl_hip_sync")
    assert np.array_equal(d2h(b.ptr + 5, src.size, np.uint8), src)
    a.release()
    b.release()


@pytest.mark.parametrize("offset,size", [(0, 4096), (3, 1), (5, 10), (13, 1001), (1, 15), (16, 16), (7, 65537)])
def test_memset_any_alignment_and_size_leaves_neighbours_alone(hip, offset, size):
    buf = raw_device_buffer(70000)
    h2d(buf.ptr, np.full(70000, 0x11, np.uint8))
    capi.call("vtl_hip_memset", buf.ptr + offset, 0xC3, size)
    capi.call("vtl_hip_sync")
    got = d2h(buf.ptr, 70000, np.uint8)
    want = np.full(70000, 0x11, np.uint8)
    want[offset:offset + size] = 0xC3
    assert np.array_equal(got, want)
    buf.release()


def test_events_time_a_kernel(hip):
    e0, e1 = C.c_void_p(), C.c_void_p()
    capi.call("vtl_hip_event_create", C.byref(e0))
    capi.call("vtl_hip_event_create", C.byref(e1))
    x = HipTensor.from_host(np.ones((2048, 4096), np.float32))
    capi.call("vtl_hip_event_record", e0)
    q, s = x.quantize_i8(0)
    capi.call("vtl_hip_event_record", e1)
    ms = C.c_float(-1.0)
    capi.call("vtl_hip_event_elapsed_ms", e0, e1, C.byref(ms))
    assert 0.0 < ms.value < 100.0
    assert np.all(q.cpu() == 127) and np.all(s.cpu() == np.float32(1.0) / np.float32(127.0))
    capi.call("vtl_hip_event_destroy", e0)
    capi.call("vtl_hip_event_destroy", e1)
    for h in (x, q, s):
        h.release()


def test_unsupported_shapes_return_status(hip):
    buf = raw_device_buffer(4096)
    assert capi.status("vtl_hip_gemm_i8_i32", buf.ptr, buf.ptr, buf.ptr, 4, 4, 0) == capi.ERR_UNSUPPORTED
    assert capi.status("vtl_hip_linear_i8_f32", buf.ptr, buf.ptr, 1, buf.ptr, buf.ptr, 1, None, buf.ptr,
                       4, 4, 0, 0) == capi.ERR_UNSUPPORTED
    # workspace too small / misaligned for the dynamic-quantization entry point
    assert capi.status("vtl_hip_linear_f32_dynquant", buf.ptr, buf.ptr, buf.ptr, None, buf.ptr, 8, 8, 64, 0,
                       buf.ptr, 16) == capi.ERR_INVALID_ARG
    assert capi.status("vtl_hip_linear_f32_dynquant", buf.ptr, buf.ptr, buf.ptr, None, buf.ptr, 8, 8, 64, 0,
                       buf.ptr + 4, 4000) == capi.ERR_INVALID_ARG
    buf.release()


def test_compute_on_a_caller_stream(hip):
    """vtl_hip_set_stream: the entry points enqueue on a stream the caller made (default
    priority); results equal those on the null stream."""
    import oracle
    hiprt = C.CDLL("libamdhip64.so")
    stream = C.c_void_p()
    assert hiprt.hipStreamCreate(C.byref(stream)) == 0
    try:
        capi.call("vtl_hip_set_stream", stream)
        got = C.c_void_p()
        capi.call("vtl_hip_get_stream", C.byref(got))
        assert got.value == stream.value
        rng = np.random.default_rng(61)
        x = rng.standard_normal((64, 1024)).astype(np.float32)
        w = rng.integers(-127, 128, (256, 1024), dtype=np.int8)
        sw = rng.uniform(0.5, 1.5, 256).astype(np.float32)
        X, W, SW = HipTensor.from_host(x), HipTensor.from_host(w), HipTensor.from_host(sw)
        Y = HipTensor.empty([64, 256], np.float32)
        for _ in range(3):
            capi.call("vtl_hip_linear_f32_dynquant", X.ptr, W.ptr, SW.ptr, None, Y.ptr, 64, 256, 1024, 1, None, 0)
        capi.call("vtl_hip_sync")                      # waits on the caller's stream
        assert np.array_equal(Y.cpu(), oracle.linear_f32_dynquant(x, w, sw, None, relu=True))
        q, s = X.quantize_i8(0)
        assert np.array_equal(q.dequantize(s, 0).cpu(), oracle.dequantize(*oracle.quantize(x, True), True))
        for t in (X, W, SW, Y, q, s):
            t.release()
    finally:
        capi.call("vtl_hip_set_stream", None)
        assert hiprt.hipStreamDestroy(stream) == 0


def test_entry_points_capture_into_a_hip_graph(hip):
    """Quantize + int8 linear recorded once into a HIP graph on a caller stream and
    replayed with new activations: every replay equals the oracle.  (The recorded
    entry points allocate nothing and record no memset; kernel attributes are set
    by a warm-up call before the capture.)"""
    import oracle
    hiprt = C.CDLL("libamdhip64.so")
    stream, graph, gexec = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert hiprt.hipStreamCreate(C.byref(stream)) == 0
    rng = np.random.default_rng(62)
    m, n, k = 48, 512, 1024
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = rng.uniform(0.5, 1.5, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    X, W, SW, B = (HipTensor.from_host(a) for a in (x, w, sw, bias))
    XQ, SX, Y = HipTensor.empty([m, k], np.int8), HipTensor.empty([m], np.float32), HipTensor.empty([m, n], np.float32)

    def enqueue():
        capi.call("vtl_hip_quantize_f32_i8", X.ptr, m, k, 1, XQ.ptr, SX.ptr)
        capi.call("vtl_hip_linear_i8_f32", XQ.ptr, SX.ptr, 1, W.ptr, SW.ptr, 1, B.ptr, Y.ptr, m, n, k, 1)

    try:
        capi.call("vtl_hip_set_stream", stream)
        enqueue()                                   # warm-up outside the capture
        capi.call("vtl_hip_sync")
        assert hiprt.hipStreamBeginCapture(stream, 0) == 0
        enqueue()
        assert hiprt.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert hiprt.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
        for rep in range(4):
            xr = (rng.standard_normal((m, k)) * (rep + 1)).astype(np.float32)
            capi.call("vtl_hip_memcpy_h2d", X.ptr, xr.ctypes.data, xr.nbytes)     # eager work between replays
            assert hiprt.hipGraphLaunch(gexec, stream) == 0
            capi.call("vtl_hip_sync")
            wq_ref = oracle.linear_f32_dynquant(xr, w, sw, bias, relu=True)
            assert np.array_equal(Y.cpu(), wq_ref), f"replay {rep}"
    finally:
        capi.call("vtl_hip_set_stream", None)
        if gexec:
            hiprt.hipGraphExecDestroy(gexec)
        if graph:
            hiprt.hipGraphDestroy(graph)
        hiprt.hipStreamDestroy(stream)
        for t in (X, W, SW, B, XQ, SX, Y):
            t.release()


def test_library_scratch_recorded_into_a_graph_survives_growth_and_never_grows_under_capture(hip):
    """vtl_hip_linear_f32_dynquant without a caller workspace stages the activation codes in the
    library's own buffer, whose address a stream capture bakes into the graph.  A later eager
    call that needs a larger buffer must not free the recorded one (replays still write to it),
    and a call that would have to grow the buffer during a capture is refused with a status."""
    import oracle
    hiprt = C.CDLL("libamdhip64.so")
    stream, graph, gexec = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert hiprt.hipStreamCreate(C.byref(stream)) == 0
    rng = np.random.default_rng(63)
    m, n, k = 40, 256, 1024
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = rng.uniform(0.5, 1.5, n).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    X, W, SW = (HipTensor.from_host(a) for a in (x, w, sw))
    Y = HipTensor.empty([m, n], np.float32)
    # the eager call that makes the staging buffer grow: 96 MiB of codes, more than any other test stages
    mb, kb = 24576, 4096
    XB = HipTensor.empty([mb, kb], np.float32)
    WB = HipTensor.from_host(rng.integers(-127, 128, (64, kb), dtype=np.int8))
    YB = HipTensor.empty([mb, 64], np.float32)
    capi.call("vtl_hip_memset", XB.ptr, 0, mb * kb * 4)
    # Asked for under capture only: 64 GiB of codes, more than the staging buffer can have grown to
    # whatever ran before in this process (other tests stage f32 rows of outputs beyond 2^32
    # elements there).  The call must be refused before anything is recorded, so it is handed
    # the buffers of the eager call; were it accepted, its kernels would only be recorded into
    # a graph that is destroyed without a launch.
    mc = 1 << 24
    XC, YC = XB, YB

    def small():
        capi.call("vtl_hip_linear_f32_dynquant", X.ptr, W.ptr, SW.ptr, None, Y.ptr, m, n, k, 0, None, 0)

    try:
        capi.call("vtl_hip_set_stream", stream)
        small()                                     # warm-up: the buffer exists, kernel attributes are set
        capi.call("vtl_hip_sync")
        assert hiprt.hipStreamBeginCapture(stream, 0) == 0
        small()
        assert hiprt.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert hiprt.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
        capi.call("vtl_hip_linear_f32_dynquant", XB.ptr, WB.ptr, SW.ptr, None, YB.ptr, mb, 64, kb, 0, None, 0)
        capi.call("vtl_hip_sync")
        for rep in range(3):
            xr = (rng.standard_normal((m, k)) * (rep + 2)).astype(np.float32)
            capi.call("vtl_hip_memcpy_h2d", X.ptr, xr.ctypes.data, xr.nbytes)
            assert hiprt.hipGraphLaunch(gexec, stream) == 0
            capi.call("vtl_hip_sync")
            assert np.array_equal(Y.cpu(), oracle.linear_f32_dynquant(xr, w, sw, None)), f"replay {rep}"
        # under capture the buffer may be used, never grown: 64 GiB of codes do not fit what exists
        assert hiprt.hipStreamBeginCapture(stream, 0) == 0
        st = capi.status("vtl_hip_linear_f32_dynquant", XC.ptr, WB.ptr, SW.ptr, None, YC.ptr, mc, 64, kb, 0, None, 0)
        graph2 = C.c_void_p()
        assert hiprt.hipStreamEndCapture(stream, C.byref(graph2)) == 0
        if graph2:
            hiprt.hipGraphDestroy(graph2)
        assert st == capi.ERR_UNSUPPORTED and b"stream capture" in capi.lib().vtl_hip_last_error()
    finally:
        capi.call("vtl_hip_set_stream", None)
        if gexec:
            hiprt.hipGraphExecDestroy(gexec)
        if graph:
            hiprt.hipGraphDestroy(graph)
        hiprt.hipStreamDestroy(stream)
        for t in (X, W, SW, Y, XB, WB, YB):
            t.release()


def test_mfma_probe_runs_and_leaves_its_sink_alone(hip):
    """The measurement aid behind bench.py's `mfma_only` figures: launches, finishes, and
    never writes its sink (the sums it keeps alive cannot reach the sentinel)."""
    ops = HipTensor.from_host(np.random.default_rng(0).integers(-127, 128, 256 * 1024, dtype=np.int8))
    sink = HipTensor.from_host(np.array([-7, 0, 0, 0], np.int32))
    from vtl_amd import build as vb
    assert os.path.exists(vb.BENCH_PROBE_PATH), "libvtlbenchprobe.so is not built"
    for sym in ("vtl_bench_probe_mfma_i8", "vtl_bench_probe_mfma_i8_rotating"):
        probe = getattr(C.CDLL(vb.BENCH_PROBE_PATH), sym)
        probe.restype, probe.argtypes = C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
        assert probe(ops.ptr, 3, sink.ptr, None) == 0
        assert probe(ops.ptr, 0, sink.ptr, None) == 0
        capi.call("vtl_hip_sync")
        assert sink.cpu()[0] == -7
        assert probe(ops.ptr + 1, 3, sink.ptr, None) == 1
    ops.release()
    sink.release()


def test_guard_bands_notice_a_write_past_either_end(hip, guard_bands):
    """The out-of-bounds check of the ragged-shape parity tests, checked itself: a byte written
    just before or just past a buffer (inside the guarded allocation, so nothing faults) is
    reported when the buffer is released; an untouched buffer is not."""
    clean = HipTensor.from_host(np.arange(100, dtype=np.float32))
    assert np.array_equal(clean.cpu(), np.arange(100, dtype=np.float32))
    clean.release()
    assert guard_bands == []
    past = HipTensor.empty([3, 7], np.int8)
    capi.call("vtl_hip_memset", past.ptr + 21, 0, 1)
    past.release()
    assert len(guard_bands) == 1 and "after the buffer" in guard_bands[0] and "offset 0 " in guard_bands[0]
    before = HipTensor.empty([5], np.int32)
    capi.call("vtl_hip_memset", before.ptr - 2, 7, 1)
    before.release()
    assert len(guard_bands) == 2 and "before the buffer" in guard_bands[1] and "offset -2 " in guard_bands[1]
    guard_bands.clear()
