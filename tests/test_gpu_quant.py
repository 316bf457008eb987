"""GPU parity of absmax / quantize / dequantize / ReLU through the C ABI.

Bar: scales, int8 codes and dequantized values bit-exact against the CPU
oracle on the same inputs; known-answer vectors; size-independent properties
at the full benchmark size.
"""
import numpy as np
import pytest

import oracle
from helpers import KAT, d2h, dev, f32_list, h2d, quantize_with_scale_mt, raw_device_buffer, CPU_THREADS
from vtl_amd import capi, workloads

pytestmark = pytest.mark.gpu


def _codes_with_scale(hip, x, scale, per_row=False):
    t, s = dev(x), dev(np.asarray(scale, np.float32).reshape(-1))
    q = t.quantize_i8_with_scale(s, 0 if per_row else -1)
    out = q.cpu()
    for h in (t, s, q):
        h.release()
    return out


@pytest.mark.parametrize("name", ["round_half_even", "scaled_ties"])
def test_round_half_even_known_answers(hip, name):
    k = KAT[name]
    x = f32_list(k["x"])[None, :]
    got = _codes_with_scale(hip, x, [k["scale"]])
    assert got[0].tolist() == k["code"]
    # same vectors through the scalar (unaligned) kernel: odd length
    got = _codes_with_scale(hip, x[:, :-1], [k["scale"]])
    assert got[0].tolist() == k["code"][:-1]


def test_special_values(hip):
    s = KAT["special_values"]
    c = s["nan_with_scale_1"]
    assert _codes_with_scale(hip, f32_list(c["x"])[None, :], [1.0])[0].tolist() == c["code"]
    for key in ("all_zero_row", "inf_row"):
        case = s[key]
        x = f32_list(case["x"])[None, :]
        for axis in (0, -1):
            t = dev(x)
            q, sc = t.quantize_i8(axis)
            assert sc.cpu()[0] == np.float32(float(case["scale"]))
            assert q.cpu()[0].tolist() == case["code"]
            if "dequant" in case:
                assert q.dequantize(sc, axis).cpu()[0].tolist() == case["dequant"]
    n = s["nan_ignored_by_absmax"]
    t = dev(f32_list(n["x"])[None, :])
    assert t.absmax(0).cpu()[0] == n["absmax"] and t.absmax(-1).cpu()[0] == n["absmax"]
    # a row of NaNs only: absmax 0, codes 0
    t = dev(np.full((2, 8), np.nan, np.float32))
    q, sc = t.quantize_i8(0)
    assert not sc.cpu().any() and not q.cpu().any()


def test_row_quantize_known_answers(hip):
    for case in KAT["row_quantize"]["cases"]:
        x = np.array([case["x"]], np.float32)
        for axis in (0, -1):
            q, s = dev(x).quantize_i8(axis)
            assert s.cpu()[0] == np.float32(case["scale"])
            assert q.cpu()[0].tolist() == case["code"]


SHAPES = [(1, 1), (1, 3), (7, 64), (5, 256), (3, 1000), (16, 784), (4, 4096), (2, 16384), (3, 16388),
          (2, 65536), (1, 70000), (3, 777), (2, 262148), (129, 12), (1000, 4), (64, 129),
          # short rows: workgroups span several rows, rows straddle workgroups
          (5000, 1000), (70000, 8), (1025, 4092), (3000, 2052), (2, 4092),
          # one row length per workgroup size of the fused kernel
          (9, 512), (10, 2048), (6, 8192), (3, 5000), (5, 11008),
          # many short rows: 16 or 32 lanes a row, several rows per wave (and just outside that form)
          (4096, 16), (5000, 64), (4097, 100), (4100, 4), (6001, 68), (4096, 128), (4095, 64), (4096, 132), (4099, 256), (5000, 200), (4096, 260),
          # a few very long rows: cut into pieces that meet in an atomic max (and just outside that form)
          (3, 131072), (5, 262148), (128, 131072), (129, 131072), (2, 131073), (7, 131068),
          # row lengths that are no multiple of four: rows start at any alignment
          (1000, 1001), (300, 4095), (5, 16383), (2, 70001), (4096, 5), (4096, 3), (77, 66), (33, 4099)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("axis", [0, -1])
def test_quantize_dequantize_absmax_match_oracle(hip, shape, axis):
    rng = np.random.Generator(np.random.Philox(shape[0] * 7919 + shape[1]))
    x = rng.standard_normal(shape, dtype=np.float32)
    x[rng.random(shape) < 0.002] *= 20
    # plant exact ties: half-integers times a power of two survive the division
    x.reshape(-1)[: min(4, x.size)] = np.array([0.5, 1.5, -2.5, 3.5], np.float32)[: min(4, x.size)]
    per_row = axis == 0
    t = dev(x)
    am = t.absmax(axis)
    assert np.array_equal(am.cpu(), oracle.absmax(x, per_row))
    q, s = t.quantize_i8(axis)
    qr, sr = oracle.quantize(x, per_row, threads=CPU_THREADS)
    assert np.array_equal(s.cpu(), sr)
    assert np.array_equal(q.cpu(), qr)
    q2 = t.quantize_i8_with_scale(s, axis)
    assert np.array_equal(q2.cpu(), qr)
    d = q.dequantize(s, axis)
    assert np.array_equal(d.cpu(), oracle.dequantize(qr, sr, per_row))
    for h in (t, am, q, s, q2, d):
        h.release()


@pytest.mark.parametrize("rows,cols", [(0, 16), (5, 0), (0, 0)])
def test_empty_inputs(hip, rows, cols):
    buf = raw_device_buffer(256)
    scales = raw_device_buffer(256)
    for per_row in (0, 1):
        capi.call("vtl_hip_memset", scales.ptr, 0xFF, 256)
        capi.call("vtl_hip_quantize_f32_i8", buf.ptr, rows, cols, per_row, buf.ptr, scales.ptr)
        capi.call("vtl_hip_absmax_f32", buf.ptr, rows, cols, per_row, scales.ptr)
        capi.call("vtl_hip_dequantize_i8_f32", buf.ptr, scales.ptr, rows, cols, per_row, buf.ptr)
        capi.call("vtl_hip_sync")
        n = rows if per_row else 1
        if n:
            assert not d2h(scales.ptr, n, np.float32).any()   # empty slices have absmax 0
    buf.release()
    scales.release()


def test_unaligned_pointers_take_the_scalar_path(hip):
    rng = np.random.Generator(np.random.Philox(99))
    x = rng.standard_normal((6, 128), dtype=np.float32)
    src = raw_device_buffer(x.nbytes + 64)
    dst = raw_device_buffer(x.size + 64)
    sc = raw_device_buffer(64)
    back = raw_device_buffer(x.nbytes + 64)
    h2d(src.ptr + 4, x)                                   # 4-byte aligned only
    for per_row in (1, 0):
        capi.call("vtl_hip_quantize_f32_i8", src.ptr + 4, 6, 128, per_row, dst.ptr + 1, sc.ptr)
        qr, sr = oracle.quantize(x, bool(per_row))
        assert np.array_equal(d2h(dst.ptr + 1, x.shape, np.int8), qr)
        assert np.array_equal(d2h(sc.ptr, sr.shape, np.float32), sr)
        capi.call("vtl_hip_dequantize_i8_f32", dst.ptr + 1, sc.ptr, 6, 128, per_row, back.ptr + 4)
        assert np.array_equal(d2h(back.ptr + 4, x.shape, np.float32), oracle.dequantize(qr, sr, bool(per_row)))
    for h in (src, dst, sc, back):
        h.release()


def test_extreme_scales_take_the_exact_division_path(hip):
    """Subnormal, tiny and huge magnitudes: 1/scale is not usable there."""
    rng = np.random.Generator(np.random.Philox(5))
    base = rng.standard_normal((8, 512), dtype=np.float32)
    for mag in (1e-45, 1e-42, 1e-38, 3e-35, 1e-30, 1e30, 2e37, 3e38):
        x = (base.astype(np.float64) * mag).astype(np.float32)
        q, s = dev(x).quantize_i8(0)
        qr, sr = oracle.quantize(x, True)
        assert np.array_equal(s.cpu(), sr), mag
        assert np.array_equal(q.cpu(), qr), mag


def test_bit_pattern_sweep_against_oracle(hip):
    """Every 2^7-th f32 bit pattern (all exponents, signs, NaNs, infinities,
    subnormals) and a dense window around the clamp boundary, for several
    scales, against the oracle's true division."""
    pats = np.arange(0, 2 ** 32, 2 ** 7, dtype=np.uint64).astype(np.uint32)
    lo = np.float32(120.0).view(np.uint32)
    dense = np.arange(lo, lo + 2 ** 21, dtype=np.uint32)          # 120 .. 136, every float
    x = np.concatenate([pats, dense, dense | np.uint32(0x80000000)]).view(np.float32)
    x = x[: (x.size // 1024) * 1024].reshape(-1, 1024)
    for scale in (1.0, 0.25, 3.7 / 127, 1.0 / 3.0, 1e-3, 7.0, 1e-39, 1e35):
        sc = np.array([scale], np.float32)
        got = _codes_with_scale(hip, x, sc)
        ref = quantize_with_scale_mt(x, sc, False)
        bad = np.argwhere(got != ref)
        assert bad.size == 0, (scale, x[tuple(bad[0])], got[tuple(bad[0])], ref[tuple(bad[0])])
        # dense near-tie sweep scaled so that x/scale crosses every k + 0.5
        with np.errstate(all="ignore"):
            xs = (x * np.float32(scale)).astype(np.float32)
        got = _codes_with_scale(hip, xs, sc)
        ref = quantize_with_scale_mt(xs, sc, False)
        assert np.array_equal(got, ref), scale


@pytest.mark.parametrize("scale", [3.7 / 127, 1e-39])
def test_all_f32_bit_patterns_one_scale(hip, scale):
    """All 2^32 f32 bit patterns through the quantizer with one scale (a normal
    one that is no power of two; a subnormal one, which takes the kernel's
    exact-division path), against the oracle's true division, in chunks of 2^27."""
    sc = np.array([scale], np.float32)
    chunk = 1 << 27
    for c in range((1 << 32) // chunk):
        x = np.arange(c * chunk, (c + 1) * chunk, dtype=np.uint64).astype(np.uint32).view(np.float32)
        x = x.reshape(-1, 1 << 16)
        got = _codes_with_scale(hip, x, sc)
        ref = quantize_with_scale_mt(x, sc, False)
        if not np.array_equal(got, ref):
            bad = tuple(np.argwhere(got != ref)[0])
            raise AssertionError((c, x[bad].view(np.uint32), got[bad], ref[bad]))


def test_engineered_near_ties_per_row(hip):
    """Rows whose quotients sit within an ulp or two of k + 0.5."""
    rng = np.random.Generator(np.random.Philox(17))
    rows, cols = 64, 4096
    am = (np.abs(rng.standard_normal(rows)) + 0.1).astype(np.float32)
    scale = (am / np.float32(127)).astype(np.float32)
    k = rng.integers(-127, 127, (rows, cols))
    x0 = ((k + 0.5) * scale[:, None].astype(np.float64)).astype(np.float32)
    pick = rng.integers(0, 3, (rows, cols))
    x = np.where(pick == 0, x0, np.where(pick == 1, np.nextafter(x0, np.float32(np.inf)),
                                         np.nextafter(x0, np.float32(-np.inf)))).astype(np.float32)
    x[:, 0] = am                                            # pins the row absmax
    x = np.clip(x, -am[:, None], am[:, None]).astype(np.float32)
    q, s = dev(x).quantize_i8(0)
    qr, sr = oracle.quantize(x, True, threads=CPU_THREADS)
    assert np.array_equal(s.cpu(), sr) and np.array_equal(q.cpu(), qr)


def _tensor_quantize(X, rows, cols, Q, S):
    capi.call("vtl_hip_quantize_f32_i8", X.ptr, rows, cols, 0, Q.ptr, S.ptr)


@pytest.mark.parametrize("shape", [(1, 65540), (257, 257), (1000, 1001), (1024, 1024), (2048, 4100), (4096, 4096),
                                   (4096, 4097)])
def test_whole_tensor_quantize_in_two_launches_equals_four(hip, shape, knobs):
    """Above 65536 elements a whole-tensor quantize collects the absmax in cells that the library
    keeps per stream and its second launch derives the scale from them (up to 16 M elements;
    the last shape is past that).  Codes and scale must be those of the four-launch form and
    of the oracle, call after call: a call must not see the maximum of the one before."""
    rows, cols = shape
    rng = np.random.Generator(np.random.Philox(rows * 31 + cols))
    base = rng.standard_normal(shape, dtype=np.float32)
    base.reshape(-1)[:4] = [0.5, 1.5, -2.5, 3.5]
    X = raw_device_buffer(base.nbytes + 16)
    Q = raw_device_buffer(base.size + 16)
    S, A = raw_device_buffer(64), raw_device_buffer(64)
    small = rows * cols <= 1 << 21
    # descending magnitudes: a maximum left over from an earlier call would show
    for step, (mag, off) in enumerate(((64.0, 0), (1.0, 0), (1.0, 4), (0.015625, 0), (0.0, 0))):
        if off and not small:
            continue
        x = base * np.float32(mag)
        if step == 1:
            x[rows // 2, cols // 3] = np.nan        # ignored by the absmax, code 0
        h2d(X.ptr + off, x)
        want_q, want_s = oracle.quantize(x, False, threads=CPU_THREADS)
        got = {}
        for form in ("two", "four"):
            if form == "four":
                knobs.setenv("VTL_HIP_QUANT_FOUR_LAUNCHES", "1")
            capi.call("vtl_hip_memset", S.ptr, 0xFF, 64)
            capi.call("vtl_hip_quantize_f32_i8", X.ptr + off, rows, cols, 0, Q.ptr + off // 4, S.ptr)
            capi.call("vtl_hip_absmax_f32", X.ptr + off, rows, cols, 0, A.ptr)
            got[form] = (d2h(Q.ptr + off // 4, shape, np.int8), d2h(S.ptr, 1, np.float32), d2h(A.ptr, 1, np.float32))
            if form == "four":
                knobs.delenv("VTL_HIP_QUANT_FOUR_LAUNCHES")
        for form, (codes, scale, amax) in got.items():
            assert scale.view(np.uint32)[0] == want_s.view(np.uint32).reshape(-1)[0], (form, step)
            assert amax[0] == oracle.absmax(x, False).reshape(-1)[0], (form, step)
            assert np.array_equal(codes, want_q), (form, step)
    for h in (X, Q, S, A):
        h.release()


def test_whole_tensor_quantize_on_many_streams(hip):
    """Every stream has absmax cells of its own (the first 16 streams that ask; further ones
    take the four-launch form): calls enqueued on 20 streams without waiting in between, three
    rounds with a different tensor per stream and round, each give their own scale and codes."""
    import ctypes as C
    hiprt = C.CDLL("libamdhip64.so")
    rows, cols = 300, 1000
    rng = np.random.Generator(np.random.Philox(4242))
    lanes = []
    try:
        for i in range(20):
            st = C.c_void_p()
            assert hiprt.hipStreamCreate(C.byref(st)) == 0
            xs = [rng.standard_normal((rows, cols), dtype=np.float32) * np.float32(2.0 ** (i % 7 - rnd)) for rnd in range(3)]
            lanes.append({"stream": st, "xs": xs, "X": [dev(x) for x in xs],
                          "Q": [raw_device_buffer(rows * cols) for _ in xs], "S": [raw_device_buffer(64) for _ in xs]})
        for rnd in range(3):
            for ln in lanes:
                capi.call("vtl_hip_set_stream", ln["stream"])
                _tensor_quantize(ln["X"][rnd], rows, cols, ln["Q"][rnd], ln["S"][rnd])
        for ln in lanes:
            capi.call("vtl_hip_set_stream", ln["stream"])
            capi.call("vtl_hip_sync")
        for i, ln in enumerate(lanes):
            for rnd in range(3):
                want_q, want_s = oracle.quantize(ln["xs"][rnd], False, threads=CPU_THREADS)
                assert d2h(ln["S"][rnd].ptr, 1, np.float32)[0] == want_s.reshape(-1)[0], (i, rnd)
                assert np.array_equal(d2h(ln["Q"][rnd].ptr, (rows, cols), np.int8), want_q), (i, rnd)
    finally:
        capi.call("vtl_hip_set_stream", None)
        capi.call("vtl_hip_sync")
        for ln in lanes:
            hiprt.hipStreamDestroy(ln["stream"])
            for t in [*ln["X"], *ln["Q"], *ln["S"]]:
                t.release()


def test_whole_tensor_quantize_under_stream_capture(hip):
    """The cells a call uses alternate from call to call, which a recorded graph cannot follow:
    under capture the library records the form that uses the caller's memory only, and replays
    with eager calls between them all give the oracle's bits."""
    import ctypes as C
    hiprt = C.CDLL("libamdhip64.so")
    stream, graph, gexec = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert hiprt.hipStreamCreate(C.byref(stream)) == 0
    rows, cols = 512, 1024
    rng = np.random.Generator(np.random.Philox(515))
    x = rng.standard_normal((rows, cols), dtype=np.float32)
    X = dev(x)
    Q, S, A = raw_device_buffer(rows * cols), raw_device_buffer(64), raw_device_buffer(64)

    def call():
        _tensor_quantize(X, rows, cols, Q, S)
        capi.call("vtl_hip_absmax_f32", X.ptr, rows, cols, 0, A.ptr)

    def check(xr, what):
        want_q, want_s = oracle.quantize(xr, False, threads=CPU_THREADS)
        assert d2h(S.ptr, 1, np.float32)[0] == want_s.reshape(-1)[0], what
        assert d2h(A.ptr, 1, np.float32)[0] == np.abs(xr).max(), what
        assert np.array_equal(d2h(Q.ptr, (rows, cols), np.int8), want_q), what

    try:
        capi.call("vtl_hip_set_stream", stream)
        call()
        capi.call("vtl_hip_sync")
        check(x, "eager")
        assert hiprt.hipStreamBeginCapture(stream, 0) == 0
        call()
        assert hiprt.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert hiprt.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
        for rep in range(4):
            xr = (rng.standard_normal((rows, cols)) * 2.0 ** (3 - rep)).astype(np.float32)
            capi.call("vtl_hip_memcpy_h2d", X.ptr, xr.ctypes.data, xr.nbytes)
            if rep % 2:
                call()
                capi.call("vtl_hip_sync")
                check(xr, f"eager {rep}")
                capi.call("vtl_hip_memset", Q.ptr, 0, rows * cols)
            assert hiprt.hipGraphLaunch(gexec, stream) == 0
            capi.call("vtl_hip_sync")
            check(xr, f"replay {rep}")
    finally:
        capi.call("vtl_hip_set_stream", None)
        if gexec:
            hiprt.hipGraphExecDestroy(gexec)
        if graph:
            hiprt.hipGraphDestroy(graph)
        hiprt.hipStreamDestroy(stream)
        for t in (X, Q, S, A):
            t.release()


def test_relu_matches_oracle(hip):
    x = np.array([-1.0, -0.0, 0.0, 2.5, -1e-30, np.inf, -np.inf, np.nan] * 37, np.float32)
    t = dev(x)
    got = t.relu_().cpu()
    ref = oracle.relu(x)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))   # bit patterns, incl. -0.0 and NaN


def test_roundtrip_config_full_size(hip):
    """Config 2 at its real size [16384,16384]: oracle parity on a sample of
    rows, properties on everything."""
    rows = cols = 16384
    x = workloads.outlier_matrix(rows, cols)
    t = dev(x)
    q, s = t.quantize_i8(0)
    d = q.dequantize(s, 0)
    codes, scales = q.cpu(), s.cpu()
    sample = np.r_[0:64, 8000:8064, rows - 64:rows]
    qr, sr = oracle.quantize(x[sample], True, threads=CPU_THREADS)
    assert np.array_equal(scales[sample], sr) and np.array_equal(codes[sample], qr)
    xh = d.cpu()
    assert np.array_equal(xh[sample], oracle.dequantize(qr, sr, True))
    # properties over the whole tensor
    assert np.array_equal(scales, np.abs(x).max(axis=1) / np.float32(127))
    assert codes.min() >= -127 and np.all(np.abs(codes).max(axis=1) == 127)
    # half a step, plus the rounding of the quotient (<= 127 * 2^-24 steps) and of the product
    assert np.all(np.abs(x - xh) <= scales[:, None] * np.float32(0.50002))
    # re-quantizing the dequantized tensor with the same scales returns the codes
    q2 = d.quantize_i8_with_scale(s, 0)
    assert np.array_equal(q2.cpu(), codes)
    # whole-tensor mode on the same data
    qt, st = t.quantize_i8(-1)
    assert st.cpu()[0] == np.abs(x).max() / np.float32(127)
    assert np.array_equal(qt.cpu()[sample], oracle.quantize_with_scale(x[sample], st.cpu(), False))
    for h in (t, q, s, d, q2, qt, st):
        h.release()
