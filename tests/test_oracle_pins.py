"""Pins the CPU oracle before anything is compared against it.

Every check here is independent of the oracle's own formulae: the reference's
own unit-test vectors for the vocabulary the path is composed from, hand-derived
known answers (tests/golden/kat_vectors.json), exact rational arithmetic, numpy
routines, closed forms and invariants.  CPU only.
"""
import json
import math
import os
from fractions import Fraction

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "kat_vectors.json")))


def f32(v):
    if isinstance(v, str):
        return np.float32(float(v))
    return np.float32(v)


def f32_list(vs):
    return np.array([f32(v) for v in vs], np.float32)


# ---- reference vocabulary vectors -------------------------------------------------

def test_abs_and_max_vectors_from_reference_tests():
    voc = KAT["reference_vocabulary"]
    a = voc["abs"]
    x = np.array([a["in"]], np.float32)
    # absmax of each single element == abs (tests/core/math_test.v:5-10)
    got = [oracle.absmax(x[:, i:i + 1], per_row=True)[0] for i in range(x.shape[1])]
    assert got == a["out"]
    m = voc["max_axis_1"]   # tests/core/reduction_test.v:49-54, non-negative entries
    assert oracle.absmax(np.array(m["in"], np.float32), per_row=True).tolist() == m["out"]
    for case in voc["stats_max"]["cases"]:  # stats/stats_test.v:228-240
        x = np.array([case["in"]], np.float32)
        expect = np.float32(max(abs(v) for v in case["in"]))
        assert oracle.absmax(x, per_row=False)[0] == expect
        if min(case["in"]) >= 0:
            assert oracle.absmax(x, per_row=False)[0] == np.float32(case["out"])


def test_divide_and_multiply_scalar_vectors_from_reference_tests():
    voc = KAT["reference_vocabulary"]
    d = voc["divide_scalar"]   # x / 2.0 -> halves; rne(halves) known by hand
    x = np.array(d["in"], np.float32)
    q = oracle.quantize_with_scale(x, np.array([d["scalar"]], np.float32), per_row=False)
    halves = np.array(d["out"], np.float64)
    expect = np.array([[0, 1, 2, 2], [2, 3, 4, 4]], np.int8)  # rne of .5 1 1.5 2 / 2.5 3 3.5 4
    assert np.array_equal(np.rint(halves).astype(np.int8), expect)
    assert np.array_equal(q, expect)
    m = voc["multiply_scalar"]  # tests/core/math_op_test.v:88-93
    codes = np.array(m["in"], np.int8)
    got = oracle.dequantize(codes, np.array([m["scalar"]], np.float32), per_row=False)
    assert np.array_equal(got, np.array(m["out"], np.float32))


def test_matmul_identity_vector_from_reference_tests():
    v = KAT["reference_vocabulary"]["matmul_identity"]   # la/la_test.v:30-37
    a = np.array(v["a"], np.int8)
    b = np.array(v["b"], np.int8)
    # C = A.B with B given K-contiguous, i.e. as B^T rows
    got = oracle.gemm_i8_i32(a, np.ascontiguousarray(b.T))
    assert np.array_equal(got, np.array(v["out"], np.int32))


def test_f32_linear_vector_from_reference_tests():
    v = KAT["reference_vocabulary"]["linear_f64_session"]
    y = oracle.linear_f32_via_f64(np.array(v["x"], np.float32), np.array(v["w"], np.float32),
                                  np.array(v["b"], np.float32))
    assert y.shape == (1, 2)
    assert np.allclose(y, np.array(v["out"], np.float32), rtol=1e-6, atol=0)


def test_f32_linear_against_numpy_f64():
    rng = np.random.default_rng(7)
    x = rng.standard_normal((9, 33)).astype(np.float32)
    w = rng.standard_normal((5, 33)).astype(np.float32)
    b = rng.standard_normal((1, 5)).astype(np.float32)
    ref = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32) + b
    got = oracle.linear_f32_via_f64(x, w, b)
    # a transposed operand or a dropped bias fails this by orders of magnitude
    assert np.allclose(got, ref, rtol=1e-6, atol=1e-6)


# ---- rounding known answers -----------------------------------------------------------

@pytest.mark.parametrize("name", ["round_half_even", "scaled_ties"])
def test_round_half_even_known_answers(name):
    k = KAT[name]
    for x, code in zip(k["x"], k["code"]):
        assert oracle.quantize_one(f32(x), f32(k["scale"])) == code, (x, code)


def test_special_values():
    s = KAT["special_values"]
    c = s["nan_with_scale_1"]
    assert [oracle.quantize_one(f32(v), 1.0) for v in c["x"]] == c["code"]
    z = s["all_zero_row"]
    q, sc = oracle.quantize(f32_list(z["x"])[None, :], per_row=True)
    assert sc[0] == 0.0 and q[0].tolist() == z["code"]
    assert oracle.dequantize(q, sc, per_row=True)[0].tolist() == z["dequant"]
    i = s["inf_row"]
    q, sc = oracle.quantize(f32_list(i["x"])[None, :], per_row=True)
    assert math.isinf(sc[0]) and q[0].tolist() == i["code"]
    n = s["nan_ignored_by_absmax"]
    assert oracle.absmax(f32_list(n["x"])[None, :], per_row=True)[0] == n["absmax"]
    assert oracle.absmax(f32_list(n["x"])[None, :], per_row=False)[0] == n["absmax"]


def test_row_quantize_known_answers():
    for case in KAT["row_quantize"]["cases"]:
        x = np.array([case["x"]], np.float32)
        for per_row in (True, False):
            q, s = oracle.quantize(x, per_row=per_row)
            assert s[0] == np.float32(case["scale"])
            assert q[0].tolist() == case["code"]


# ---- exact arithmetic ---------------------------------------------------------------------

def _rne_fraction(fr: Fraction) -> int:
    fl = math.floor(fr)
    rem = fr - fl
    if rem > Fraction(1, 2):
        return fl + 1
    if rem < Fraction(1, 2):
        return fl
    return fl if fl % 2 == 0 else fl + 1


def _round_to_f32(fr: Fraction) -> Fraction:
    """Correctly rounded (nearest-even) binary32 value of a rational, normal range."""
    if fr == 0:
        return Fraction(0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = math.floor(math.log2(float(a)))
    while Fraction(2) ** e > a:
        e -= 1
    while Fraction(2) ** (e + 1) <= a:
        e += 1
    ulp = Fraction(2) ** (e - 23)
    return sign * _rne_fraction(a / ulp) * ulp


def test_quantize_one_against_exact_rationals():
    """x/scale rounded once to f32 (checked against exact rationals), then tie-to-even,
    then clamp: evaluated with fractions, no floating point involved."""
    rng = np.random.default_rng(11)
    xs = rng.standard_normal(300).astype(np.float32) * np.float32(3.0)
    scales = np.abs(rng.standard_normal(300)).astype(np.float32) * np.float32(0.05) + np.float32(1e-3)
    # add engineered near-tie cases: x = (k + 0.5) * s rounded to f32
    ks = rng.integers(-126, 127, 100)
    s2 = np.abs(rng.standard_normal(100)).astype(np.float32) + np.float32(0.01)
    x2 = ((ks + 0.5) * s2.astype(np.float64)).astype(np.float32)
    xs = np.concatenate([xs, x2])
    scales = np.concatenate([scales, s2])
    for x, s in zip(xs, scales):
        quotient = _round_to_f32(Fraction(float(x)) / Fraction(float(s)))
        assert quotient == Fraction(float(np.float32(x) / np.float32(s)))  # numpy f32 division is IEEE
        code = max(-127, min(127, _rne_fraction(quotient)))
        assert oracle.quantize_one(x, s) == code, (x, s)


def test_scale_is_one_f32_division():
    rng = np.random.default_rng(5)
    for a in np.abs(rng.standard_normal(200)).astype(np.float32) * np.float32(10):
        assert oracle.scale_from_absmax(a) == np.float32(a) / np.float32(127.0)
        assert Fraction(float(oracle.scale_from_absmax(a))) == _round_to_f32(Fraction(float(a)) / 127)


# ---- numpy cross-checks and invariants ---------------------------------------------------------

def _numpy_quantize(x, per_row):
    """Independent restatement with numpy primitives (np.rint is ties-to-even)."""
    ax = np.abs(x)
    am = np.nanmax(np.where(np.isnan(ax), 0, ax), axis=1) if per_row else \
        np.array([np.nanmax(np.where(np.isnan(ax), 0, ax))], np.float32)
    am = am.astype(np.float32)
    scale = am / np.float32(127.0)
    s = scale[:, None] if per_row else scale[0]
    with np.errstate(divide="ignore", invalid="ignore"):
        t = (x / s).astype(np.float32)
    r = np.rint(t)
    r = np.where(np.isnan(r), 0, np.clip(r, -127, 127))
    return r.astype(np.int8), scale


@pytest.mark.parametrize("shape", [(1, 1), (3, 7), (16, 784), (5, 4096), (2, 16384), (64, 129)])
@pytest.mark.parametrize("per_row", [True, False])
def test_quantize_matches_numpy(shape, per_row):
    rng = np.random.default_rng(shape[0] * 1000 + shape[1])
    x = rng.standard_normal(shape).astype(np.float32)
    x[rng.random(shape) < 0.01] *= 20
    q, s = oracle.quantize(x, per_row=per_row)
    qn, sn = _numpy_quantize(x, per_row)
    assert np.array_equal(s, sn)
    assert np.array_equal(q, qn)
    assert np.array_equal(oracle.absmax(x, per_row), np.abs(x).max(axis=1) if per_row else [np.abs(x).max()])
    # multithreaded form is the same arithmetic
    q2, s2 = oracle.quantize(x, per_row=per_row, threads=4)
    assert np.array_equal(q, q2) and np.array_equal(s, s2)


def test_quantize_invariants():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((32, 512)).astype(np.float32)
    q, s = oracle.quantize(x, per_row=True)
    assert q.min() >= -127 and q.max() <= 127            # -128 never produced
    am = np.abs(x).max(axis=1)
    hit = np.abs(x) == am[:, None]
    assert np.all(np.abs(q[hit]) == 127)                 # the absmax element maps to +-127
    qn, sn = oracle.quantize(-x, per_row=True)
    assert np.array_equal(qn, -q) and np.array_equal(sn, s)          # odd symmetry
    perm = rng.permutation(x.shape[1])
    qp, sp = oracle.quantize(x[:, perm], per_row=True)
    assert np.array_equal(qp, q[:, perm]) and np.array_equal(sp, s)  # permutation invariance
    for kexp in (-20, -3, 5, 40):                                    # power-of-two scaling
        qk, sk = oracle.quantize(x * np.float32(2.0 ** kexp), per_row=True)
        assert np.array_equal(qk, q)
        assert np.array_equal(sk, s * np.float32(2.0 ** kexp))
    xh = oracle.dequantize(q, s, per_row=True)
    # within half a quantization step, plus the rounding of the quotient (<= 127 * 2^-24 steps)
    assert np.all(np.abs(x - xh) <= s[:, None] * np.float32(0.50002))


def test_dequantize_matches_numpy():
    rng = np.random.default_rng(9)
    q = rng.integers(-127, 128, (17, 300), dtype=np.int8)
    s_row = np.abs(rng.standard_normal(17)).astype(np.float32)
    assert np.array_equal(oracle.dequantize(q, s_row, True), q.astype(np.float32) * s_row[:, None])
    s_one = np.array([0.0123], np.float32)
    assert np.array_equal(oracle.dequantize(q, s_one, False), q.astype(np.float32) * s_one[0])
    assert np.array_equal(oracle.dequantize(q, s_row, True, threads=3), oracle.dequantize(q, s_row, True))


@pytest.mark.parametrize("mnk", [(1, 1, 1), (5, 7, 64), (33, 65, 48), (64, 256, 784), (17, 19, 23)])
def test_gemm_matches_numpy_int64(mnk):
    m, n, k = mnk
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    a = rng.integers(-127, 128, (m, k), dtype=np.int8)
    bt = rng.integers(-127, 128, (n, k), dtype=np.int8)
    ref = a.astype(np.int64) @ bt.astype(np.int64).T
    for threads in (1, 4):
        got = oracle.gemm_i8_i32(a, bt, threads=threads)
        assert got.dtype == np.int32 and np.array_equal(got, ref)


@pytest.mark.parametrize("k", KAT["gemm_closed_forms"]["k_values"])
def test_gemm_closed_forms(k):
    ones = np.full((3, k), 127, np.int8)
    assert np.all(oracle.gemm_i8_i32(ones, ones) == k * 16129)
    assert np.all(oracle.gemm_i8_i32(ones, -ones) == -k * 16129)
    alt = np.tile(np.array([1, -1], np.int8), k // 2)[None, :].repeat(3, 0)
    assert np.all(oracle.gemm_i8_i32(alt, np.ones((4, k), np.int8)) == 0)
    eye = np.eye(k, dtype=np.int8)[:8] * 127           # 127 * I picks out rows of Bt
    b = np.arange(5 * k, dtype=np.int64).reshape(5, k) % 255 - 127
    assert np.array_equal(oracle.gemm_i8_i32(eye, b.astype(np.int8)), 127 * b[:, :8].T)


def test_epilogue_known_answers_and_op_order():
    e = KAT["epilogue"]
    acc = np.array(e["acc"], np.int32)
    sa, sw, bias = f32_list(e["sa"]), f32_list(e["sw"]), f32_list(e["bias"])
    assert np.array_equal(oracle.epilogue(acc, sa, sw, bias), np.array(e["out"], np.float32))
    assert np.array_equal(oracle.epilogue(acc, sa, sw, bias, relu=True), np.array(e["out_relu"], np.float32))
    # op-by-op numpy float32 evaluation on random values (each step rounded separately)
    rng = np.random.default_rng(21)
    acc = rng.integers(-6 * 10 ** 7, 6 * 10 ** 7, (13, 29), dtype=np.int32)
    sa = (rng.uniform(0.5, 1.5, 13) / 127).astype(np.float32)
    sw = (rng.uniform(0.5, 1.5, 29) / 127).astype(np.float32)
    bias = (rng.standard_normal(29) * 0.02).astype(np.float32)
    s = (sa[:, None] * sw[None, :]).astype(np.float32)
    y = (acc.astype(np.float32) * s).astype(np.float32)
    yb = (y + bias[None, :]).astype(np.float32)
    assert np.array_equal(oracle.epilogue(acc, sa, sw, bias), yb)
    assert np.array_equal(oracle.epilogue(acc, sa, sw, None), y)
    assert np.array_equal(oracle.epilogue(acc, sa, sw, bias, relu=True), np.where(yb < 0, np.float32(0), yb))
    # scalar scales broadcast
    assert np.array_equal(oracle.epilogue(acc, sa[:1], sw[:1], None),
                          (acc.astype(np.float32) * np.float32(sa[0] * sw[0])).astype(np.float32))
    # against f64: three roundings of ~2^-24 each
    y64 = acc.astype(np.float64) * sa[:, None].astype(np.float64) * sw[None, :] + bias[None, :]
    assert np.allclose(yb, y64, rtol=3e-7, atol=1e-9)


def test_relu_closed_form():
    x = np.array([-1.0, -0.0, 0.0, 2.5, -1e-30, np.inf, -np.inf], np.float32)
    y = oracle.relu(x)
    assert y.tolist() == [0.0, -0.0, 0.0, 2.5, 0.0, np.inf, 0.0]
    assert np.signbit(y[1])                       # -0.0 is not < 0 and passes through
    assert np.isnan(oracle.relu(np.array([np.nan], np.float32))[0])


def test_linear_compositions_agree():
    rng = np.random.default_rng(31)
    x = rng.standard_normal((6, 96)).astype(np.float32)
    w = rng.standard_normal((10, 96)).astype(np.float32) * np.float32(0.02)
    bias = rng.standard_normal(10).astype(np.float32)
    wq, sw = oracle.quantize(w, per_row=True)
    xq, sx = oracle.quantize(x, per_row=True)
    acc = xq.astype(np.int64) @ wq.astype(np.int64).T
    expect = oracle.epilogue(acc.astype(np.int32), sx, sw, bias, relu=True)
    assert np.array_equal(oracle.linear_i8_f32(xq, sx, wq, sw, bias, relu=True), expect)
    assert np.array_equal(oracle.linear_f32_dynquant(x, wq, sw, bias, relu=True), expect)
    # the int8 linear approximates the f32 linear (sanity of the whole composition)
    ref = x @ w.T + bias
    got = oracle.linear_f32_dynquant(x, wq, sw, bias, relu=False)
    assert np.abs(got - ref).max() < 0.05 * np.abs(ref).max()
