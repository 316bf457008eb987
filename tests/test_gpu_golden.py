"""The five benchmark configurations at their full sizes on the device, against
the committed SHA-256 digests of the CPU oracle's outputs
(tests/golden/config_fixtures.json): every byte of every output, without
running the oracle on the GPU box."""
import hashlib
import json
import os

import numpy as np
import pytest

from helpers import dev
from vtl_amd import workloads
from vtl_amd.tensor import HipTensor, gemm_i8_hip, linear_f32_dynquant_hip, linear_i8_hip

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = json.load(open(os.path.join(HERE, "golden", "config_fixtures.json")))


def digest(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).view(np.uint8).reshape(-1)).hexdigest()


def check(fx: dict, key: str, arr: np.ndarray):
    assert list(arr.shape) == fx[key]["shape"] and str(arr.dtype) == fx[key]["dtype"], key
    assert digest(arr) == fx[key]["sha256"], f"{key}: digest differs (first values {arr.reshape(-1)[:4]})"


def test_config0_mnist_first_layer(hip):
    fx = FIXTURES["configs[0]"]
    x, w, b = workloads.mnist_mlp_first_layer()
    check(fx, "x", x), check(fx, "w", w)
    X, W, B = dev(x), dev(w), dev(b.reshape(-1))
    xq, sx = X.quantize_i8(-1)
    wq, sw = W.quantize_i8(-1)
    check(fx, "xq", xq.cpu()), check(fx, "sx", sx.cpu().reshape(-1))
    check(fx, "wq", wq.cpu()), check(fx, "sw", sw.cpu().reshape(-1))
    y = linear_i8_hip(xq, sx, wq, sw, B)
    check(fx, "y", y.cpu())
    for t in (X, W, B, xq, sx, wq, sw, y):
        t.release()


def test_config1_quantize_dequantize_roundtrip(hip):
    fx = FIXTURES["configs[1]"]
    x = workloads.outlier_matrix()
    check(fx, "x", x)
    X = dev(x)
    del x
    q, s = X.quantize_i8(0)
    check(fx, "q", q.cpu()), check(fx, "scales", s.cpu().reshape(-1))
    d = q.dequantize(s, 0)
    check(fx, "dequantized", d.cpu())
    for t in (X, q, s, d):
        t.release()


def test_config2_square_int8_linear(hip):
    fx = FIXTURES["configs[2]"]
    a, bt, sa, sb, bias = workloads.square_int8_gemm()
    for k, v in (("a", a), ("bt", bt), ("sa", sa), ("sb", sb), ("bias", bias)):
        check(fx, k, v)
    A, B, SA, SB, BIAS = dev(a), dev(bt), dev(sa), dev(sb), dev(bias)
    acc = HipTensor.empty([4096, 4096], np.int32)
    gemm_i8_hip(acc, A, B)
    check(fx, "acc", acc.cpu())
    y = linear_i8_hip(A, SA, B, SB, BIAS)
    check(fx, "y", y.cpu())
    for t in (A, B, SA, SB, BIAS, acc, y):
        t.release()


def test_config3_decode_linear(hip):
    fx = FIXTURES["configs[3]"]
    _, w = workloads.decode_linear(1)
    check(fx, "w", w)
    W = dev(w)
    wq, sw = W.quantize_i8(0)
    check(fx, "wq", wq.cpu()), check(fx, "sw", sw.cpu().reshape(-1))
    for m in (1, 8, 32, 128):
        x, _ = workloads.decode_linear(m)
        check(fx[f"M={m}"], "x", x)
        X = dev(x)
        y = linear_f32_dynquant_hip(X, wq, sw, None)
        check(fx[f"M={m}"], "y", y.cpu())
        X.release(), y.release()
    for t in (W, wq, sw):
        t.release()


def test_config4_mlp_chain(hip):
    fx = FIXTURES["configs[4]"]
    x, ws = workloads.mlp_chain()
    check(fx, "x", x)
    cur = dev(x)
    for i, w in enumerate(ws):
        check(fx[f"layer{i}"], "w", w)
        W = dev(w)
        wq, sw = W.quantize_i8(0)
        check(fx[f"layer{i}"], "wq", wq.cpu())
        nxt = linear_f32_dynquant_hip(cur, wq, sw, None, relu=i < len(ws) - 1)
        check(fx[f"layer{i}"], "y", nxt.cpu())
        for t in (W, wq, sw, cur):
            t.release()
        cur = nxt
    cur.release()
