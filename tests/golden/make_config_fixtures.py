#!/usr/bin/env python3
"""Writes tests/golden/config_fixtures.json: SHA-256 digests of the inputs and of
the expected outputs of the five benchmark configurations at their full sizes.

The inputs come from vtl_amd.workloads (numpy Philox, seeded); the expected
outputs from the CPU oracle (oracle/, pinned by tests/test_oracle_pins.py).
Nothing of the reference is imported or run.  The GPU tests hash what the
device produced and compare; the CPU tests re-derive the cheaper entries with
the oracle, so a drift of the generator, of numpy or of the oracle shows up.

    python tests/golden/make_config_fixtures.py            (about a minute on 8 cores)
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from vtl_amd import workloads  # noqa: E402

THREADS = min(16, os.cpu_count() or 1)


def digest(a: np.ndarray) -> str:
    a = np.ascontiguousarray(a)
    return hashlib.sha256(a.view(np.uint8).reshape(-1)).hexdigest()


def entry(**arrays):
    return {k: {"sha256": digest(v), "dtype": str(v.dtype), "shape": list(v.shape),
                "head": [float(t) for t in np.asarray(v).reshape(-1)[:4]]} for k, v in arrays.items()}


def config1():
    x, w, b = workloads.mnist_mlp_first_layer()
    xq, sx = oracle.quantize(x, False)
    wq, sw = oracle.quantize(w, False)
    y = oracle.linear_i8_f32(xq, sx, wq, sw, b.reshape(-1))
    return entry(x=x, w=w, xq=xq, sx=sx, wq=wq, sw=sw, y=y)


def config2():
    x = workloads.outlier_matrix()
    q, s = oracle.quantize(x, True, threads=THREADS)
    d = oracle.dequantize(q, s, True, threads=THREADS)
    return entry(x=x, q=q, scales=s, dequantized=d)


def config3():
    a, bt, sa, sb, bias = workloads.square_int8_gemm()
    acc = oracle.gemm_i8_i32(a, bt, threads=THREADS)
    y = oracle.epilogue(acc, sa, sb, bias)
    return entry(a=a, bt=bt, sa=sa, sb=sb, bias=bias, acc=acc, y=y)


def config4():
    out = {}
    w = None
    for m in (1, 8, 32, 128):
        x, w = workloads.decode_linear(m)
        if "wq" not in out:
            wq, sw = oracle.quantize(w, True, threads=THREADS)
            out.update(entry(w=w, wq=wq, sw=sw))
        y = oracle.linear_f32_dynquant(x, wq, sw, None, threads=THREADS)
        out.update({f"M={m}": entry(x=x, y=y)})
    return out


def config5():
    x, ws = workloads.mlp_chain()
    out = entry(x=x)
    cur = x
    for i, w in enumerate(ws):
        wq, sw = oracle.quantize(w, True, threads=THREADS)
        cur = oracle.linear_f32_dynquant(cur, wq, sw, None, relu=i < len(ws) - 1, threads=THREADS)
        out.update({f"layer{i}": entry(w=w, wq=wq, y=cur)})
    return out


def main():
    fixtures = {"_comment": "SHA-256 of inputs (vtl_amd.workloads, numpy Philox) and of the CPU oracle's outputs "
                            "for the five benchmark configurations at full size; made by make_config_fixtures.py",
                "numpy": np.__version__}
    for name, fn in (("configs[0]", config1), ("configs[1]", config2), ("configs[2]", config3),
                     ("configs[3]", config4), ("configs[4]", config5)):
        print(name, flush=True)
        fixtures[name] = fn()
    with open(os.path.join(HERE, "config_fixtures.json"), "w") as f:
        json.dump(fixtures, f, indent=1)
    print("written", os.path.join(HERE, "config_fixtures.json"))


if __name__ == "__main__":
    main()
