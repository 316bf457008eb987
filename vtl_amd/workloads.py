"""Synthetic inputs of the five benchmark configurations.

The reference's own RNG cannot be seeded (`random_seed` ignores its argument,
rand.v:82-84), so "seed N" means this module's generator: numpy's
counter-based Philox, seeded with N.  Every function takes size arguments so
that tests can draw the same distributions at reduced sizes.
"""
from __future__ import annotations

import numpy as np


def _rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.Philox(seed))


def mnist_mlp_first_layer(batch: int = 64, in_features: int = 784, out_features: int = 256,
                          seed: int = 0):
    """Config 1: activations U[0,1), Kaiming-uniform weights stored [out, in]
    (limit per nn/internal/init.v:21-65, whose compute_fans multiplies the
    fan by shape[1]), zero bias [1, out]; per-tensor quantization of both."""
    rng = _rng(seed)
    x = rng.random((batch, in_features), dtype=np.float32)
    fan = out_features * in_features
    limit = np.float32(np.sqrt(3.0) * np.sqrt(2.0 / fan))
    w = rng.uniform(-limit, limit, (out_features, in_features)).astype(np.float32)
    b = np.zeros((1, out_features), np.float32)
    return x, w, b


def outlier_matrix(rows: int = 16384, cols: int = 16384, seed: int = 1, chunk_rows: int = 1024,
                   out: np.ndarray | None = None) -> np.ndarray:
    """Config 2: ~N(0,1) with each element independently multiplied by 20 with
    probability 0.001.  Generated in row chunks to bound host memory."""
    rng = _rng(seed)
    x = out if out is not None else np.empty((rows, cols), np.float32)
    for r0 in range(0, rows, chunk_rows):
        r1 = min(rows, r0 + chunk_rows)
        blk = rng.standard_normal((r1 - r0, cols), dtype=np.float32)
        mask = rng.random((r1 - r0, cols), dtype=np.float32) < np.float32(0.001)
        blk[mask] *= np.float32(20.0)
        x[r0:r1] = blk
    return x


def square_int8_gemm(m: int = 4096, n: int = 4096, k: int = 4096, seed: int = 2):
    """Config 3: int8 codes uniform in [-127,127], per-row / per-column f32
    scales U[0.5,1.5)/127, bias ~N(0, 0.02)."""
    rng = _rng(seed)
    a = rng.integers(-127, 128, (m, k), dtype=np.int8)
    bt = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sa = (rng.uniform(0.5, 1.5, m) / 127.0).astype(np.float32)
    sb = (rng.uniform(0.5, 1.5, n) / 127.0).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.02).astype(np.float32)
    return a, bt, sa, sb, bias


def decode_linear_activations(m: int, k: int = 4096, seed: int = 3) -> np.ndarray:
    """Config 4's activations ~N(0,1) [m, k] alone (a stream of their own per m, so that the
    weights do not depend on m)."""
    return _rng(seed * 1000 + m).standard_normal((m, k), dtype=np.float32)


def decode_linear(m: int, k: int = 4096, n: int = 14336, seed: int = 3):
    """Config 4: f32 weights ~N(0, 0.02) stored [n, k], activations ~N(0,1) [m, k]."""
    rng = _rng(seed)
    w = (rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))
    return decode_linear_activations(m, k, seed), w


def xavier_uniform(out_features: int, in_features: int, rng: np.random.Generator) -> np.ndarray:
    limit = np.sqrt(6.0 / (in_features + out_features))
    return rng.uniform(-limit, limit, (out_features, in_features)).astype(np.float32)


def mlp_chain(batch: int = 256, dims=(4096, 11008, 4096, 1024), seed: int = 4):
    """Config 5: x ~N(0,1) [batch, dims[0]], Xavier-uniform weights
    [dims[i+1], dims[i]], no bias; ReLU after every layer but the last."""
    rng = _rng(seed)
    x = rng.standard_normal((batch, dims[0]), dtype=np.float32)
    ws = [xavier_uniform(dims[i + 1], dims[i], rng) for i in range(len(dims) - 1)]
    return x, ws
