"""GPU parity of the layer-level path (linear_forward_f32 hook, QuantLinearLayer,
Sequential) on the benchmark configurations, through the host-side mirror."""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import CPU_THREADS, KAT, dev, rel_err
from vtl_amd import (PER_CHANNEL, PER_TENSOR, HipSession, QuantLinearLayer, Sequential, capi, linear_i8_requant_hip,
                     linear_forward_hip_f32, workloads)
from vtl_amd.tensor import HipTensor, linear_f32_dynquant_hip

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("guard_bands")]

F32_REL_TOL = 1e-5


def _oracle_linear(x, w, bias, mode, relu=False):
    per_row = mode == PER_CHANNEL
    wq, sw = oracle.quantize(w, per_row, threads=CPU_THREADS)
    xq, sx = oracle.quantize(x, per_row, threads=CPU_THREADS)
    b = None if bias is None else np.asarray(bias, np.float32).reshape(-1)
    return oracle.linear_i8_f32(xq, sx, wq, sw, b, relu=relu, threads=CPU_THREADS)


def test_mnist_mlp_first_layer_config(hip, monkeypatch):
    """Config 1: [64,784] x [256,784]^T, per-tensor scales, zero bias."""
    monkeypatch.setenv("VTL_USE_HIP", "1")
    x, w, b = workloads.mnist_mlp_first_layer()
    got = linear_forward_hip_f32(x, w, b, mode=PER_TENSOR)
    want = _oracle_linear(x, w, b, PER_TENSOR)
    assert got.shape == (64, 256)
    assert rel_err(got, want) <= F32_REL_TOL and np.array_equal(got, want)
    # the int8 result tracks the reference's documented f32 Linear y = x.W^T + b
    f32 = oracle.linear_f32_via_f64(x, w, b)
    assert np.abs(got - f32).max() <= 0.02 * np.abs(f32).max()


def test_tiny_linear_literals_from_reference_session_test(hip):
    """x, W, b of autograd_cuda/device_session_test.v:34-36; y = [1.41, 3.22] in f32 math."""
    v = KAT["reference_vocabulary"]["linear_f64_session"]
    x, w, b = (np.array(v[k], np.float32) for k in ("x", "w", "b"))
    layer = QuantLinearLayer(w, b, mode=PER_CHANNEL)
    got = layer.forward(x)
    assert got.shape == (1, 2)
    assert np.array_equal(got, _oracle_linear(x, w, b, PER_CHANNEL))
    assert np.allclose(got, np.array(v["out"], np.float32), rtol=0.02)   # int8 resolution
    layer.release()


@pytest.mark.parametrize("m", [1, 8, 32, 128])
def test_decode_linear_config(hip, m):
    """Config 4: K=4096, N=14336, per-output-channel weights, per-token activations."""
    x, w = workloads.decode_linear(m)
    wq, sw = oracle.quantize(w, True, threads=CPU_THREADS)
    W = dev(w)
    Wq, Sw = W.quantize_i8(0)
    assert np.array_equal(Wq.cpu(), wq) and np.array_equal(Sw.cpu(), sw)
    X = dev(x)
    y = linear_f32_dynquant_hip(X, Wq, Sw, None)
    got = y.cpu()
    want = oracle.linear_f32_dynquant(x, wq, sw, None, threads=CPU_THREADS)
    assert got.shape == (m, 14336)
    assert rel_err(got, want) <= F32_REL_TOL and np.array_equal(got, want)
    for h in (W, Wq, Sw, X, y):
        h.release()


# the requantizing linear: tile kernel with and without a K split, ragged tiles, every row-kernel
# size class (N <= 1024 ... 16384), and the shapes that fall back to linear + row quantizer
# (few rows, N % 4 != 0, N > 16384, K % 16 != 0)
REQUANT_SHAPES = [(256, 1024, 4096), (256, 4096, 11008), (256, 11008, 4096), (100, 1200, 1360), (64, 2048, 512),
                  (130, 4100, 640), (200, 8200, 272), (96, 16384, 256), (129, 200, 128),
                  (33, 6000, 256), (40, 16384, 128), (300, 4, 2432), (1000, 512, 64),
                  (8, 2048, 1024), (32, 300, 512), (64, 1002, 256), (40, 16388, 64), (64, 256, 100)]


@pytest.mark.parametrize("wide", ["0", "1"])
@pytest.mark.parametrize("mnk", REQUANT_SHAPES)
def test_requantizing_linear_equals_linear_then_row_quantize(hip, mnk, wide, knobs):
    """vtl_hip_linear_i8_requant gives the codes, scales and (when asked for) f32 rows of
    vtl_hip_linear_i8_f32 followed by the per-row quantizer, and of the oracle.  `wide` picks
    between the two forms of the launch without a K split (VTL_HIP_REQUANT_WIDE: row maxima in
    the tile kernel's epilogue and a wide quantizer, or int32 sums and one workgroup per row)."""
    knobs.setenv("VTL_HIP_REQUANT_WIDE", wide)
    m, n, k = mnk
    rng = np.random.Generator(np.random.Philox(m * 13 + n * 5 + k))
    a = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sa = (rng.uniform(0.5, 1.5, m) * np.exp(rng.uniform(-10, 10, m)) / 127).astype(np.float32)
    sw = (rng.uniform(0.5, 1.5, n) / 127).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    A, W, SA, SW, B = dev(a), dev(w), dev(sa), dev(sw), dev(bias)
    for relu, b_dev, b_host in ((True, B, bias), (False, None, None)):
        q_ref, s_ref, y_ref = oracle.linear_i8_requant(a, sa, w, sw, b_host, relu=relu, threads=CPU_THREADS)
        yq, sy, y = linear_i8_requant_hip(A, SA, W, SW, b_dev, relu=relu, keep_f32=True)
        assert np.array_equal(y.cpu(), y_ref) and np.array_equal(sy.cpu(), s_ref)
        assert np.array_equal(yq.cpu(), q_ref)
        yq2, sy2 = linear_i8_requant_hip(A, SA, W, SW, b_dev, relu=relu)       # no f32 rows wanted
        assert np.array_equal(yq2.cpu(), q_ref) and np.array_equal(sy2.cpu(), s_ref)
        knobs.setenv("VTL_HIP_NO_FUSED_REQUANT", "1")                    # linear, then row quantizer
        yq3, sy3 = linear_i8_requant_hip(A, SA, W, SW, b_dev, relu=relu)
        knobs.delenv("VTL_HIP_NO_FUSED_REQUANT")
        assert np.array_equal(yq3.cpu(), q_ref) and np.array_equal(sy3.cpu(), s_ref)
        for h in (yq, sy, y, yq2, sy2, yq3, sy3):
            h.release()
    # rows that come out all zero (ReLU of a negative row): scale 0, codes 0
    neg = dev(np.full(n, -1e30, np.float32))
    yq, sy = linear_i8_requant_hip(A, SA, W, SW, neg, relu=True)
    assert not yq.cpu().any() and not sy.cpu().any()
    for h in (A, W, SA, SW, B, neg, yq, sy):
        h.release()


def test_mlp_chain_config(hip):
    """Config 5: 256x4096 -> 11008 -> ReLU -> 4096 -> ReLU -> 1024 through Sequential."""
    x, ws = workloads.mlp_chain()
    model = Sequential(mode=PER_CHANNEL).input([4096])
    model.linear(11008, ws[0]).relu().linear(4096, ws[1]).relu().linear(1024, ws[2])
    got = model.forward(x)
    cur = x
    for i, w in enumerate(ws):
        cur = _oracle_linear(cur, w, np.zeros(w.shape[0], np.float32), PER_CHANNEL, relu=i < 2)
    assert got.shape == (256, 1024)
    assert rel_err(got, cur) <= F32_REL_TOL and np.array_equal(got, cur)
    model.release()


@pytest.mark.parametrize("m", [1, 8, 32, 33])
def test_mlp_chain_with_few_tokens(hip, m):
    """Up to 32 tokens Sequential keeps the activations f32 between the layers and every layer
    quantizes its input inside its own launch; from 33 on codes go from layer to layer.  Both
    give the oracle's bits (4096 -> 2048 -> ReLU -> 1024 -> ReLU -> 512)."""
    rng = np.random.Generator(np.random.Philox(600 + m))
    dims = [4096, 2048, 1024, 512]
    ws = [(rng.standard_normal((dims[i + 1], dims[i])) * 0.02).astype(np.float32) for i in range(3)]
    bs = [rng.standard_normal(dims[i + 1]).astype(np.float32) for i in range(3)]
    x = rng.standard_normal((m, dims[0]), dtype=np.float32)
    model = Sequential(mode=PER_CHANNEL).input([dims[0]])
    model.linear(dims[1], ws[0], bs[0]).relu().linear(dims[2], ws[1], bs[1]).relu().linear(dims[3], ws[2], bs[2])
    for _ in range(2):                                   # second pass: cached weights, same route
        got = model.forward(x, no_grad=True)
        cur = x
        for i in range(3):
            cur = _oracle_linear(cur, ws[i], bs[i], PER_CHANNEL, relu=i < 2)
        assert np.array_equal(got, cur)
    model.release()


@pytest.mark.parametrize("mnk", [(2, 2048, 1024), (4, 4100, 2048), (8, 2050, 1024), (16, 3000, 4096), (32, 2048, 2048)])
def test_weight_cache_policy_does_not_change_the_bits(hip, mnk, knobs):
    """The kernels for 2 to 32 rows read large weight matrices with non-temporal loads
    (VTL_HIP_STREAM_WEIGHTS_MIB sets the size; 0: every matrix): same results either way."""
    m, n, k = mnk
    rng = np.random.Generator(np.random.Philox(m + n + k))
    x = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    X, W, SW, B = dev(x), dev(w), dev(sw), dev(bias)
    want = oracle.linear_f32_dynquant(x, w, sw, bias, relu=True, threads=CPU_THREADS)
    for mib in ("0", "1000000"):
        knobs.setenv("VTL_HIP_STREAM_WEIGHTS_MIB", mib)
        for rows_kernel in (None, "1", "0"):
            if rows_kernel is None:
                knobs.delenv("VTL_HIP_GEMV_ROWS", raising=False)
            else:
                knobs.setenv("VTL_HIP_GEMV_ROWS", rows_kernel)
            assert np.array_equal(linear_f32_dynquant_hip(X, W, SW, B, relu=True).cpu(), want), (mib, rows_kernel)
    for h in (X, W, SW, B):
        h.release()


def test_sequential_builder_rules(hip):
    with pytest.raises(ValueError):
        Sequential().linear(4)                       # no input layer yet
    model = Sequential(seed=3).input([48]).linear(32).relu().linear(16)
    assert [l[0] for l in model.layers] == ["input", "linear", "relu", "linear"]
    assert model.layers[1][1].weights.shape == (32, 48) and model.layers[3][1].weights.shape == (16, 32)
    x = np.random.default_rng(0).standard_normal((5, 48)).astype(np.float32)
    got = model.forward(x)
    h = _oracle_linear(x, model.layers[1][1].weights, model.layers[1][1].bias, PER_CHANNEL, relu=True)
    want = _oracle_linear(h, model.layers[3][1].weights, model.layers[3][1].bias, PER_CHANNEL)
    assert np.array_equal(got, want)
    with pytest.raises(ValueError, match="Invalid shapes"):
        model.forward(np.zeros((2, 40), np.float32))
    # a standalone ReLU layer (not preceded by a Linear) runs the ReLU kernel
    m2 = Sequential().input([8]).relu()
    assert np.array_equal(m2.forward(np.array([[-1, 2, -3, 4, 0, -0.5, 7, -8]], np.float32)),
                          np.array([[0, 2, 0, 4, 0, 0, 7, 0]], np.float32))
    model.release()


def test_weight_cache_follows_parameter_replacement(hip):
    rng = np.random.default_rng(1)
    w1 = rng.standard_normal((8, 64)).astype(np.float32)
    w2 = rng.standard_normal((8, 64)).astype(np.float32)
    x = rng.standard_normal((3, 64)).astype(np.float32)
    layer = QuantLinearLayer(w1, requires_grad=False)
    y1 = layer.forward(x)
    first = layer.quantized()
    assert layer.quantized() is first                 # frozen parameter, same object: reused
    layer.weights = w2                                # Adam assigns a new tensor (adam.v:115,136)
    y2 = layer.forward(x)
    assert layer.quantized() is not first
    assert np.array_equal(y1, _oracle_linear(x, w1, None, PER_CHANNEL))
    assert np.array_equal(y2, _oracle_linear(x, w2, None, PER_CHANNEL))
    layer.release()


def test_weight_cache_sees_in_place_optimizer_steps(hip):
    """SGD, AdaGrad, AdamW and RMSProp update `v.value` in place (nn/optimizers/sgd.v:46-53 ->
    nn/internal/optimizers.v:6-12): the tensor object stays the same while its contents change.
    A trainable layer therefore quantizes its parameters on every forward; a frozen one keeps
    them, and still notices an in-place edit through the content fingerprint."""
    rng = np.random.default_rng(7)
    w = rng.standard_normal((8, 64)).astype(np.float32)
    b = rng.standard_normal((1, 8)).astype(np.float32)
    g = rng.standard_normal((8, 64)).astype(np.float32)
    x = rng.standard_normal((3, 64)).astype(np.float32)
    layer = QuantLinearLayer(w, b)                    # requires_grad, like every reference Variable
    y0 = layer.forward(x)
    assert np.array_equal(y0, _oracle_linear(x, w.copy(), b.reshape(-1), PER_CHANNEL))
    for step in range(2):                             # sgd_optimize: value.set(i, val - lr * grad)
        layer.weights -= np.float32(0.1) * g
        layer.bias -= np.float32(0.05)
        assert layer.weights is w and np.shares_memory(layer.bias, b)   # same tensors, new contents
        y = layer.forward(x)
        assert np.array_equal(y, _oracle_linear(x, w.copy(), b.reshape(-1), PER_CHANNEL)), step
    assert layer.quantize_count == 3                  # every training forward re-quantized
    # inference: the copy made under no_grad is kept ...
    n0 = layer.quantize_count
    y_a = layer.forward(x, no_grad=True)
    y_b = layer.forward(x, no_grad=True)
    assert layer.quantize_count == n0 + 1 and np.array_equal(y_a, y_b)
    # ... a training forward in between never trusts it, nor is its own copy trusted afterwards
    layer.forward(x)
    layer.weights += np.float32(0.25) * g
    y_c = layer.forward(x, no_grad=True)
    assert np.array_equal(y_c, _oracle_linear(x, w.copy(), b.reshape(-1), PER_CHANNEL))
    # ... and an in-place edit of frozen parameters (a checkpoint loaded into the same tensors)
    layer.requires_grad = False
    layer.forward(x)
    n1 = layer.quantize_count
    layer.forward(x)
    assert layer.quantize_count == n1
    w[...] = rng.standard_normal((8, 64)).astype(np.float32)
    y_d = layer.forward(x)
    assert layer.quantize_count == n1 + 1
    assert np.array_equal(y_d, _oracle_linear(x, w.copy(), b.reshape(-1), PER_CHANNEL))
    b[...] = 0.5                                      # the bias alone
    y_e = layer.forward(x)
    assert np.array_equal(y_e, _oracle_linear(x, w.copy(), b.reshape(-1), PER_CHANNEL))
    layer.invalidate()
    assert np.array_equal(layer.forward(x), y_e) and layer.quantize_count == n1 + 3
    layer.release()


def test_session_reuses_buffers_on_second_forward(hip):
    """cf. test_device_session_reuses_buffers_on_second_forward,
    autograd_cuda/device_session_test.v:25-48."""
    s = HipSession()
    a = s.ensure("dynquant", 1000)
    assert s.ensure("dynquant", 500) is a and s.ensure("dynquant", 1000) is a
    b = s.ensure("dynquant", 5000)
    assert b is not a and b.size >= 5000
    rng = np.random.default_rng(2)
    layer = QuantLinearLayer(rng.standard_normal((16, 128)).astype(np.float32))
    X = dev(rng.standard_normal((4, 128)).astype(np.float32))
    y1 = layer.forward_device(X, session=s).cpu()
    buf = s.ensure("dynquant", 1)
    y2 = layer.forward_device(X, session=s).cpu()
    assert s.ensure("dynquant", 1) is buf and np.array_equal(y1, y2)
    s.release()
    layer.release()


@pytest.mark.parametrize("mnk", [(2, 2048, 256), (2, 3001, 1008), (2, 2050, 2048), (2, 2048, 4096), (2, 2064, 3088),
                                 (3, 2048, 1024), (4, 4099, 1040), (4, 2048, 2048), (3, 2051, 272),
                                 (5, 2048, 512), (8, 2050, 1024), (7, 9000, 1008), (6, 2048, 16 * 17),
                                 (8, 70001, 256), (2, 1, 256), (3, 7, 2048), (8, 64, 1024), (4, 100, 272),
                                 (2, 1536, 4096),
                                 # 48 MiB of weights and more: the instances with non-temporal weight loads
                                 (2, 14336, 4096), (4, 16400, 3072), (2, 8192, 8192), (7, 12300, 4096)])
def test_few_token_fused_decode_equals_two_launch_path(hip, mnk, knobs):
    """2 to 8 tokens with short rows take the few-token kernel whose workgroups quantize the
    rows themselves (forced here for every size it is built for); it must give the bits of
    the quantize-then-linear path and of the oracle, special values included."""
    m, n, k = mnk
    rng = np.random.Generator(np.random.Philox(m * 7 + n + k))
    x = rng.standard_normal((m, k), dtype=np.float32)
    x[0, :4] = [0.5, 1.5, -2.5, 3.5]
    x[m - 1] *= np.float32(1e-30)            # a row with a tiny scale
    if m > 2:
        x[1] = 0.0                           # an all-zero row: scale 0, codes 0
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    X, W, SW, B = dev(x), dev(w), dev(sw), dev(bias)
    want = oracle.linear_f32_dynquant(x, w, sw, bias, relu=True, threads=CPU_THREADS)
    knobs.setenv("VTL_HIP_GEMV_ROWS", "1")
    fused = linear_f32_dynquant_hip(X, W, SW, B, relu=True).cpu()
    knobs.setenv("VTL_HIP_NO_FUSED_DECODE", "1")
    plain = linear_f32_dynquant_hip(X, W, SW, B, relu=True).cpu()
    knobs.delenv("VTL_HIP_NO_FUSED_DECODE")
    knobs.delenv("VTL_HIP_GEMV_ROWS")
    auto = linear_f32_dynquant_hip(X, W, SW, B, relu=True).cpu()
    assert np.array_equal(fused, want) and np.array_equal(plain, want) and np.array_equal(auto, want)
    knobs.setenv("VTL_HIP_GEMV_ROWS", "1")
    for special in (np.nan, np.inf, -np.inf):
        xs = x.copy()
        xs[0, 7] = special
        xs[m - 1, k - 1] = special
        S = dev(xs)
        got = linear_f32_dynquant_hip(S, W, SW, None, relu=False).cpu()
        ref = oracle.linear_f32_dynquant(xs, w, sw, None)
        assert np.array_equal(got, ref, equal_nan=True), special
        S.release()
    for h in (X, W, SW, B):
        h.release()


@pytest.mark.parametrize("mnk", [(2, 2048, 256), (8, 14336, 4096), (8, 2077, 1280), (9, 3001, 512), (16, 12300, 8192),
                                 (17, 4096, 2048), (31, 2050, 4096), (32, 14336, 4096), (3, 14336, 4096),
                                 # fewer than 2048 weight rows: the four-wave form of the kernel
                                 (12, 512, 1024), (32, 1920, 2048), (5, 128, 4096), (16, 1000, 4096), (8, 300, 2048)])
def test_decode_launch_that_quantizes_its_rows_equals_two_launch_path(hip, mnk, knobs):
    """2 to 32 tokens against thousands of weight rows: one launch whose first workgroups
    quantize the rows while the others wait for them.  Same bits as quantizer + linear and as
    the oracle, special values included; also when no workgroup waits at all (spin limit 0:
    every workgroup quantizes the rows itself) or waits for one poll only, and when the same
    staging buffer is used again for other activations."""
    m, n, k = mnk
    rng = np.random.Generator(np.random.Philox(m * 11 + n + k))
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    W, SW, B = dev(w), dev(sw), dev(bias)
    session = HipSession()
    need = int(capi.lib().vtl_hip_linear_f32_dynquant_workspace(m, k))
    ws = session.ensure("dynquant", need)
    xs = []
    for variant in range(3):
        x = (rng.standard_normal((m, k), dtype=np.float32) * np.float32(variant + 1))
        x[0, :4] = [0.5, 1.5, -2.5, 3.5]
        x[m - 1] *= np.float32(1e-30)            # a row with a tiny scale
        if variant == 1:
            x[m // 2] = 0.0                      # an all-zero row: scale 0, codes 0
        xs.append(x)
    for special in (np.nan, np.inf, -np.inf):
        x = xs[0].copy()
        x[0, 7] = special
        x[m - 1, k - 1] = special
        xs.append(x)
    wants = [oracle.linear_f32_dynquant(x, w, sw, bias, relu=True, threads=CPU_THREADS) for x in xs]
    for spin in (None, "0", "1", "two launches"):
        if spin == "two launches":
            knobs.setenv("VTL_HIP_NO_FUSED_DECODE", "1")
        elif spin is not None:
            knobs.setenv("VTL_HIP_STAGE_SPIN", spin)
        for x, want in zip(xs, wants):           # the same staging buffer, other activations
            X = dev(x)
            got = linear_f32_dynquant_hip(X, W, SW, B, relu=True, workspace=ws).cpu()
            assert np.array_equal(got, want, equal_nan=True), (spin, mnk)
            X.release()
        knobs.delenv("VTL_HIP_STAGE_SPIN", raising=False)
        knobs.delenv("VTL_HIP_NO_FUSED_DECODE", raising=False)
    session.release()
    for h in (W, SW, B):
        h.release()


def test_decode_with_a_staging_buffer_that_starts_inside_a_cache_line(hip):
    """The one-launch form needs the staging buffer to own its cache lines; a buffer that is
    16-byte but not 128-byte aligned gets quantizer + linear, with the same bits, and what lies
    in front of it in the same line is left alone."""
    m, n, k = 8, 4096, 1024
    rng = np.random.Generator(np.random.Philox(80))
    x = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
    X, W, SW = dev(x), dev(w), dev(sw)
    Y = HipTensor.empty([m, n], np.float32)
    need = int(capi.lib().vtl_hip_linear_f32_dynquant_workspace(m, k))
    buf = HipTensor.from_host(np.full(need + 256, 0x5A, np.uint8))
    want = oracle.linear_f32_dynquant(x, w, sw, None)
    for shift in (16, 48, 112, 0):
        capi.call("vtl_hip_linear_f32_dynquant", X.ptr, W.ptr, SW.ptr, None, Y.ptr, m, n, k, 0,
                  C.c_void_p(int(buf.ptr) + shift), need)
        assert np.array_equal(Y.cpu(), want), shift
        host = buf.cpu()
        assert (host[:shift] == 0x5A).all() and (host[shift + need:] == 0x5A).all(), shift
    for t in (X, W, SW, Y, buf):
        t.release()


def test_decode_launch_counters_are_per_stream_and_run_out_gracefully(hip):
    """The workgroups of that launch meet on a counter the library keeps per stream (16 of
    them): calls that alternate between streams, and calls on more streams than there are
    counters (those take the two-launch path), all give the oracle's bits."""
    hiprt = C.CDLL("libamdhip64.so")
    m, n, k = 8, 2048, 512
    rng = np.random.Generator(np.random.Philox(77))
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
    W, SW = dev(w), dev(sw)
    streams = []
    try:
        for i in range(20):
            st = C.c_void_p()
            assert hiprt.hipStreamCreate(C.byref(st)) == 0
            streams.append(st)
        for rnd in range(3):
            for i, st in enumerate(streams):
                x = rng.standard_normal((m, k), dtype=np.float32) * np.float32(i + 1)
                X = dev(x)
                Y = HipTensor.empty([m, n], np.float32)
                capi.call("vtl_hip_set_stream", st)
                capi.call("vtl_hip_linear_f32_dynquant", X.ptr, W.ptr, SW.ptr, None, Y.ptr, m, n, k, 0, None, 0)
                capi.call("vtl_hip_sync")
                assert np.array_equal(Y.cpu(), oracle.linear_f32_dynquant(x, w, sw, None)), (rnd, i)
                X.release()
                Y.release()
    finally:
        capi.call("vtl_hip_set_stream", None)
        for st in streams:
            hiprt.hipStreamDestroy(st)
        W.release()
        SW.release()


def test_decode_launches_on_two_streams_may_overlap(hip):
    """Two streams, a staging buffer and a counter each: calls are enqueued on both without
    waiting in between, so the launches are free to run at the same time, and each must wait
    for its own rows only."""
    hiprt = C.CDLL("libamdhip64.so")
    n, k = 14336, 4096
    rng = np.random.Generator(np.random.Philox(79))
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
    W, SW = dev(w), dev(sw)
    lanes = []
    try:
        for i, m in enumerate((8, 32)):
            st = C.c_void_p()
            assert hiprt.hipStreamCreate(C.byref(st)) == 0
            need = int(capi.lib().vtl_hip_linear_f32_dynquant_workspace(m, k))
            xs = [rng.standard_normal((m, k), dtype=np.float32) * np.float32(j + 1 + 3 * i) for j in range(3)]
            lanes.append({"stream": st, "m": m, "ws": HipTensor.empty([need], np.uint8), "xs": xs,
                          "X": [dev(x) for x in xs], "Y": [HipTensor.empty([m, n], np.float32) for _ in xs],
                          "want": [oracle.linear_f32_dynquant(x, w, sw, None, threads=CPU_THREADS) for x in xs]})
        for rnd in range(4):
            for j in range(3):
                for ln in lanes:                    # alternate between the streams, no waiting
                    capi.call("vtl_hip_set_stream", ln["stream"])
                    capi.call("vtl_hip_linear_f32_dynquant", ln["X"][j].ptr, W.ptr, SW.ptr, None, ln["Y"][j].ptr,
                              ln["m"], n, k, 0, ln["ws"].ptr, ln["ws"].size)
            for ln in lanes:
                capi.call("vtl_hip_set_stream", ln["stream"])
                capi.call("vtl_hip_sync")
            for ln in lanes:
                for j in range(3):
                    assert np.array_equal(ln["Y"][j].cpu(), ln["want"][j]), (rnd, ln["m"], j)
                    capi.call("vtl_hip_memset", ln["Y"][j].ptr, 0, ln["m"] * n * 4)
    finally:
        capi.call("vtl_hip_set_stream", None)
        capi.call("vtl_hip_sync")
        for ln in lanes:
            hiprt.hipStreamDestroy(ln["stream"])
            for t in [ln["ws"], *ln["X"], *ln["Y"]]:
                t.release()
        W.release()
        SW.release()


def test_decode_launch_is_replaced_by_two_launches_under_stream_capture(hip):
    """A graph replays the kernel arguments it recorded, and the launch that quantizes its own
    rows waits for a counter value that is new on every call: under capture the library records
    quantizer + linear instead, and every replay gives the oracle's bits."""
    hiprt = C.CDLL("libamdhip64.so")
    stream, graph, gexec = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert hiprt.hipStreamCreate(C.byref(stream)) == 0
    m, n, k = 16, 4096, 1024
    rng = np.random.Generator(np.random.Philox(78))
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
    x = rng.standard_normal((m, k), dtype=np.float32)
    X, W, SW = dev(x), dev(w), dev(sw)
    Y = HipTensor.empty([m, n], np.float32)

    def call():
        capi.call("vtl_hip_linear_f32_dynquant", X.ptr, W.ptr, SW.ptr, None, Y.ptr, m, n, k, 0, None, 0)

    try:
        capi.call("vtl_hip_set_stream", stream)
        call()                                      # eager: the one-launch form; the staging buffer exists now
        capi.call("vtl_hip_sync")
        assert np.array_equal(Y.cpu(), oracle.linear_f32_dynquant(x, w, sw, None))
        assert hiprt.hipStreamBeginCapture(stream, 0) == 0
        call()
        assert hiprt.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert hiprt.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
        for rep in range(4):
            xr = (rng.standard_normal((m, k)) * (rep + 2)).astype(np.float32)
            capi.call("vtl_hip_memcpy_h2d", X.ptr, xr.ctypes.data, xr.nbytes)
            if rep % 2:
                call()                              # eager calls between the replays, on the same stream
                capi.call("vtl_hip_sync")
                assert np.array_equal(Y.cpu(), oracle.linear_f32_dynquant(xr, w, sw, None)), f"eager {rep}"
                capi.call("vtl_hip_memset", Y.ptr, 0, m * n * 4)
            assert hiprt.hipGraphLaunch(gexec, stream) == 0
            capi.call("vtl_hip_sync")
            assert np.array_equal(Y.cpu(), oracle.linear_f32_dynquant(xr, w, sw, None)), f"replay {rep}"
    finally:
        capi.call("vtl_hip_set_stream", None)
        if gexec:
            hiprt.hipGraphExecDestroy(gexec)
        if graph:
            hiprt.hipGraphDestroy(graph)
        hiprt.hipStreamDestroy(stream)
        for t in (X, W, SW, Y):
            t.release()


@pytest.mark.parametrize("nk", [(2048, 256), (2050, 512), (3001, 4096), (2077, 1280), (1, 16), (7, 48), (300, 784),
                                (14336, 4080), (4097, 5120), (2048, 8192), (1000, 7168), (2050, 8208),
                                (64, 11008), (2050, 9232), (4096, 11008), (300, 11280), (1000, 14336), (70, 14352),
                                # long rows and more weight rows than 64 per wave of the halved grid
                                (131072, 6160), (131073, 6160), (152064, 8192)])
def test_single_token_fused_decode_equals_two_launch_path(hip, nk, knobs):
    """M = 1 takes the matrix-vector kernel that quantizes the token itself (rows of
    up to 14336 codes, any multiple of 16; longer rows take two launches); it must
    give the bits of the quantize-then-linear path and of the oracle."""
    n, k = nk
    rng = np.random.Generator(np.random.Philox(n + k))
    x = rng.standard_normal((1, k), dtype=np.float32)
    x[0, :4] = [0.5, 1.5, -2.5, 3.5]
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    X, W, SW, B = dev(x), dev(w), dev(sw), dev(bias)
    want = oracle.linear_f32_dynquant(x, w, sw, bias, relu=True, threads=CPU_THREADS)
    fused = linear_f32_dynquant_hip(X, W, SW, B, relu=True).cpu()
    knobs.setenv("VTL_HIP_NO_FUSED_DECODE", "1")
    plain = linear_f32_dynquant_hip(X, W, SW, B, relu=True).cpu()
    assert np.array_equal(fused, want) and np.array_equal(plain, want)
    # degenerate token: all zeros -> scale 0 -> output is the bias (ReLU applied)
    Z = dev(np.zeros((1, k), np.float32))
    knobs.delenv("VTL_HIP_NO_FUSED_DECODE")
    got = linear_f32_dynquant_hip(Z, W, SW, B, relu=False).cpu()
    assert np.array_equal(got, oracle.linear_f32_dynquant(np.zeros((1, k), np.float32), w, sw, bias))
    # NaN elements are ignored by the absmax and quantize to 0; an infinite element makes the
    # scale infinite and every code 0 -- the fused kernel follows the same rules
    for special in (np.nan, np.inf, -np.inf):
        xs = x.copy()
        xs[0, 7] = special
        xs[0, k - 1] = special
        S = dev(xs)
        got = linear_f32_dynquant_hip(S, W, SW, B, relu=False).cpu()
        ref = oracle.linear_f32_dynquant(xs, w, sw, bias)
        assert np.array_equal(got, ref, equal_nan=True), special
        S.release()
    for h in (X, W, SW, B, Z):
        h.release()


@pytest.mark.parametrize("mnk", [(8, 2048, 4096), (256, 512, 11008), (37, 300, 1360), (1, 4096, 4096)])
def test_dynquant_without_caller_workspace(hip, mnk):
    """workspace = NULL: the library stages the quantized activations in a buffer of its
    own, separate from the one its split-K launches use."""
    m, n, k = mnk
    rng = np.random.Generator(np.random.Philox(m + n + k))
    x = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = (rng.uniform(0.5, 1.5, n) * 1e-3).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    X, W, SW, B = dev(x), dev(w), dev(sw), dev(bias)
    Y = HipTensor.empty([m, n], np.float32)
    want = oracle.linear_f32_dynquant(x, w, sw, bias, relu=True, threads=CPU_THREADS)
    for _ in range(2):
        capi.call("vtl_hip_linear_f32_dynquant", X.ptr, W.ptr, SW.ptr, B.ptr, Y.ptr, m, n, k, 1, None, 0)
        assert np.array_equal(Y.cpu(), want)
    for h in (X, W, SW, B, Y):
        h.release()
