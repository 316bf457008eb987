"""Linear layer on the INT8 HIP path: the Python mirror of the V files
`nn/layers/hip_config.v`, `linear_hip_hooks_d_hip.v` and `linear_hip_d_hip.v`.

The reference's f32 Linear is `y = x.W^T + b` with W stored
`[out_features, in_features]` and bias `[1, out_features]`
(nn/layers/linear.v:10-33); its backend hook is
`linear_forward_f32` (nn/layers/linear_forward_f32.v:7-14), which asks
`linear_forward_f32_use_<backend>()` and tries the device path.  This module
adds the HIP branch of that hook.  The device path returns host tensors, like
every GPU path of the reference (docs/DEVICE_MEMORY.md:9-16), unless the
caller chains layers on the device explicitly (`forward_device`).

There is no CPU arithmetic in here: a failing device call raises
`capi.VtlHipError`.  (In V the hook site keeps the reference's own
`or { return linear_forward_f32_cpu(...) }`, which is VTL's code, not this
library's.)
"""
from __future__ import annotations

import os

import numpy as np

from . import capi
from .storage import HipParams, HipStorage
from .tensor import (HipTensor, linear_backward_hip, linear_f32_dynquant_hip, linear_hip, linear_i8_hip,
                     matmul_hip)


# -- nn/layers/hip_config.v (cf. vulkan_config.v:12-24, cuda_config.v:11-23) ----

def hip_linear_enabled() -> bool:
    """True when the user opts in with VTL_USE_HIP=1 (and the build has `-d hip`)."""
    return os.environ.get("VTL_USE_HIP") == "1"


def hip_tests_enabled() -> bool:
    """Gate for device tests, VTL_TEST_HIP=1 (cf. vulkan_tests_enabled)."""
    return os.environ.get("VTL_TEST_HIP") == "1"


def linear_forward_f32_use_hip() -> bool:
    """Hook consulted by linear_forward_f32 (cf. linear_vulkan_hooks_d_vulkan.v:9)."""
    return hip_linear_enabled()


# -- quantization granularity ------------------------------------------------------

PER_TENSOR = "per_tensor"      # one scale for x, one for W
PER_CHANNEL = "per_channel"    # one scale per row of x (token) and per row of W (output channel)


def hip_backward_enabled() -> bool:
    """Linear gate gradients on the device: VTL_USE_HIP=1 and VTL_HIP_BACKWARD=1
    (cf. cuda_backward_enabled, autograd_cuda/gpu_config.v:20-23)."""
    return os.environ.get("VTL_USE_HIP") == "1" and os.environ.get("VTL_HIP_BACKWARD") == "1"


def linear_gate_use_hip_backward() -> bool:
    """Hook asked by LinearGate.backward (cf. linear_gate_use_vulkan_backward,
    nn/gates/layers/linear_gate_vulkan_hooks_d_vulkan.v:6-8)."""
    return hip_backward_enabled() and capi.device_count() > 0


class HipSession:
    """Reusable device buffers for one Context, cf. DeviceSession
    (autograd_cuda/device_session.v:13-24) and GpuDevBuf.ensure
    (autograd_cuda/device_session_gpu_d_cuda.v:24-39): a buffer grows when a
    larger request arrives and is otherwise reused."""

    def __init__(self, params: HipParams | None = None):
        self.params = params or HipParams()
        self._bufs: dict[str, HipStorage] = {}

    def ensure(self, name: str, nbytes: int) -> HipStorage:
        cur = self._bufs.get(name)
        if cur is not None and cur.size >= nbytes:
            return cur
        if cur is not None:
            cur.release()
        buf = HipStorage.empty(max(int(nbytes), 256), np.uint8, self.params)
        self._bufs[name] = buf
        return buf

    def release(self) -> None:
        for b in self._bufs.values():
            b.release()
        self._bufs.clear()


def content_fingerprint(t: np.ndarray) -> int:
    """Cheap fingerprint of a parameter tensor's contents: FNV-1a over the bit patterns of
    up to 64 elements at even strides plus the last one, and the element count.  It is
    the second line of defence of the weight cache (the first is the frozen rule of
    QuantLinearLayer.quantized): an in-place edit of a frozen parameter - a checkpoint
    loaded into the same tensor, a manual `set` - changes it with near certainty when
    the edit touches most elements, as every optimizer step and every load does."""
    flat = np.ascontiguousarray(t).reshape(-1).view(np.uint32 if t.dtype.itemsize == 4 else np.uint64)
    n = flat.size
    h = 0xcbf29ce484222325 ^ n
    if n:
        step = max(1, n // 64)
        for v in list(flat[::step][:64]) + [flat[n - 1]]:
            h = ((h ^ int(v)) * 0x100000001b3) & 0xffffffffffffffff
    return h


class QuantizedWeights:
    """Device-resident int8 weights of one Linear layer, derived from the f32
    parameter.  `source` / `bias_source` are the host tensors the device copies
    were made from, `fingerprint` / `bias_fingerprint` their content fingerprints at
    that moment and `frozen` whether the parameters were frozen then (see
    QuantLinearLayer.quantized for the rule that decides re-use)."""

    def __init__(self, weights: np.ndarray, bias: np.ndarray | None, mode: str,
                 params: HipParams | None = None, frozen: bool = False):
        if weights.ndim != 2:
            raise ValueError("Matrix expected")
        if mode not in (PER_TENSOR, PER_CHANNEL):
            raise ValueError(f"unknown quantization mode {mode!r}")
        self.mode = mode
        self.source = weights
        self.bias_source = bias
        self.frozen = frozen
        self.fingerprint = content_fingerprint(weights)
        self.bias_fingerprint = None if bias is None else content_fingerprint(np.asarray(bias))
        self.out_features, self.in_features = weights.shape
        w_dev = HipTensor.from_host(np.asarray(weights, np.float32), params)
        try:
            self.w_q, self.sw = w_dev.quantize_i8(0 if mode == PER_CHANNEL else -1)
        finally:
            w_dev.release()
        self.bias = None
        if bias is not None:
            b = np.asarray(bias, np.float32).reshape(-1)
            if b.size != self.out_features:
                raise ValueError(f"bias has {b.size} entries, expected {self.out_features}")
            self.bias = HipTensor.from_host(b, params)

    def release(self) -> None:
        self.w_q.release()
        self.sw.release()
        if self.bias is not None:
            self.bias.release()


def linear_forward_hip_i8_device(x: HipTensor, qw: QuantizedWeights, relu: bool = False,
                                 session: HipSession | None = None) -> HipTensor:
    """x[M,K] f32 on the device -> y[M,N] f32 on the device."""
    if not x.is_matrix():
        raise ValueError("Matrix expected")
    if x.shape[1] != qw.in_features:
        raise ValueError(
            f"Invalid shapes for matrix multiplication {x.shape} and {[qw.in_features, qw.out_features]}")
    if qw.mode == PER_CHANNEL:
        ws = None
        if session is not None:
            need = int(capi.lib().vtl_hip_linear_f32_dynquant_workspace(x.shape[0], x.shape[1]))
            ws = session.ensure("dynquant", need)
        return linear_f32_dynquant_hip(x, qw.w_q, qw.sw, qw.bias, relu=relu, workspace=ws)
    x_q, sx = x.quantize_i8(-1)
    try:
        return linear_i8_hip(x_q, sx, qw.w_q, qw.sw, qw.bias, relu=relu)
    finally:
        capi.call("vtl_hip_sync")
        x_q.release()
        sx.release()


def linear_forward_hip_f32(x: np.ndarray, weights: np.ndarray, bias: np.ndarray | None,
                           mode: str = PER_CHANNEL) -> np.ndarray:
    """`linear_forward_hip_f32(x, weights, bias) !&vtl.Tensor[f32]`: the HIP entry
    of the f32 hook (cf. linear_forward_vulkan_f32, linear_vulkan_d_vulkan.v:7-12).
    Uploads, quantizes both operands, runs the int8 linear, returns a host tensor."""
    if not hip_linear_enabled():
        raise RuntimeError("linear_forward_hip_f32: set VTL_USE_HIP=1 to enable")
    return _linear_host_roundtrip(x, weights, bias, mode)


def _linear_host_roundtrip(x, weights, bias, mode) -> np.ndarray:
    x = np.asarray(x, np.float32)
    if x.ndim != 2 or np.ndim(weights) != 2:
        raise ValueError("Matrix expected")
    qw = QuantizedWeights(weights, bias, mode)
    x_dev = HipTensor.from_host(x)
    try:
        y = linear_forward_hip_i8_device(x_dev, qw)
        try:
            return y.cpu()
        finally:
            y.release()
    finally:
        x_dev.release()
        qw.release()


class QuantLinearLayer:
    """`LinearLayer[f32]` (nn/layers/linear.v:17-74) whose forward runs on the
    INT8 HIP path.  Parameters stay on the host as f32 (as in the reference);
    the int8 copy on the device is derived state.

    `requires_grad` mirrors the flag of the layer's weight Variable
    (autograd/variable.v:64, default true): while it is set an optimizer may
    change the parameters between any two forwards, and most of the reference's
    optimizers do so IN PLACE (SGD: nn/optimizers/sgd.v:46-53 ->
    nn/internal/optimizers.v:6-12 `value.set`; likewise adagrad.v:60, adamw.v:95,
    rmsprop.v:81), only Adam assigns a new tensor (adam.v:115,136).  So the
    tensor's identity says nothing about its contents, and a trainable layer
    uploads and quantizes its parameters on every forward, as the reference's
    own device chain uploads them on every forward
    (autograd_cuda/device_session_gpu_d_cuda.v:107).  The codes are kept from
    one forward to the next only for frozen parameters (requires_grad false, or
    a forward under no_grad)."""

    def __init__(self, weights: np.ndarray, bias: np.ndarray | None = None, mode: str = PER_CHANNEL,
                 params: HipParams | None = None, requires_grad: bool = True):
        weights = np.asarray(weights, np.float32)
        if weights.ndim != 2:
            raise ValueError("Matrix expected")
        self.weights = weights                                   # [out, in]
        self.bias = (np.zeros((1, weights.shape[0]), np.float32) if bias is None
                     else np.asarray(bias, np.float32).reshape(1, -1))  # [1, out]
        self.mode = mode
        self.params = params or HipParams()
        self.requires_grad = requires_grad
        self.quantize_count = 0      # how often the parameters were uploaded and quantized (tests)
        self._cache: QuantizedWeights | None = None

    def output_shape(self):
        return [self.weights.shape[0]]

    def variables(self):
        return [self.weights, self.bias]

    def invalidate(self) -> None:
        """Drops the device copy: the next forward uploads and quantizes again.  For
        callers that edit a frozen parameter in place."""
        if self._cache is not None:
            self._cache.release()
            self._cache = None

    def quantized(self, no_grad: bool = False) -> QuantizedWeights:
        """The layer's int8 weights for one forward.  Re-used from the previous forward only
        when ALL of these hold: the parameters are frozen now (`requires_grad` false, or this
        forward runs under `no_grad`) and were frozen when the copy was made, `weights` and
        `bias` are still the same tensor objects, and their content fingerprints have not
        changed.  Otherwise the parameters are uploaded and quantized again."""
        frozen = no_grad or not self.requires_grad
        c = self._cache
        fresh = (c is not None and frozen and c.frozen and c.source is self.weights
                 and c.bias_source is self.bias and c.fingerprint == content_fingerprint(self.weights)
                 and c.bias_fingerprint == content_fingerprint(self.bias))
        if not fresh:
            if c is not None:
                c.release()
            self._cache = QuantizedWeights(self.weights, self.bias, self.mode, self.params, frozen=frozen)
            self.quantize_count += 1
        return self._cache

    def forward_device(self, x: HipTensor, relu: bool = False,
                       session: HipSession | None = None, no_grad: bool = False) -> HipTensor:
        return linear_forward_hip_i8_device(x, self.quantized(no_grad), relu=relu, session=session)

    def forward(self, x: np.ndarray, no_grad: bool = False) -> np.ndarray:
        x = np.asarray(x, np.float32)
        if x.ndim != 2:
            raise ValueError("Matrix expected")
        x_dev = HipTensor.from_host(x, self.params)
        try:
            y = self.forward_device(x_dev, no_grad=no_grad)
            try:
                return y.cpu()
            finally:
                y.release()
        finally:
            x_dev.release()

    def release(self) -> None:
        if self._cache is not None:
            self._cache.release()
            self._cache = None


def kaiming_normal(shape, rng: np.random.Generator) -> np.ndarray:
    """Weight initialiser of linear_layer (nn/layers/linear.v:25, nn/internal/init.v:21-70):
    N(0, sqrt(2 / fan_in)) where compute_fans multiplies both fans by shape[1]."""
    f0 = shape[0] * int(np.prod(shape[1:]))
    std = np.sqrt(2.0 / f0)
    return (rng.standard_normal(shape) * std).astype(np.float32)


# -- la.matmul / Linear forward and backward in full precision -----------------

def _as_float_matrix(t, what: str) -> np.ndarray:
    a = np.asarray(t)
    if a.dtype not in (np.float32, np.float64):
        raise TypeError(f"{what}: f32 or f64 tensor expected, got {a.dtype}")
    if a.ndim != 2:
        raise ValueError("Matrix expected")
    return a


def matmul_hip_host(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """`la.matmul[T](a, b)` (la/la.v:38-55) through the device: upload both
    operands, f64-accumulating matmul, download.  Shape errors carry the
    reference's message."""
    a = _as_float_matrix(a, "matmul")
    b = _as_float_matrix(b, "matmul")
    if a.shape[1] != b.shape[0]:
        raise ValueError(f"Invalid shapes for matrix multiplication {list(a.shape)} and {list(b.shape)}")
    a_dev = HipTensor.from_host(a)
    b_dev = HipTensor.from_host(b.astype(a.dtype, copy=False))
    try:
        c_dev = matmul_hip(a_dev, b_dev)
        try:
            return c_dev.cpu()
        finally:
            c_dev.release()
    finally:
        a_dev.release()
        b_dev.release()


def linear_forward_hip_exact(x: np.ndarray, weights: np.ndarray, bias: np.ndarray | None) -> np.ndarray:
    """The unquantized Linear forward on the device with the arithmetic of
    linear_forward_f32_cpu (nn/layers/linear_forward_f32.v:16-18): matmul(x, W^T)
    through f64, then the bias added in the tensor's type."""
    x = _as_float_matrix(x, "linear")
    w = _as_float_matrix(weights, "linear").astype(x.dtype, copy=False)
    x_dev, w_dev = HipTensor.from_host(x), HipTensor.from_host(w)
    b_dev = None if bias is None else HipTensor.from_host(np.asarray(bias, x.dtype).reshape(1, -1))
    try:
        y_dev = linear_hip(x_dev, w_dev, b_dev)
        try:
            return y_dev.cpu()
        finally:
            y_dev.release()
    finally:
        for t in (x_dev, w_dev, b_dev):
            if t is not None:
                t.release()


def linear_backward_hip_f32(grad: np.ndarray, input: np.ndarray, weight: np.ndarray,
                            bias_needs_grad: bool):
    """`linear_backward_hip_f32(grad, input, weight, bias_needs_grad) ![]&vtl.Tensor[f32]`:
    [d_input, d_weight, d_bias] of a Linear layer, the HIP counterpart of
    linear_backward_vulkan_f32 (nn/internal/linear_vulkan_backward_d_vulkan.v:9-38)
    and linear_backward_f64 (autograd_cuda/linear_backward_cuda_d_cuda.v:9-36).
    d_bias is [1, out_features]: the column sums of grad, or zeros when the bias
    needs no gradient.  Works for f32 and f64 host tensors alike."""
    if not hip_backward_enabled():
        raise RuntimeError("linear_backward_hip_f32: set VTL_USE_HIP=1 and VTL_HIP_BACKWARD=1")
    g = _as_float_matrix(grad, "linear backward")
    x = _as_float_matrix(input, "linear backward").astype(g.dtype, copy=False)
    w = _as_float_matrix(weight, "linear backward").astype(g.dtype, copy=False)
    g_dev, x_dev, w_dev = HipTensor.from_host(g), HipTensor.from_host(x), HipTensor.from_host(w)
    outs = []
    try:
        outs = linear_backward_hip(g_dev, x_dev, w_dev, need_db=bias_needs_grad)
        d_in, d_w = outs[0].cpu(), outs[1].cpu()
        d_b = outs[2].cpu() if bias_needs_grad else np.zeros((1, w.shape[0]), g.dtype)
        return [d_in, d_w, d_b]
    finally:
        for t in (g_dev, x_dev, w_dev, *outs):
            if t is not None:
                t.release()


# -- activation hooks (cf. relu_forward_f32 / sigmoid_forward_f32,
#    nn/layers/activation_forward_f32.v:7-24, and their Vulkan bodies
#    nn/layers/activation_vulkan_d_vulkan.v:16-29) ---------------------------------

def _activation_host_roundtrip(x, op: str) -> np.ndarray:
    a = np.asarray(x)
    if a.dtype not in (np.float32, np.float64):
        raise TypeError(f"{op}: f32 or f64 tensor expected, got {a.dtype}")
    if a.size == 0:
        return a.copy()
    t = HipTensor.from_host(a)
    try:
        if op == "relu":
            return t.relu_().cpu()
        out = t.sigmoid_hip()
        try:
            return out.cpu()
        finally:
            out.release()
    finally:
        t.release()


def relu_forward_hip_f32(x: np.ndarray) -> np.ndarray:
    """`relu_forward_hip_f32(x) !&vtl.Tensor[f32]`: ReLU through the device (x < 0 -> 0,
    nn/internal/activation.v:63-70); the HIP body of relu_forward_f32's device branch."""
    if not hip_linear_enabled():
        raise RuntimeError("relu_forward_hip_f32: set VTL_USE_HIP=1 to enable")
    return _activation_host_roundtrip(x, "relu")


def sigmoid_forward_hip_f32(x: np.ndarray) -> np.ndarray:
    """`sigmoid_forward_hip_f32(x) !&vtl.Tensor[f32]`: 1 / (1 + exp(-x)) through the device
    with the arithmetic of nn/internal/activation.v:35-40."""
    if not hip_linear_enabled():
        raise RuntimeError("sigmoid_forward_hip_f32: set VTL_USE_HIP=1 to enable")
    return _activation_host_roundtrip(x, "sigmoid")


def matmul_gate_backward_hip(grad: np.ndarray, a: np.ndarray, b: np.ndarray):
    """`MatMulGate.backward` (autograd/gates_blas.v:43-48) through the device:
    [grad . b^T, a^T . grad], the transposes taken by flag instead of `.t()` copies."""
    if not hip_backward_enabled():
        raise RuntimeError("matmul_gate_backward_hip: set VTL_USE_HIP=1 and VTL_HIP_BACKWARD=1")
    g = _as_float_matrix(grad, "matmul backward")
    av = _as_float_matrix(a, "matmul backward").astype(g.dtype, copy=False)
    bv = _as_float_matrix(b, "matmul backward").astype(g.dtype, copy=False)
    if av.shape[1] != bv.shape[0] or g.shape != (av.shape[0], bv.shape[1]):
        raise ValueError(f"Invalid shapes for matrix multiplication {list(av.shape)} and {list(bv.shape)}")
    g_dev, a_dev, b_dev = HipTensor.from_host(g), HipTensor.from_host(av), HipTensor.from_host(bv)
    outs = []
    try:
        outs.append(matmul_hip(g_dev, b_dev, False, True))    # [M,N] . [K,N]^T -> [M,K]
        outs.append(matmul_hip(a_dev, g_dev, True, False))    # [M,K]^T . [M,N] -> [K,N]
        return [t.cpu() for t in outs]
    finally:
        for t in (g_dev, a_dev, b_dev, *outs):
            t.release()
