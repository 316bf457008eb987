"""`Sequential` builder restricted to what the INT8 path needs: the Python
mirror of nn/models/sequential.v:52-220 for input / linear / relu / forward.

`linear(n)` takes its input width from the previous layer
(nn/models/sequential_info.v:53-60); `forward` loops over the layers
(sequential.v:204-215).  Between Linear layers the activations stay on the
device, as per-token int8 codes when the next layer is a Linear again (as f32
rows for up to FEW_TOKENS rows), and ReLU
is folded into the producing Linear's epilogue, in the spirit
of the reference's GPU activation chain
(autograd_cuda/device_session_gpu_d_cuda.v:88-181).
"""
from __future__ import annotations

import numpy as np

from .layers import PER_CHANNEL, HipSession, QuantLinearLayer, kaiming_normal
from .storage import HipParams
from .tensor import HipTensor, linear_i8_hip, linear_i8_requant_hip


# Rows up to which the library's linear on f32 rows quantizes them inside its own launch.
FEW_TOKENS = 32


class Sequential:
    def __init__(self, mode: str = PER_CHANNEL, seed: int = 0, params: HipParams | None = None):
        self.mode = mode
        self.params = params or HipParams()
        self.rng = np.random.Generator(np.random.Philox(seed))
        self.layers: list = []          # ("input", [k]) | ("linear", layer) | ("relu",)
        self._width: int | None = None
        self.session = HipSession(self.params)

    def input(self, shape) -> "Sequential":
        if len(shape) != 1:
            raise ValueError("only flat inputs reach a Linear layer")
        self._width = int(shape[0])
        self.layers.append(("input", list(shape)))
        return self

    def linear(self, output_size: int, weights: np.ndarray | None = None,
               bias: np.ndarray | None = None) -> "Sequential":
        if self._width is None:
            raise ValueError("Sequential.linear: add an input layer first")
        if weights is None:
            weights = kaiming_normal([output_size, self._width], self.rng)
        weights = np.asarray(weights, np.float32)
        if list(weights.shape) != [output_size, self._width]:
            raise ValueError(f"weights {list(weights.shape)}, expected {[output_size, self._width]}")
        self.layers.append(("linear", QuantLinearLayer(weights, bias, self.mode, self.params)))
        self._width = output_size
        return self

    def relu(self) -> "Sequential":
        self.layers.append(("relu",))
        return self

    def forward(self, x: np.ndarray, no_grad: bool = False) -> np.ndarray:
        """`no_grad` is the Context's flag (autograd/context.v:19-21): under it the layers'
        quantized weights are kept from one forward to the next, otherwise every trainable
        layer uploads and quantizes its parameters again (QuantLinearLayer.quantized)."""
        x = np.asarray(x, np.float32)
        if x.ndim != 2:
            raise ValueError("Matrix expected")
        cur = HipTensor.from_host(x, self.params)   # f32 activations, or None while they exist as codes
        cur_q = None                                # (codes, row scales) between two int8 layers
        try:
            i, n = 0, len(self.layers)
            while i < n:
                kind = self.layers[i][0]
                if kind == "linear":
                    layer = self.layers[i][1]
                    fuse = i + 1 < n and self.layers[i + 1][0] == "relu"
                    j = i + (2 if fuse else 1)
                    # Up to FEW_TOKENS rows every layer quantizes its input inside its own launch
                    # (one launch a layer; 1 token through 4096 -> 11008 -> 4096 -> 1024: 23.4
                    # against 28.0 us), so the activations stay f32 between the layers; with more
                    # rows the codes go from layer to layer.  The bits are the same either way.
                    feeds_linear = (self.mode == PER_CHANNEL and j < n and self.layers[j][0] == "linear"
                                    and x.shape[0] > FEW_TOKENS)
                    if cur_q is None and not feeds_linear:
                        nxt = layer.forward_device(cur, relu=fuse, session=self.session, no_grad=no_grad)
                        cur.release()
                        cur = nxt
                    else:
                        # per-token codes go from layer to layer; the f32 rows in between are
                        # never written (same bits as quantizing them in a pass of its own)
                        if cur_q is None:
                            cur_q = cur.quantize_i8(0)
                            cur.release()
                            cur = None
                        qw = layer.quantized(no_grad)
                        if feeds_linear:
                            nxt_q = linear_i8_requant_hip(cur_q[0], cur_q[1], qw.w_q, qw.sw, qw.bias, relu=fuse)
                        else:
                            cur = linear_i8_hip(cur_q[0], cur_q[1], qw.w_q, qw.sw, qw.bias, relu=fuse)
                            nxt_q = None
                        for t in cur_q:
                            t.release()
                        cur_q = nxt_q
                    i = j
                elif kind == "relu":
                    cur.relu_()
                    i += 1
                else:
                    i += 1
            return cur.cpu()
        finally:
            if cur is not None:
                cur.release()
            if cur_q is not None:
                for t in cur_q:
                    t.release()

    def release(self) -> None:
        for l in self.layers:
            if l[0] == "linear":
                l[1].release()
        self.session.release()
