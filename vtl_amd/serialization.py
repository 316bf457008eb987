"""Model-file serialization of quantized Linear weights, in the reference's format.

The reference stores a model as JSON `ModelFile{version, layers[], layer_data[],
optimizer, metadata}` (nn/models/serialization.v:11-63); a LinearLayer has the
config keys `in_features` / `out_features` and the weight keys `weight` /
`bias` (serialization.v:128-137, 307-310), and every tensor is the string
    "d0,d1;row_major|base64(big-endian f64 per element)"
(encode_tensor / decode_tensor, serialization.v:416-471) - every dtype is
widened to f64, which is lossless for f32 values and for int8 codes.

This module adds two keys to a LinearLayer's weight map, `weight_q` (the int8
codes) and `weight_scale` (the f32 scales), next to the unchanged `weight` and
`bias`; a file without them is an ordinary reference model file, and a reader
that does not know them ignores them.
"""
from __future__ import annotations

import base64
import json

import numpy as np

from .layers import PER_CHANNEL, QuantLinearLayer

MODEL_VERSION = "1.0"   # serialization.v:11


def encode_tensor(t: np.ndarray) -> str:
    """`encode_tensor` (serialization.v:416-435): shape, memory order, f64 big-endian base64."""
    a = np.ascontiguousarray(t)
    shape_str = ",".join(str(int(d)) for d in a.shape)
    payload = a.astype(">f8").tobytes()
    return f"{shape_str};row_major|{base64.b64encode(payload).decode('ascii')}"


def decode_tensor(encoded: str, shape, dtype=np.float32) -> np.ndarray:
    """`decode_tensor` (serialization.v:438-471), with its two error cases."""
    parts = encoded.split("|")
    if len(parts) != 2:
        raise ValueError("Invalid tensor encoding: missing shape delimiter")
    head = parts[0].split(";")
    decoded_shape = [int(v) for v in head[0].split(",")] if head[0] else []
    if list(decoded_shape) != [int(d) for d in shape]:
        raise ValueError(f"Shape mismatch: encoded {decoded_shape}, expected {list(shape)}")
    raw = base64.b64decode(parts[1])
    vals = np.frombuffer(raw[: len(raw) // 8 * 8], dtype=">f8")
    arr = vals.astype(dtype).reshape(decoded_shape)
    if len(head) > 1 and head[1] == "col_major":
        arr = np.asfortranarray(arr)
    return arr


def linear_layer_entry(layer: QuantLinearLayer, in_shape, with_quantized: bool = True):
    """(LayerDef, SerializedLayer) dictionaries of one Linear layer."""
    out_f, in_f = layer.weights.shape
    layer_def = {"layer_type": "LinearLayer", "in_shape": [int(d) for d in in_shape],
                 "config": {"in_features": int(in_f), "out_features": int(out_f)}}
    weights = {"weight": encode_tensor(layer.weights), "bias": encode_tensor(layer.bias)}
    if with_quantized:
        qw = layer.quantized()                      # device-resident codes and scales
        weights["weight_q"] = encode_tensor(qw.w_q.cpu())
        weights["weight_scale"] = encode_tensor(qw.sw.cpu())
    return layer_def, {"weights": weights}


def save_model(path: str, layers, input_shape, with_quantized: bool = True, epoch: int = 0,
               loss: float = 0.0) -> None:
    """Write a model file for a stack of QuantLinearLayer / "relu" entries behind
    an input layer of `input_shape`, as Sequential.save_checkpoint does
    (nn/models/serialization.v:108-124): the input layer is layer 0 with an empty
    in_shape and its dimensions in the config (sequential_info.v:43-49), every
    later layer records the output shape of the layer before it."""
    shape = [int(d) for d in input_shape]
    defs = [{"layer_type": "InputLayer", "in_shape": [], "config": {f"shape_{i}": d for i, d in enumerate(shape)}}]
    data = [{"weights": {}}]
    for l in layers:
        if isinstance(l, QuantLinearLayer):
            d, w = linear_layer_entry(l, shape, with_quantized)
            shape = l.output_shape()
        elif l == "relu":
            d, w = {"layer_type": "ReLULayer", "in_shape": shape, "config": {}}, {"weights": {}}
        else:
            raise ValueError(f"unsupported layer {l!r}")
        defs.append(d)
        data.append(w)
    model = {"version": MODEL_VERSION, "layers": defs, "layer_data": data,
             "optimizer": {"optimizer_type": "", "learning_rate": 0.0, "config": {}, "moments": {}},
             "metadata": {"epoch": int(epoch), "loss": float(loss), "saved_at": "", "version": MODEL_VERSION}}
    with open(path, "w") as f:
        json.dump(model, f)


def load_linear_layers(path: str, mode: str = PER_CHANNEL):
    """Read the Linear layers of a model file.  Returns a list of
    (QuantLinearLayer, stored) where `stored` is None or the (codes, scales) pair
    found in the file, so a caller can check them against a fresh quantization."""
    with open(path) as f:
        model = json.load(f)
    if model.get("version") != MODEL_VERSION:
        raise ValueError(f"unsupported model version {model.get('version')!r}")
    out = []
    for d, w in zip(model["layers"], model["layer_data"]):
        if d["layer_type"] != "LinearLayer":
            continue
        out_f, in_f = d["config"]["out_features"], d["config"]["in_features"]
        ws = w["weights"]
        weight = decode_tensor(ws["weight"], [out_f, in_f], np.float32)
        bias = decode_tensor(ws["bias"], [1, out_f], np.float32)
        stored = None
        if "weight_q" in ws and "weight_scale" in ws:
            n_scales = out_f if mode == PER_CHANNEL else 1
            stored = (decode_tensor(ws["weight_q"], [out_f, in_f], np.int8),
                      decode_tensor(ws["weight_scale"], [n_scales], np.float32))
        out.append((QuantLinearLayer(weight, bias, mode), stored))
    return out
