"""Model-file format of quantized Linear weights (reference format:
nn/models/serialization.v:416-471).  The string format is pinned by a
hand-computed vector; the device round trip is a GPU test."""
import json

import numpy as np
import pytest

from vtl_amd import serialization as ser


def test_tensor_encoding_known_answer():
    # 1.0 = 3FF0000000000000, -2.0 = C000000000000000 (IEEE-754 binary64, big-endian)
    t = np.array([[1.0, -2.0]], np.float32)
    assert ser.encode_tensor(t) == "1,2;row_major|P/AAAAAAAADAAAAAAAAAAA=="
    back = ser.decode_tensor("1,2;row_major|P/AAAAAAAADAAAAAAAAAAA==", [1, 2])
    assert back.dtype == np.float32 and back.tolist() == [[1.0, -2.0]]
    # int8 codes are widened to f64 like every dtype: -127 = C05FC00000000000
    assert ser.encode_tensor(np.array([-127], np.int8)) == "1;row_major|wF/AAAAAAAA="
    assert ser.decode_tensor("1;row_major|wF/AAAAAAAA=", [1], np.int8).tolist() == [-127]


def test_tensor_encoding_round_trip_and_errors():
    rng = np.random.default_rng(0)
    for arr in (rng.standard_normal((3, 5)).astype(np.float32), rng.integers(-127, 128, (4, 7), dtype=np.int8),
                np.zeros((1, 6), np.float32)):
        back = ser.decode_tensor(ser.encode_tensor(arr), arr.shape, arr.dtype)
        assert back.dtype == arr.dtype and np.array_equal(back, arr)
    with pytest.raises(ValueError, match="missing shape delimiter"):
        ser.decode_tensor("1,2;row_major", [1, 2])
    with pytest.raises(ValueError, match="Shape mismatch"):
        ser.decode_tensor(ser.encode_tensor(np.zeros((2, 3), np.float32)), [3, 2])


def test_layer_definitions_known_answer(tmp_path):
    """The LayerDef list a reference Sequential (input -> linear -> relu -> linear) writes:
    nn/models/serialization.v:108-137 with sequential_info.v:43-60 (the input layer is layer 0,
    in_shape empty; then each layer's in_shape is the output shape of the one before)."""
    from vtl_amd import QuantLinearLayer
    l1 = QuantLinearLayer(np.zeros((24, 48), np.float32))
    l2 = QuantLinearLayer(np.zeros((8, 24), np.float32))
    path = str(tmp_path / "defs.json")
    ser.save_model(path, [l1, "relu", l2], [48], with_quantized=False)
    text = open(path).read()
    model = json.loads(text)
    assert model["layers"] == [
        {"layer_type": "InputLayer", "in_shape": [], "config": {"shape_0": 48}},
        {"layer_type": "LinearLayer", "in_shape": [48], "config": {"in_features": 48, "out_features": 24}},
        {"layer_type": "ReLULayer", "in_shape": [24], "config": {}},
        {"layer_type": "LinearLayer", "in_shape": [24], "config": {"in_features": 24, "out_features": 8}}]
    assert [list(d["weights"]) for d in model["layer_data"]] == [[], ["weight", "bias"], [], ["weight", "bias"]]
    # key order of the Linear config as the reference inserts it
    assert text.index('"in_features"') < text.index('"out_features"')


@pytest.mark.gpu
def test_model_file_round_trip_with_quantized_weights(hip, tmp_path):
    import oracle
    from vtl_amd import PER_CHANNEL, QuantLinearLayer
    rng = np.random.default_rng(1)
    l1 = QuantLinearLayer(rng.standard_normal((24, 48)).astype(np.float32) * 0.1, rng.standard_normal((1, 24)).astype(np.float32))
    l2 = QuantLinearLayer(rng.standard_normal((8, 24)).astype(np.float32) * 0.1)
    path = str(tmp_path / "model.json")
    ser.save_model(path, [l1, "relu", l2], [48], epoch=3, loss=0.25)
    model = json.load(open(path))
    assert model["version"] == "1.0" and [d["layer_type"] for d in model["layers"]] == ["InputLayer", "LinearLayer", "ReLULayer", "LinearLayer"]
    assert model["layers"][0]["in_shape"] == [] and model["layers"][1]["in_shape"] == [48]
    assert model["layers"][1]["config"] == {"out_features": 24, "in_features": 48}
    assert set(model["layer_data"][1]["weights"]) == {"weight", "bias", "weight_q", "weight_scale"}
    loaded = ser.load_linear_layers(path, PER_CHANNEL)
    assert len(loaded) == 2
    x = rng.standard_normal((5, 48)).astype(np.float32)
    for (layer, stored), orig in zip(loaded, (l1, l2)):
        assert np.array_equal(layer.weights, orig.weights) and np.array_equal(layer.bias, orig.bias)
        codes, scales = stored
        qr, sr = oracle.quantize(orig.weights, True)
        assert np.array_equal(codes, qr) and np.array_equal(scales, sr)      # stored codes = oracle codes
        fresh = layer.quantized()
        assert np.array_equal(fresh.w_q.cpu(), codes) and np.array_equal(fresh.sw.cpu(), scales)
    h = loaded[0][0].forward(x)
    assert np.array_equal(h, l1.forward(x))
    # a file written without the extra keys is an ordinary reference model file
    ser.save_model(path, [l1], [48], with_quantized=False)
    assert set(json.load(open(path))["layer_data"][1]["weights"]) == {"weight", "bias"}
    assert ser.load_linear_layers(path)[0][1] is None
    for l in (l1, l2, loaded[0][0], loaded[1][0]):
        l.release()
