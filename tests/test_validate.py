"""The converted-JSON checker: files from the package's writers come out clean, and each kind of damage an exporter bug
or a hand edit can do is reported in words that name the layer (all findings at once, not only the first)."""
import copy
import importlib
import json

import numpy as np
import pytest


@pytest.fixture(scope="module")
def validate():
    return importlib.import_module("frugally-deep_amd.validate")


def generated_models(modelgen):
    yield "small_cnn", modelgen.small_cnn()
    yield "resnet", modelgen.resnet50(input_size=32, width=8, blocks=(1, 1, 1, 1), classes=10, random_bn=True)
    yield "mobilenet", modelgen.mobilenet_v2(input_size=32, alpha=0.25, classes=10, truncate=4)
    yield "encoder", modelgen.encoder(layers=1, seq=8, d_model=16, heads=2, ffn=32)
    yield "gpt2", modelgen.gpt2(layers=1, d_model=16, heads=2, vocab=50, max_pos=16)
    b = modelgen.Builder("mixed", 7)
    x = b.input((8, 8, 4), "img")
    y = b.separable_conv2d(x, 6, 3, "sep", padding="same", activation="swish")
    y = b.conv2d_transpose(y, 5, 3, "up", strides=2, padding="same", activation="relu")
    y = b.rmsnorm(y, "rms")
    y = b.prelu(y, "prelu")
    z = b.einsum_dense(y, "abcd,de->abce", (5, 3), "ein", bias_axes="e")
    yield "mixed", b.finish([z])


def test_writers_produce_clean_files(validate, modelgen):
    for name, spec in generated_models(modelgen):
        found = validate.problems(modelgen.dumps(spec))
        assert found == [], (name, found)


def test_every_damage_is_reported(validate, modelgen):
    good = json.loads(modelgen.dumps(modelgen.small_cnn()))
    layers = good["architecture"]["config"]["layers"]
    conv = next(l for l in layers if l["class_name"] == "Conv2D")
    dense = next(l for l in layers if l["class_name"] == "Dense")

    bad = copy.deepcopy(good)
    bad["image_data_format"] = "channels_first"
    del bad["trainable_params"][conv["name"]]["bias"]
    bl = bad["architecture"]["config"]["layers"]
    next(l for l in bl if l["name"] == dense["name"])["config"].pop("units")
    next(l for l in bl if l["name"] == conv["name"])["config"]["activation"] = "mish"
    bl.append({"class_name": "LSTM", "name": "rnn", "config": {}, "inbound_nodes": [
        {"args": [{"class_name": "__keras_tensor__", "config": {"keras_history": ["nowhere", 0, 0]}}], "kwargs": {}}]})
    bad["architecture"]["config"]["output_layers"] = [["ghost", 0, 0]]
    found = "\n".join(validate.problems(bad))
    assert "image_data_format" in found
    assert "parameter 'bias' missing under trainable_params['%s']" % conv["name"] in found
    assert "config key 'units' missing" in found
    assert "activation 'mish' is not known" in found
    assert "layer 'rnn' (LSTM): class is not run on the device" in found
    assert "inbound layer 'nowhere' does not exist" in found
    assert "output_layers: names unknown layer 'ghost'" in found


def test_parameter_lengths_and_chunks(validate, modelgen):
    good = json.loads(modelgen.dumps(modelgen.small_cnn()))
    conv = next(l for l in good["architecture"]["config"]["layers"] if l["class_name"] == "Conv2D")
    bad = copy.deepcopy(good)
    p = bad["trainable_params"][conv["name"]]
    p["bias"] = modelgen.encode_floats(np.zeros(conv["config"]["filters"] + 1, np.float32))
    p["weights"] = ["".join(p["weights"])]           # one chunk, longer than 1024 characters
    found = "\n".join(validate.problems(bad))
    assert "bias has %d values, expected %d" % (conv["config"]["filters"] + 1, conv["config"]["filters"]) in found
    assert "chunk longer than 1024 characters" in found
    bad = copy.deepcopy(good)
    bad["trainable_params"][conv["name"]]["weights"] = ["not base64 !!"]
    assert "not a list of base64 fp32 chunks" in "\n".join(validate.problems(bad))


def test_nested_model_parameters_carry_the_outer_name(validate, modelgen):
    inner = modelgen.Builder("inner", 3)
    xi = inner.input((6,), "inner_in")
    yi = inner.dense(xi, 4, "fc", activation="relu")
    outer = modelgen.Builder("outer", 4)
    x = outer.input((6,), "x")
    y = outer.nested(inner.finish([yi]), [x], "block")
    spec = outer.finish([y] if not isinstance(y, (list, tuple)) else list(y))
    assert validate.problems(modelgen.dumps(spec)) == []
    broken = json.loads(modelgen.dumps(spec))
    broken["trainable_params"]["fc"] = broken["trainable_params"].pop("block_fc")  # prefix dropped
    assert any("trainable_params['block_fc']" in f for f in validate.problems(broken))


def test_not_json_and_wrong_top_level(validate):
    assert validate.problems("{ not json")[0].startswith("file: not valid JSON")
    assert validate.problems("[1, 2]") == ["file: top level must be an object"]
    assert any("architecture.config missing" in f for f in validate.problems({"image_data_format": "channels_last"}))
