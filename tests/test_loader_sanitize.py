"""The host half of the C++ model loader (JSON reader, base64 decoder, einsum analysis, graph builder, fusion, shape
inference) built with g++ -fsanitize=address,undefined and fed good files, the damaged-file corpus of the validator tests,
truncations at many offsets, broken / oversized base64 chunks and random byte flips.  No file may trip a sanitizer, every
good file must pass and every damaged one must come back with an error status (a message, not a crash).
The file format is the reference's: include/fdeep/import_model.hpp:274-297 (parameter arrays), base64.hpp:65-108."""
import copy
import json
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "frugally-deep_amd")
CSRC = os.path.join(PKG, "csrc")


@pytest.fixture(scope="module")
def harness(fdx, tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("san") / "loader_sanitize.bin")
    flags = ["-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer",
             "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-w"]
    # the loader's own source, sanitized; everything else it names (launchers, runtime) comes from the built library
    subprocess.check_call(["g++"] + flags + [os.path.join(ROOT, "tests", "cpp", "loader_sanitize.cpp"), os.path.join(CSRC, "model.cpp"),
                                           "-L", PKG, "-lfdx", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath," + PKG,
                                           "-Wl,-rpath,/opt/rocm/lib", "-pthread", "-o", exe])
    return exe


def run(exe, paths, tmp_path):
    lst = tmp_path / "list.txt"
    lst.write_text("\n".join(str(p) for p in paths) + "\n")
    # (the two opt-in fusions are switched on so that their load-time passes -- filter packing, gamma / beta folding -- run too)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1",
               FDX_CHAIN="1", FDX_LN_FOLD="1")
    out = subprocess.run([exe, str(lst)], capture_output=True, text=True, timeout=600, env=env)
    assert out.returncode == 0 and "loader_sanitize done: %d files" % len(paths) in out.stdout, (out.stdout[-2000:], out.stderr[-4000:])
    status = {}
    for line in out.stdout.splitlines():
        if line[:1].isdigit():
            code, path = line.split(" ", 1)
            status[path] = int(code)
    return status


def good_models(modelgen):
    yield "small_cnn", modelgen.small_cnn()
    yield "resnet", modelgen.resnet50(input_size=32, width=8, blocks=(1, 1, 1, 1), classes=10, random_bn=True)
    yield "mobilenet", modelgen.mobilenet_v2(input_size=32, alpha=0.25, classes=10, truncate=4)
    yield "encoder", modelgen.encoder(layers=1, seq=8, d_model=16, heads=2, ffn=32)
    yield "gpt2", modelgen.gpt2(layers=1, d_model=16, heads=2, vocab=50, max_pos=16)
    # bottleneck blocks wide enough for the loader to join the shortcut convolution with the block's last convolution and to
    # pack the filters of a block tail / next block head pair
    b = modelgen.Builder("blocks", 8)
    x = b.input((6, 6, 64), "img")
    for blk in range(2):
        y = b.conv2d(x, 64, 1, "b%d_c1" % blk, strides=2 if blk == 0 else 1, activation="relu")
        z = b.conv2d(y, 128, 1, "b%d_c3" % blk, use_bias=False)
        z = b.batchnorm(z, "b%d_bn" % blk, random_stats=True)
        sc = b.conv2d(x, 128, 1, "b%d_sc" % blk, strides=2) if blk == 0 else x
        x = b.relu(b.add([sc, z], "b%d_sum" % blk), "b%d_out" % blk)
    yield "blocks", b.finish([b.conv2d(x, 64, 1, "tail")])
    b = modelgen.Builder("mixed", 7)
    x = b.input((8, 8, 4), "img")
    y = b.separable_conv2d(x, 6, 3, "sep", padding="same", activation="swish")
    y = b.conv2d_transpose(y, 5, 3, "up", strides=2, padding="same", activation="relu")
    y = b.rmsnorm(y, "rms")
    y = b.prelu(y, "prelu")
    z = b.einsum_dense(y, "abcd,de->abce", (5, 3), "ein", bias_axes="e")
    yield "mixed", b.finish([z])


def test_loader_survives_good_and_damaged_files(harness, modelgen, tmp_path):
    rng = np.random.default_rng(61)
    good, bad = [], []

    def put(name, data, into):
        p = tmp_path / name
        p.write_bytes(data if isinstance(data, bytes) else data.encode())
        into.append(str(p))

    texts = {}
    for name, spec in good_models(modelgen):
        texts[name] = modelgen.dumps(spec)
        texts[name] = texts[name] if isinstance(texts[name], bytes) else texts[name].encode()
        put(name + ".json", texts[name], good)
    # a good file that carries an embedded test case
    spec = modelgen.small_cnn()
    spec["tests"] = [{"inputs": [np.zeros((32, 32, 3), np.float32)], "outputs": [np.full((10,), 0.1, np.float32)]}]
    put("with_test.json", modelgen.dumps(spec), good)

    # the validator tests' damage, as files
    base = json.loads(texts["small_cnn"])
    layers = base["architecture"]["config"]["layers"]
    conv = next(l for l in layers if l["class_name"] == "Conv2D")
    dense = next(l for l in layers if l["class_name"] == "Dense")

    def damaged(fn):
        d = copy.deepcopy(base)
        fn(d)
        return json.dumps(d)

    def layer(d, name):
        return next(l for l in d["architecture"]["config"]["layers"] if l["name"] == name)

    cases = {
        "channels_first": lambda d: d.__setitem__("image_data_format", "channels_first"),
        "no_bias": lambda d: d["trainable_params"][conv["name"]].pop("bias"),
        "no_units": lambda d: layer(d, dense["name"])["config"].pop("units"),
        "mish": lambda d: layer(d, conv["name"])["config"].__setitem__("activation", "mish"),
        "ghost_output": lambda d: d["architecture"]["config"].__setitem__("output_layers", [["ghost", 0, 0]]),
        "dangling_inbound": lambda d: layer(d, dense["name"])["inbound_nodes"][0]["args"][0]["config"].__setitem__("keras_history", ["nowhere", 0, 0]),
        "long_bias": lambda d: d["trainable_params"][conv["name"]].__setitem__("bias", modelgen.encode_floats(np.zeros(conv["config"]["filters"] + 1, np.float32))),
        "not_base64": lambda d: d["trainable_params"][conv["name"]].__setitem__("weights", ["not base64 !!"]),
        "chunk_cut_mid_quantum": lambda d: d["trainable_params"][conv["name"]].__setitem__("weights", [d["trainable_params"][conv["name"]]["weights"][0][:-3]]),
        "chunk_one_char": lambda d: d["trainable_params"][conv["name"]].__setitem__("weights", ["A"]),
        "chunk_padding_only": lambda d: d["trainable_params"][conv["name"]].__setitem__("weights", ["===="]),
        "chunk_not_fp32_multiple": lambda d: d["trainable_params"][conv["name"]].__setitem__("weights", ["AAAAAA=="]),
        "weights_number": lambda d: d["trainable_params"][conv["name"]].__setitem__("weights", 5),
        "weights_nested": lambda d: d["trainable_params"][conv["name"]].__setitem__("weights", [["AAAA"]]),
        "huge_filters": lambda d: layer(d, conv["name"])["config"].__setitem__("filters", 2 ** 40),
        "negative_kernel": lambda d: layer(d, conv["name"])["config"].__setitem__("kernel_size", [-3, 3]),
        "zero_stride": lambda d: layer(d, conv["name"])["config"].__setitem__("strides", [0, 0]),
        "layers_not_array": lambda d: d["architecture"]["config"].__setitem__("layers", {"a": 1}),
        "input_shape_strings": lambda d: d.__setitem__("input_shapes", [["x", "y", "z"]]),
        "test_values_short": lambda d: d.__setitem__("tests", [{"inputs": [{"shape": [32, 32, 3], "values": ["AAAA"]}], "outputs": [{"shape": [10], "values": ["AAAA"]}]}]),
        "self_loop": lambda d: layer(d, dense["name"])["inbound_nodes"][0]["args"][0]["config"].__setitem__("keras_history", [dense["name"], 0, 0]),
    }
    for name, fn in cases.items():
        put("bad_" + name + ".json", damaged(fn), bad)
    # one oversized chunk: the whole array as a single string
    d = copy.deepcopy(base)
    w = d["trainable_params"][dense["name"]]["weights"]
    d["trainable_params"][dense["name"]]["weights"] = ["".join(w)]
    put("one_big_chunk.json", json.dumps(d), [])  # accepted or refused; must only not trip the sanitizer
    # truncations: at a spread of offsets of every good text, plus the last bytes one by one
    for name, t in texts.items():
        cuts = sorted(set(int(c) for c in np.linspace(0, len(t) - 1, 24)) | set(range(max(0, len(t) - 8), len(t))))
        for c in cuts:
            put("cut_%s_%d.json" % (name, c), t[:c], bad)
    # random byte flips in the structural part (the first 6000 bytes hold the architecture) and in the parameters
    fuzz = []
    for name in ("small_cnn", "gpt2", "mixed"):
        t = bytearray(texts[name])
        for k in range(40):
            u = bytearray(t)
            for _ in range(int(rng.integers(1, 4))):
                pos = int(rng.integers(0, min(len(u), 6000) if k % 2 == 0 else len(u)))
                u[pos] = int(rng.integers(0, 256))
            put("flip_%s_%d.json" % (name, k), bytes(u), fuzz)
    not_json = []
    put("empty.json", b"", not_json)
    put("brace.json", b"{", not_json)
    put("deep.json", b"[" * 100000, not_json)
    put("string_open.json", b'{"a": "', not_json)
    put("escape_end.json", b'{"a": "\\', not_json)
    put("unicode_cut.json", b'{"a": "\\u12', not_json)
    put("number_huge.json", b'{"image_data_format": 1e999999}', not_json)

    one_big = [str(tmp_path / "one_big_chunk.json")]
    status = run(harness, good + bad + one_big + fuzz + not_json, tmp_path)
    for p in good:
        assert status[p] == 0, p
    for p in bad + not_json:
        assert status[p] != 0, p
