"""CPU checks that pin the model-level parts of the oracle without the reference: the file format
(base64 chunks, connection forms, parameter prefixes of nested models), the definition of causal
attention by the prefix identity against torch's scaled_dot_product_attention(is_causal=True),
BatchNormalization against its folded form, LayerNormalization over arbitrary axes against a
float64 numpy statement, and the graph walk (nested model == the same layers written inline)."""
import base64
import json

import numpy as np
import pytest
import torch
from scipy import special


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    assert a.shape == b.shape, (a.shape, b.shape)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def test_base64_chunks_match_stdlib(oracle, modelgen):
    r = np.random.default_rng(0)
    for n in (1, 2, 3, 191, 192, 193, 1000):
        v = r.standard_normal(n).astype(np.float32)
        chunks = modelgen.encode_floats(v)
        assert all(len(c) <= 1024 for c in chunks)
        # 1024 characters hold exactly 768 bytes = 192 floats, so every chunk decodes on its own
        assert b"".join(base64.b64decode(c) for c in chunks) == v.astype("<f4").tobytes()
        assert np.array_equal(oracle.decode_floats(chunks), v)
    # url-safe alphabet and plain number arrays are accepted too (base64.hpp:65-108, import_model.hpp:274-297)
    v = np.frombuffer(bytes([0xfb, 0xff, 0xbf, 0x3f]), "<f4")
    std = base64.b64encode(v.tobytes()).decode()
    assert "+" in std or "/" in std
    assert np.array_equal(oracle.decode_floats([std.replace("+", "-").replace("/", "_")]), v)
    assert np.array_equal(oracle.decode_floats([1.5, -2.0]), np.array([1.5, -2.0], np.float32))
    with pytest.raises(RuntimeError):
        oracle.decode_floats([base64.b64encode(b"abc").decode()])


def test_single_connection_may_be_a_flat_triple(oracle, modelgen):
    spec = modelgen.small_cnn()
    x = np.random.default_rng(1).uniform(-1, 1, (32, 32, 3)).astype(np.float32)
    want = oracle.OracleModel(modelgen.dumps(spec)).predict([x])[0]
    cfg = spec["architecture"]["config"]
    cfg["input_layers"] = cfg["input_layers"][0]
    cfg["output_layers"] = cfg["output_layers"][0]
    got = oracle.OracleModel(modelgen.dumps(spec)).predict([x])[0]
    assert np.array_equal(got, want)


def test_causal_prefix_identity_equals_sdpa_is_causal(oracle, modelgen):
    """Row t of causal self-attention is MHA(query = x[t:t+1], value = x[0:t+1]); with identity-like projections
    removed this must be torch's causal SDPA on the projected tensors."""
    b = modelgen.Builder("causal_probe", 9)
    T, D, H, dk = 9, 16, 2, 8
    x_in = b.input((T, D), "x")
    out = b.mha(x_in, x_in, "attn", heads=H, key_dim=dk, std=0.3, bias_std=0.2)
    spec = b.finish([out])
    x = np.random.default_rng(2).standard_normal((T, D)).astype(np.float32)
    got = oracle.OracleModel(modelgen.dumps(spec)).predict([x], causal=True)[0]
    w = [np.asarray(v, np.float64) for v in spec["trainable_params"]["attn"]["weights"]]
    qw, qb, kw, kb, vw, vb, ow, ob = w
    X = x.astype(np.float64)
    q = np.einsum("td,dhk->htk", X, qw) + qb[:, None, :]
    k = np.einsum("td,dhk->htk", X, kw) + kb[:, None, :]
    v = np.einsum("td,dhk->htk", X, vw) + vb[:, None, :]
    o = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v),
                                                         is_causal=True).numpy()
    want = np.einsum("htk,hkd->td", o, ow) + ob
    assert rel(got, want) <= 2e-6
    # and without the flag the same file is the reference's unmasked attention
    o = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v)).numpy()
    assert rel(oracle.OracleModel(modelgen.dumps(spec)).predict([x])[0], np.einsum("htk,hkd->td", o, ow) + ob) <= 2e-6


def test_cached_decoder_equals_causal_prediction_rows(oracle, modelgen):
    """The oracle's KV-cached decoder (the timed CPU baseline of the decode benchmark) fed token by token returns, at
    step t, row t of the causal prediction of the whole sequence, which is defined through the reference's own
    MultiHeadAttention(query = x[t:t+1], value = x[0:t+1]); with and without attention biases."""
    for bias_std in (0.1, 0.0):
        spec = modelgen.gpt2(seed=61, layers=2, d_model=32, heads=4, vocab=53, max_pos=16, bias_std=bias_std,
                             random_affine=True, std=0.2)
        ref = oracle.OracleModel(modelgen.dumps(spec))
        ids = np.random.default_rng(62).integers(0, 53, 11).astype(np.float32)
        want = ref.predict([ids, np.arange(11, dtype=np.float32)], causal=True)[0]
        dec = oracle.CachedDecoder(ref)
        for t in range(11):
            assert rel(dec.step(ids[t]), want[t]) <= 2e-6, t


def test_batchnorm_equals_folded_convolution(oracle, modelgen):
    """conv -> BN equals a convolution with W' = W * inv[n], b' = b * inv + beta - mean * inv (the load-time fold
    the GPU path applies), to 1e-6."""
    b = modelgen.Builder("bn_probe", 12)
    x_in = b.input((9, 9, 5), "x")
    c = b.conv2d(x_in, 7, 3, "conv", padding="same", bias_std=0.3)
    spec = b.finish([b.batchnorm(c, "bn", random_stats=True)])
    x = np.random.default_rng(3).standard_normal((9, 9, 5)).astype(np.float32)
    want = oracle.OracleModel(modelgen.dumps(spec)).predict([x])[0]
    p = spec["trainable_params"]
    eps = [l for l in spec["architecture"]["config"]["layers"] if l["name"] == "bn"][0]["config"]["epsilon"]
    inv = p["bn"]["gamma"].astype(np.float64) / np.sqrt(p["bn"]["moving_variance"].astype(np.float64) + eps)
    w = p["conv"]["weights"].reshape(7, 3, 3, 5).astype(np.float64) * inv[:, None, None, None]
    bias = p["conv"]["bias"].astype(np.float64) * inv + p["bn"]["beta"] - p["bn"]["moving_mean"] * inv
    xt = torch.from_numpy(x.astype(np.float64)).permute(2, 0, 1)[None]
    y = torch.nn.functional.conv2d(xt, torch.from_numpy(w).permute(0, 3, 1, 2), torch.from_numpy(bias), padding=1)
    assert rel(want, y[0].permute(1, 2, 0).numpy()) <= 1e-6


@pytest.mark.parametrize("shape,axes", [((6, 7, 8), [-1]), ((6, 7, 8), [1]), ((6, 7, 8), [1, 3]), ((6, 7, 8), [2, 3]),
                                        ((3, 4, 5, 6), [2, 4]), ((6, 7, 8), [1, 2, 3])])
def test_layernorm_axes_vs_float64(oracle, shape, axes):
    r = np.random.default_rng(4)
    x = (r.standard_normal(shape) * 3 + 2).astype(np.float32)
    rank = len(shape)
    pos = sorted(a + rank + 1 if a < 0 else a for a in axes)
    pshape = [shape[a - 1] if a in pos else 1 for a in range(1, rank + 1)]
    n = int(np.prod(pshape))
    g, b = r.standard_normal(n).astype(np.float32), r.standard_normal(n).astype(np.float32)
    X = x.astype(np.float64)
    ax = tuple(a - 1 for a in pos)
    mean, var = X.mean(ax, keepdims=True), X.var(ax, keepdims=True)  # biased variance
    want = (X - mean) / np.sqrt(var + 1e-3) * g.reshape(pshape) + b.reshape(pshape)
    assert rel(oracle.layernorm_axes(x, axes, g, b, 1e-3), want) <= 2e-6
    if pos == list(range(rank - len(pos) + 1, rank + 1)):  # trailing axes: torch's layer_norm is the same formula
        t = torch.nn.functional.layer_norm(torch.from_numpy(X), [shape[a - 1] for a in pos],
                                           torch.from_numpy(g.astype(np.float64)).reshape([shape[a - 1] for a in pos]),
                                           torch.from_numpy(b.astype(np.float64)).reshape([shape[a - 1] for a in pos]), 1e-3)
        assert rel(oracle.layernorm_axes(x, axes, g, b, 1e-3), t.numpy()) <= 2e-6


def test_nested_model_equals_inline_layers(oracle, modelgen):
    """A Functional model used as a layer computes what its layers compute when written into the outer model, and
    reads its parameters under "<layer>_<inner layer>"."""
    def body(b, x, prefix):
        h = b.dense(x, 12, prefix + "fc1", activation="relu", bias_std=0.2)
        return b.add([b.dense(h, 8, prefix + "fc2", bias_std=0.2), x], prefix + "res")

    inner = modelgen.Builder("blk", 5)
    inner_out = body(inner, inner.input((4, 8), "blk_in"), "")
    inner_spec = inner.finish([inner_out])

    outer = modelgen.Builder("outer", 6)
    x_in = outer.input((4, 8), "x")
    (y,) = outer.nested(inner_spec, [x_in], "blk")
    spec_nested = outer.finish([outer.dense(y, 3, "head", bias_std=0.1)])
    assert "blk_fc1" in spec_nested["trainable_params"] and "fc1" not in spec_nested["trainable_params"]

    flat = modelgen.Builder("outer", 6)
    xf = flat.input((4, 8), "x")
    yf = body(flat, xf, "blk_")
    spec_flat = flat.finish([flat.dense(yf, 3, "head", bias_std=0.1)])
    for name, prm in spec_nested["trainable_params"].items():  # same numbers under the same names
        spec_flat["trainable_params"][name] = prm
    x = np.random.default_rng(7).standard_normal((4, 8)).astype(np.float32)
    a = oracle.OracleModel(modelgen.dumps(spec_nested)).predict([x])[0]
    b = oracle.OracleModel(modelgen.dumps(spec_flat)).predict([x])[0]
    assert np.array_equal(a, b)


def test_concatenate_axis_counts_from_first_rank(oracle, modelgen):
    b = modelgen.Builder("cat_probe", 8)
    p, q = b.input((3, 4), "p"), b.input((3, 2), "q")
    spec = b.finish([b.concatenate([p, q], "cat", axis=2), b.concatenate([p, p], "cat0", axis=1)])
    r = np.random.default_rng(8)
    xp, xq = r.standard_normal((3, 4)).astype(np.float32), r.standard_normal((3, 2)).astype(np.float32)
    a, c = oracle.OracleModel(modelgen.dumps(spec)).predict([xp, xq])
    assert np.array_equal(a, np.concatenate([xp, xq], axis=1)) and np.array_equal(c, np.concatenate([xp, xp], axis=0))


def test_embedded_tests_replay_and_detect_corruption(oracle, modelgen):
    spec = modelgen.small_cnn()
    x = np.random.default_rng(9).uniform(-1, 1, (32, 32, 3)).astype(np.float32)
    y = oracle.OracleModel(modelgen.dumps(spec)).predict([x])[0]
    spec["tests"] = [{"inputs": [x], "outputs": [y]}]
    assert oracle.OracleModel(modelgen.dumps(spec)).run_embedded_tests()
    spec["tests"] = [{"inputs": [x], "outputs": [y + 1e-3]}]
    with pytest.raises(RuntimeError, match="test failed"):
        oracle.OracleModel(modelgen.dumps(spec)).run_embedded_tests()
    # the file is plain JSON
    assert json.loads(modelgen.dumps(spec))["image_data_format"] == "channels_last"


def test_gqa_vs_float64_and_reduction_to_mha(oracle, modelgen):
    """GroupQueryAttention against an explicit float64 statement (query head h reads kv head h // group, sigmoid gate),
    and with as many kv heads as query heads and no gate it must equal MultiHeadAttention on the same kernels."""
    r = np.random.default_rng(21)
    T, S, D, hd, hq, hkv = 5, 7, 12, 4, 6, 2
    q, v = r.standard_normal((T, D)).astype(np.float32), r.standard_normal((S, D)).astype(np.float32)
    def mk(*shape):
        return (r.standard_normal(shape) * 0.4).astype(np.float32)
    for use_bias in (True, False):
        for use_gate in (True, False):
            w = []
            def put(kshape, bshape):
                w.append(mk(*kshape))
                if use_bias:
                    w.append(mk(*bshape))
            put((D, hq, hd), (hq, hd)); put((D, hkv, hd), (hkv, hd))
            if use_gate:
                put((D, hq, hd), (hq, hd))
            put((D, hkv, hd), (hkv, hd)); put((hq, hd, D), (D,))
            got = oracle.gqa(q, v, None, hd, hq, hkv, w, use_bias, use_gate)
            W = [a.astype(np.float64) for a in w]
            step = 2 if use_bias else 1
            kern = lambda i: W[i * step]
            bias = lambda i: W[i * step + 1] if use_bias else 0.0
            vi, oi = (3, 4) if use_gate else (2, 3)
            Q = np.einsum("td,dhc->thc", q.astype(np.float64), kern(0)) + bias(0)
            K = np.einsum("sd,dhc->shc", v.astype(np.float64), kern(1)) + bias(1)
            V = np.einsum("sd,dhc->shc", v.astype(np.float64), kern(vi)) + bias(vi)
            K, V = np.repeat(K, hq // hkv, axis=1), np.repeat(V, hq // hkv, axis=1)
            P = special.softmax(np.einsum("thc,shc->hts", Q, K) / np.sqrt(hd), axis=-1)
            A = np.einsum("hts,shc->thc", P, V)
            if use_gate:
                A = A * special.expit(np.einsum("td,dhc->thc", q.astype(np.float64), kern(2)) + bias(2))
            want = np.einsum("thc,hcd->td", A, kern(oi)) + bias(oi)
            assert rel(got, want) <= 3e-6
    # hkv == hq, no gate: the MultiHeadAttention layer with key_dim = value_dim = head_dim
    w = [mk(D, hq, hd), mk(hq, hd), mk(D, hq, hd), mk(hq, hd), mk(D, hq, hd), mk(hq, hd), mk(hq, hd, D), mk(D)]
    a = oracle.gqa(q, v, None, hd, hq, hq, w, True, False)
    b = oracle.mha(q, v, None, hq, hd, hd, w, True)
    assert rel(a, b) <= 2e-6


def test_rmsnorm_and_separable_conv(oracle, modelgen):
    r = np.random.default_rng(22)
    x = (r.standard_normal((6, 7, 8)) * 2 + 1).astype(np.float32)
    for axes in ([-1], [1], [1, 3]):
        pos = sorted(a + 4 if a < 0 else a for a in axes)
        pshape = [x.shape[a - 1] if a in pos else 1 for a in (1, 2, 3)]
        scale = r.standard_normal(int(np.prod(pshape))).astype(np.float32)
        X = x.astype(np.float64)
        want = X / np.sqrt((X * X).mean(tuple(a - 1 for a in pos), keepdims=True) + 1e-6) * scale.reshape(pshape)
        assert rel(oracle.rmsnorm_axes(x, axes, scale, 1e-6), want) <= 2e-6
    t = torch.nn.functional.rms_norm(torch.from_numpy(x.astype(np.float64)), [8], eps=1e-6).numpy()
    assert rel(oracle.rmsnorm_axes(x, [-1], None, 1e-6), t) <= 2e-6
    # SeparableConv2D = grouped 3x3 convolution without bias, then a 1x1 convolution with bias (torch, float64)
    b = modelgen.Builder("sep_probe", 23)
    x_in = b.input((9, 10, 6), "x")
    spec = b.finish([b.separable_conv2d(x_in, 5, 3, "sep", strides=2, padding="same")])
    xs = r.standard_normal((9, 10, 6)).astype(np.float32)
    got = oracle.OracleModel(modelgen.dumps(spec)).predict([xs])[0]
    p = spec["trainable_params"]["sep"]
    xt = torch.from_numpy(xs.astype(np.float64)).permute(2, 0, 1)[None]
    xt = torch.nn.functional.pad(xt, (0, 1, 1, 1))  # TF same, k3 s2: height 9 -> pad (1, 1), width 10 -> pad (0, 1)
    dw = torch.nn.functional.conv2d(xt, torch.from_numpy(p["slice_weights"].astype(np.float64))[:, None], stride=2, groups=6)
    pw = torch.nn.functional.conv2d(dw, torch.from_numpy(p["stack_weights"].astype(np.float64)).permute(0, 3, 1, 2),
                                    torch.from_numpy(p["bias"].astype(np.float64)))
    assert rel(got, pw[0].permute(1, 2, 0).numpy()) <= 3e-6


def test_upsampling_vs_torch_interpolate(oracle):
    """Nearest and bilinear upsampling by integer factors equal torch's interpolate (half-pixel centres,
    align_corners=False), which is the coordinate rule the reference states."""
    r = np.random.default_rng(31)
    x = r.standard_normal((5, 6, 3)).astype(np.float32)
    xt = torch.from_numpy(x.astype(np.float64)).permute(2, 0, 1)[None]
    for fy, fx in ((2, 2), (3, 1), (1, 4), (2, 3)):
        near = torch.nn.functional.interpolate(xt, scale_factor=(fy, fx), mode="nearest")[0].permute(1, 2, 0).numpy()
        assert np.array_equal(oracle.upsample2d(x, fy, fx), near.astype(np.float32))
        bil = torch.nn.functional.interpolate(xt, scale_factor=(fy, fx), mode="bilinear", align_corners=False)[0]
        assert rel(oracle.upsample2d(x, fy, fx, bilinear=True), bil.permute(1, 2, 0).numpy()) <= 2e-6


def test_rescaling_normalization_and_passthrough_layers(oracle, modelgen):
    """Rescaling and Normalization pinned by what the arithmetic fixes: statistics taken from the data itself give
    zero mean / unit variance per slice; the inverted layer undoes the plain one; an axis-less layer uses one pair;
    a variance of zero divides by the 1e-7 floor (layers/normalization_layer.hpp:38-45); augmentation layers pass
    their input through (import_model.hpp:1796-1838)."""
    r = np.random.default_rng(31)
    x = (r.standard_normal((6, 5, 4)) * 3 + 2).astype(np.float32)
    b = modelgen.Builder("prep", 31)
    xin = b.input(x.shape, "x")
    y0 = b.rescaling(xin, "scale", 1 / 127.5, -1.0)
    y1 = b.normalization(xin, "norm_c", axis=-1)
    y2 = b.normalization(y1, "denorm_c", axis=-1, invert=True)
    y3 = b.normalization(xin, "norm_w", axis=2)
    y4 = b.normalization(xin, "norm_all", axis=None)
    y5 = b._add("RandomHue", "aug", {}, [xin], x.shape)
    y5 = b._add("Pipeline", "aug2", {}, [y5], x.shape)
    b.params["norm_c"] = {"mean": x.mean((0, 1)), "variance": x.var((0, 1))}
    b.params["denorm_c"] = dict(b.params["norm_c"])
    b.params["norm_w"] = {"mean": x.mean((0, 2)), "variance": np.zeros(5, np.float32)}
    b.params["norm_all"] = {"mean": np.array([2.5], np.float32), "variance": np.array([4.0], np.float32)}
    out = oracle.OracleModel(modelgen.dumps(b.finish([y0, y1, y2, y3, y4, y5]))).predict([x])
    assert np.allclose(out[0], x.astype(np.float64) / 127.5 - 1.0, atol=1e-6)
    assert np.abs(out[1].mean((0, 1))).max() < 1e-5 and np.abs(out[1].var((0, 1)) - 1).max() < 1e-4
    assert rel(out[2], x) < 1e-6
    want3 = (x.astype(np.float64) - x.mean((0, 2)).astype(np.float64)[None, :, None]) / 1e-7
    assert rel(out[3], want3) < 1e-5
    assert rel(out[4], (x.astype(np.float64) - 2.5) / 2.0) < 1e-6
    assert np.array_equal(out[5], x)
    # two axes are refused, as in the reference (layers/normalization_layer.hpp:32)
    bad = modelgen.Builder("bad", 1)
    xb = bad.input((3, 4), "x")
    yb = bad.normalization(xb, "n", axis=-1)
    spec = bad.finish([yb])
    [l for l in spec["architecture"]["config"]["layers"] if l["name"] == "n"][0]["config"]["axis"] = [1, 2]
    with pytest.raises(Exception):
        oracle.OracleModel(modelgen.dumps(spec)).predict([np.zeros((3, 4), np.float32)])
