"""GPU parity for the strided layer forms: EinsumDense with arbitrary equations, Add with size-1
broadcasting, Concatenate, LayerNormalization over arbitrary axes, and models that nest a
Functional model, against the CPU oracle.  Tolerance: max|gpu - ref| / max|ref| <= 1e-4 per tensor
(fp32, summation order differs); pure data movement (Concatenate) must be bit-exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-4


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    assert a.shape == b.shape, (a.shape, b.shape)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def say(*a):
    print(*a, flush=True)


EINSUM = [
    # equation, sample shape, kernel shape, bias_axes
    ("abc,cd->abd", (7, 12), (12, 9), "d"),          # the three equations of the reference's test models
    ("abc,cde->abde", (5, 8), (8, 3, 4), "de"),      # (keras_export/generate_test_models.py:573-585)
    ("abc,cde->abde", (5, 8), (8, 3, 4), "ed"),      # bias stored in rhs order whatever the string says
    ("abcd,cde->abe", (4, 3, 6), (3, 6, 5), "e"),
    ("abc,cd->abd", (7, 12), (12, 9), "b"),          # bias over a row axis
    ("abc,cd->abd", (7, 12), (12, 9), None),
    ("abc,dc->abd", (6, 10), (11, 10), "d"),         # kernel stored transposed
    ("abc,cd->adb", (6, 10), (10, 4), "d"),          # output permuted
    ("abc,bcd->abd", (6, 10), (6, 10, 3), "bd"),     # a character shared by all three operands
    ("abcd,bde->ace", (3, 4, 5), (3, 5, 7), "e"),    # two summed characters that are not adjacent in the input
    ("ab,bc->ac", (33,), (33, 65), "c"),
]


@pytest.mark.parametrize("eq,xs,ks,bias_axes", EINSUM)
def test_einsum_dense_kernel(fdx, oracle, eq, xs, ks, bias_axes):
    say("einsum", eq, xs, ks, bias_axes)
    r = np.random.default_rng(abs(hash((eq, bias_axes))) % 2**31)
    batch = 3
    x = r.standard_normal((batch,) + xs).astype(np.float32)
    k = r.standard_normal(ks).astype(np.float32)
    lhs, rest = eq.split(",")
    ker, rhs = rest.split("->")
    size = dict(zip(ker, ks))
    size.update(zip(lhs[1:], xs))
    bias = None
    if bias_axes:
        bias = r.standard_normal([size[c] for c in rhs if c in bias_axes]).astype(np.float32)
    want = np.stack([oracle.einsum_dense(x[i], eq, k, list(ks), bias, bias_axes) for i in range(batch)])
    got = fdx.einsum_dense(x, eq, k, bias, bias_axes)
    assert rel(got, want) <= TOL


def test_einsum_dense_errors(fdx):
    x, k = np.zeros((1, 4, 5), np.float32), np.zeros((6, 3), np.float32)
    with pytest.raises(RuntimeError, match="inconsistent char size"):
        fdx.einsum_dense(x, "abc,cd->abd", k)
    with pytest.raises(RuntimeError, match="neither summed nor in the output"):
        fdx.einsum_dense(x, "abc,bd->ad", np.zeros((4, 3), np.float32))


BCAST = [((4, 5, 6), (4, 5, 6)), ((4, 5, 6), (1, 1, 6)), ((4, 5, 6), (4, 1, 1)), ((4, 1, 6), (1, 5, 1)), ((5, 6), (3, 1, 6)),
         ((2, 3, 4, 5, 6), (1, 3, 1, 5, 1)), ((7,), (9, 1))]


@pytest.mark.parametrize("sa,sb", BCAST)
def test_broadcast_add(fdx, oracle, sa, sb):
    say("broadcast_add", sa, sb)
    r = np.random.default_rng(5)
    a = r.standard_normal((3,) + sa).astype(np.float32)
    b = r.standard_normal((3,) + sb).astype(np.float32)
    want = np.stack([oracle.add(a[i], b[i]) for i in range(3)])
    got = fdx.broadcast_add(a, b)
    assert got.shape == want.shape and np.array_equal(got, want)
    got = fdx.broadcast_add(a, b, act=fdx.relu_act(1.5, 0.1, 0.2))
    want = np.stack([oracle.relu(oracle.add(a[i], b[i]), 1.5, 0.1, 0.2) for i in range(3)])
    assert rel(got, want) <= 1e-6


def test_broadcast_add_rejects_mismatch(fdx):
    with pytest.raises(RuntimeError, match="Invalid shapes for combining tensors"):
        fdx.broadcast_add(np.zeros((1, 4, 5), np.float32), np.zeros((1, 3, 5), np.float32))


@pytest.mark.parametrize("shapes,axis", [([(4, 5, 6), (4, 5, 2), (4, 5, 9)], -1), ([(4, 5, 6), (4, 1, 6)], 2),
                                         ([(2, 5, 6), (4, 5, 6)], 1), ([(7,), (3,)], 1), ([(3, 4), (3, 5)], -1)])
def test_concat(fdx, shapes, axis):
    say("concat", shapes, axis)
    r = np.random.default_rng(6)
    xs = [r.standard_normal((2,) + s).astype(np.float32) for s in shapes]
    rank = len(shapes[0])
    a = axis + rank + 1 if axis < 0 else axis
    assert np.array_equal(fdx.concat(xs, axis), np.concatenate(xs, axis=a))


@pytest.mark.parametrize("shape,axes", [((6, 7, 8), [-1]), ((6, 7, 8), [1]), ((6, 7, 8), [2]), ((6, 7, 8), [1, 3]),
                                        ((6, 7, 8), [2, 3]), ((6, 7, 8), [1, 2, 3]), ((5, 300), [1]), ((3, 4, 5, 6), [2, 4]),
                                        ((9,), [1]), ((6, 1, 8), [1, 3])])
def test_layernorm_axes(fdx, oracle, shape, axes):
    say("layernorm_axes", shape, axes)
    r = np.random.default_rng(7)
    x = (r.standard_normal((3,) + shape) * 2 + 1).astype(np.float32)
    rank = len(shape)
    n = int(np.prod([shape[(a + rank + 1 if a < 0 else a) - 1] for a in axes]))
    g, b = r.standard_normal(n).astype(np.float32), r.standard_normal(n).astype(np.float32)
    for gamma, beta in ((g, b), (None, None)):
        want = np.stack([oracle.layernorm_axes(x[i], axes, gamma, beta, 1e-3) for i in range(3)])
        assert rel(fdx.layernorm_axes(x, axes, gamma, beta, 1e-3), want) <= TOL


def mixed_model(modelgen, seed=21):
    """EinsumDense in GEMM form and in permuted form, Concatenate, broadcasting Add, LayerNormalization over the
    sequence axis, and a nested Functional model applied to two different tensors (shared weights)."""
    inner = modelgen.Builder("inner_block", seed + 1)
    u = inner.input((6, 16), "inner_in")
    h = inner.dense(u, 24, "inner_fc1", activation="relu", bias_std=0.2)
    h2 = inner.dense(h, 16, "inner_fc2", bias_std=0.2)
    inner_spec = inner.finish([inner.add([h2, u], "inner_add"), h])

    b = modelgen.Builder("mixed", seed)
    x = b.input((6, 16), "tokens")
    gate = b.input((1, 16), "gate")
    e1 = b.einsum_dense(x, "abc,cde->abde", (16, 2, 8), "proj_heads", bias_axes="ed")     # one GEMM
    e2 = b.einsum_dense(e1, "abde,dec->abc", (2, 8, 16), "merge_heads", bias_axes="c", activation="gelu")
    e3 = b.einsum_dense(x, "abc,cd->adb", (16, 5), "permuted", bias_axes="d")               # (5, 6): strided kernel
    n1, side = b.nested(inner_spec, [e2], "shared_block")
    s = b.add([n1, gate], "gated")                                                            # (6,16) + (1,16)
    ln = b.layernorm_axes(s, "ln_seq", [1], eps=1e-3)                                         # over the sequence axis
    cat = b.concatenate([ln, x, side], "cat", axis=-1)                                        # (6, 16+16+24)
    out = b.dense(cat, 10, "head", activation="softmax")
    return b.finish([out, e3, cat])


def test_model_with_einsum_concat_broadcast_nested(fdx, oracle, modelgen):
    say("mixed model")
    spec = mixed_model(modelgen)
    r = np.random.default_rng(3)
    x = r.standard_normal((5, 6, 16)).astype(np.float32)
    gate = r.standard_normal((5, 1, 16)).astype(np.float32)
    js = modelgen.dumps(spec)
    ref = oracle.OracleModel(js)
    want = [ref.predict([x[i], gate[i]]) for i in range(5)]
    want = [np.stack([w[k] for w in want]) for k in range(3)]
    got = fdx.Model(js).predict([x, gate])
    errs = [rel(g, w) for g, w in zip(got, want)]
    say("  rel errors:", ["%.2e" % e for e in errs])
    assert max(errs) <= TOL


def test_nested_model_applied_twice(fdx, oracle, modelgen):
    """The same nested model called on two tensors: both calls read one set of parameters; the second call is
    Keras node 2 of the nested layer."""
    say("nested twice")
    inner = modelgen.Builder("tower", 31)
    u = inner.input((8, 8, 4), "tower_in")
    c = inner.conv2d(u, 8, 3, "tower_conv", padding="same", activation="relu", bias_std=0.1)
    bn = inner.batchnorm(c, "tower_bn", random_stats=True)
    inner_spec = inner.finish([inner.gap(bn, "tower_gap")])

    b = modelgen.Builder("siamese", 30)
    xa, xb = b.input((8, 8, 4), "left"), b.input((8, 8, 4), "right")
    (fa,) = b.nested(inner_spec, [xa], "tower")
    # second application of the same layer: one more inbound node, referenced as node 2
    b.layers[-1]["inbound_nodes"].append({"args": [modelgen._kt(xb)], "kwargs": {}})
    fb = modelgen.T("tower", fa.shape)
    fb.node, fb.tensor = 2, 0
    out = b.dense(b.concatenate([fa, fb], "both", axis=-1), 3, "cmp", bias_std=0.1)
    spec = b.finish([out])
    r = np.random.default_rng(4)
    xs = [r.standard_normal((4, 8, 8, 4)).astype(np.float32) for _ in range(2)]
    js = modelgen.dumps(spec)
    ref = oracle.OracleModel(js)
    want = np.stack([ref.predict([xs[0][i], xs[1][i]])[0] for i in range(4)])
    got = fdx.Model(js).predict(xs)[0]
    assert rel(got, want) <= TOL
    # swapping the two inputs swaps the halves the head sees: a shared tower gives f(left) == f(right) on equal inputs
    same = fdx.Model(js).predict([xs[0], xs[0]])[0]
    ref_same = np.stack([ref.predict([xs[0][i], xs[0][i]])[0] for i in range(4)])
    assert rel(same, ref_same) <= TOL


def test_custom_layer_runs_on_host_between_device_segments(fdx, oracle, modelgen):
    """A layer class the device path does not implement, supplied by the caller: it sees one sample at a time as
    host arrays, receives its trainable_params through get_param and its JSON through the creator, may change the
    shape, and its fused `activation` is applied afterwards like for any other layer."""
    say("custom layer")
    b = modelgen.Builder("custom_host", 55)
    x_in = b.input((6, 8), "x")
    h = b.dense(x_in, 12, "fc1", activation="relu", bias_std=0.2)
    b.params["pairs"] = {"scale": np.linspace(0.5, 1.5, 6).astype(np.float32)}
    c = b._add("PairSum", "pairs", {"name": "pairs", "activation": "relu", "shift": -0.25}, [h], (6, 6))
    spec = b.finish([b.dense(c, 4, "fc2", bias_std=0.2), c])
    seen = []

    def creator(get_param, layer, name):
        scale = get_param(name, "scale")
        shift = layer["config"]["shift"]
        seen.append((name, layer["class_name"]))
        return lambda ins: (ins[0][:, 0::2] + ins[0][:, 1::2]) * scale + shift  # (6, 12) -> (6, 6)

    r = np.random.default_rng(8)
    x = r.standard_normal((5, 6, 8)).astype(np.float32)
    p = spec["trainable_params"]
    hid = np.stack([oracle.relu(oracle.dense(x[i], p["fc1"]["weights"].reshape(-1), p["fc1"]["bias"], 12)) for i in range(5)])
    mid = oracle.relu(((hid[:, :, 0::2] + hid[:, :, 1::2]) * p["pairs"]["scale"] - 0.25).astype(np.float32))
    want = np.stack([oracle.dense(mid[i], p["fc2"]["weights"].reshape(-1), p["fc2"]["bias"], 4) for i in range(5)])
    js = modelgen.dumps(spec)
    with pytest.raises(fdx.FdxError, match="unknown layer type: PairSum"):
        fdx.Model(js)
    model = fdx.Model(js, custom_layers={"PairSum": creator})
    assert seen == [("pairs", "PairSum")]
    got = model.predict([x])
    assert rel(got[1], mid) <= 1e-6 and rel(got[0], want) <= TOL
    # a registered class overrides a built-in one
    const = lambda gp, layer, name: (lambda ins: np.full((6, 12 if name == "fc1" else 4), 7.0, np.float32))
    over = fdx.Model(js, custom_layers={"PairSum": creator, "Dense": const})
    assert np.all(over.predict([x])[0] == 7)
    # a failing layer surfaces as an error with its message
    def broken(get_param, layer, name):
        def run(ins):
            raise ValueError("boom in " + name)
        return run
    with pytest.raises(fdx.FdxError, match="custom layer failed.*boom in pairs"):
        fdx.Model(js, custom_layers={"PairSum": broken}).predict([x])


ACTS = [("tanh", ()), ("sigmoid", ()), ("swish", ()), ("hard_sigmoid", ()), ("selu", ()), ("elu", (0.7,)), ("celu", (1.0,)),
        ("exponential", ()), ("softsign", ()), ("softplus", ()), ("leaky_relu", (0.2,)), ("hard_shrink", (0.5,)),
        ("soft_shrink", (0.5,)), ("sparse_plus", ()), ("squareplus", (4.0,)), ("tanh_shrink", ()), ("threshold", (0.25, -2.0)),
        ("log_sigmoid", ()), ("hard_tanh", ())]


@pytest.mark.parametrize("name,params", ACTS, ids=[a[0] for a in ACTS])
def test_activation_kinds(fdx, oracle, name, params):
    say("activation", name)
    r = np.random.default_rng(12)
    x = np.concatenate([r.standard_normal(1021) * 3, [-20.0, -14.0, -13.5, -3.0, -1.0, -0.5, 0.0, 0.25, 0.5, 1.0, 3.0, 13.5, 14.0, 20.0]])
    x = x.astype(np.float32)
    want = oracle.activation(name, x, *params)
    got = fdx.activation(x, fdx.named_act(name, *params))
    assert (np.abs(got - want) / np.maximum(np.abs(want), 1.0)).max() <= 2e-6


def test_epilogue_launchers_reject_other_activations(fdx):
    x = np.zeros((2, 4, 4, 8), np.float32)
    with pytest.raises(fdx.FdxError, match="fuses only NONE / RELU / GELU"):
        fdx.conv2d(x, np.zeros((8, 1, 1, 8), np.float32), None, act=fdx.named_act("tanh"))


@pytest.mark.parametrize("op", ["mul", "sub", "max", "min"])
def test_broadcast_combine(fdx, oracle, op):
    say("combine", op)
    r = np.random.default_rng(13)
    a = r.standard_normal((3, 4, 5, 6)).astype(np.float32)
    for bshape in ((4, 5, 6), (1, 5, 1), (4, 1, 6)):
        b = r.standard_normal((3,) + bshape).astype(np.float32)
        want = np.stack([oracle.combine(op, a[i], b[i]) for i in range(3)])
        assert np.array_equal(fdx.broadcast_combine(op, a, b), want)
    got = fdx.broadcast_combine("add", a, a[::-1].copy(), scale=0.5)   # Average of two
    assert np.array_equal(got, ((a + a[::-1]) * np.float32(0.5)).astype(np.float32))


def test_prelu_kernel(fdx, oracle):
    r = np.random.default_rng(14)
    x = r.standard_normal((3, 5, 6, 8)).astype(np.float32)
    for shared, ashape in (([1, 2], (1, 1, 8)), ([], (5, 6, 8)), ([3], (5, 6, 1)), ([2], (5, 1, 8))):
        alpha = r.uniform(-1, 1, ashape).astype(np.float32)
        want = np.stack([oracle.prelu(x[i], alpha.reshape(-1), shared) for i in range(3)])
        assert np.array_equal(fdx.broadcast_combine("prelu", x, alpha, b_shared=True), want)


def test_model_with_activations_and_merges(fdx, oracle, modelgen):
    """Stand-alone activation layers, activations named in a layer's config (fused or not), PReLU, log_softmax, and the
    Multiply / Subtract / Average / Maximum / Minimum merges, against the oracle."""
    say("activation / merge model")
    b = modelgen.Builder("acts", 61)
    x = b.input((6, 6, 8), "x")
    c1 = b.conv2d(x, 8, 3, "c1", padding="same", activation="swish", bias_std=0.2)
    c2 = b.conv2d(x, 8, 1, "c2", activation="tanh", bias_std=0.2)
    l1 = b.activation_layer(c1, "LeakyReLU", "leaky", {"negative_slope": 0.3})
    e1 = b.activation_layer(c2, "ELU", "elu", {"alpha": 0.5})
    p1 = b.prelu(l1, "prelu", shared_axes=[1, 2])
    mul = b.merge([p1, e1], "Multiply", "mul")
    sub = b.merge([mul, c1], "Subtract", "sub")
    avg = b.merge([sub, c2, x], "Average", "avg")
    mx = b.merge([avg, p1], "Maximum", "mx")
    mn = b.merge([mx, e1], "Minimum", "mn")
    sp = b.activation(mn, "softplus_act", "softplus")
    hs = b.activation_layer(sp, "HardSigmoid", "hsig")
    th = b.activation_layer(hs, "Threshold", "thr", {"threshold": 0.55, "default_value": -1.0})
    g = b.gap(th, "gap")
    d = b.dense(g, 5, "fc", activation="log_softmax", bias_std=0.2)
    spec = b.finish([d, mn, th])
    xs = np.random.default_rng(15).standard_normal((4, 6, 6, 8)).astype(np.float32)
    js = modelgen.dumps(spec)
    ref = oracle.OracleModel(js)
    want = [ref.predict([xs[i]]) for i in range(4)]
    want = [np.stack([w[k] for w in want]) for k in range(3)]
    got = fdx.Model(js).predict([xs])
    # the threshold layer is discontinuous: an input within rounding of the threshold may fall on either side
    errs = [rel(got[0], want[0]), rel(got[1], want[1])]
    say("  rel errors:", ["%.2e" % e for e in errs])
    assert max(errs) <= TOL
    assert (np.abs(got[2] - want[2]) > 1e-4).mean() < 0.01


@pytest.mark.parametrize("shape,axes", [((6, 7, 8), [-1]), ((6, 7, 8), [1]), ((6, 7, 8), [1, 3]), ((5, 300), [2]), ((9,), [1])])
def test_rmsnorm_axes(fdx, oracle, shape, axes):
    say("rmsnorm", shape, axes)
    r = np.random.default_rng(16)
    x = (r.standard_normal((3,) + shape) * 2 + 1).astype(np.float32)
    rank = len(shape)
    n = int(np.prod([shape[(a + rank + 1 if a < 0 else a) - 1] for a in axes]))
    scale = r.standard_normal(n).astype(np.float32)
    for sc in (scale, None):
        want = np.stack([oracle.rmsnorm_axes(x[i], axes, sc, 1e-6) for i in range(3)])
        assert rel(fdx.rmsnorm_axes(x, axes, sc, 1e-6), want) <= TOL


def test_model_with_separable_conv_rmsnorm_gqa(fdx, oracle, modelgen):
    """SeparableConv2D (depthwise + pointwise), RMSNormalization, GroupedQueryAttention with and without the sigmoid
    gate and with a separate key input, against the oracle."""
    say("separable / rmsnorm / gqa model")
    b = modelgen.Builder("next_rows", 71)
    img = b.input((10, 9, 6), "img")
    s1 = b.separable_conv2d(img, 12, 3, "sep1", strides=2, padding="same", activation="relu")
    s2 = b.separable_conv2d(s1, 16, 3, "sep2", padding="valid", use_bias=False, dilation=1)
    seq = b._add("Reshape", "to_seq", {"target_shape": [9, 16]}, [s2], (9, 16))
    n1 = b.rmsnorm(seq, "rms1")
    a1 = b.gqa(n1, n1, "gqa_self", head_dim=8, num_query_heads=4, num_kv_heads=2, use_gate=True)
    r1 = b.add([seq, a1], "res1")
    n2 = b.rmsnorm(r1, "rms2", axes=(1,))
    mem = b.input((5, 16), "memory")
    a2 = b.gqa(n2, mem, "gqa_cross", head_dim=4, num_query_heads=6, num_kv_heads=1, use_bias=False, k=mem)
    out = b.dense(b.add([r1, a2], "res2"), 7, "head", bias_std=0.1)
    spec = b.finish([out, s2, a1])
    r = np.random.default_rng(17)
    xi = r.standard_normal((4, 10, 9, 6)).astype(np.float32)
    xm = r.standard_normal((4, 5, 16)).astype(np.float32)
    js = modelgen.dumps(spec)
    ref = oracle.OracleModel(js)
    want = [ref.predict([xi[i], xm[i]]) for i in range(4)]
    want = [np.stack([w[k] for w in want]) for k in range(3)]
    got = fdx.Model(js).predict([xi, xm])
    errs = [rel(g, w) for g, w in zip(got, want)]
    say("  rel errors:", ["%.2e" % e for e in errs])
    assert max(errs) <= TOL


def test_permute_crop_upsample_kernels(fdx, oracle):
    say("permute / crop / upsample kernels")
    r = np.random.default_rng(18)
    x = r.standard_normal((3, 4, 5, 6)).astype(np.float32)
    for dims in ([1, 2, 3], [3, 1, 2], [2, 1, 3], [3, 2, 1]):
        assert np.array_equal(fdx.permute(x, dims), np.transpose(x, [0] + dims))
    assert np.array_equal(fdx.permute(x[:, 0], [2, 1]), np.transpose(x[:, 0], [0, 2, 1]))
    assert np.array_equal(fdx.crop2d(x, 1, 0, 2, 1), x[:, 1:, 2:4])
    for fy, fx in ((2, 2), (3, 1), (1, 4)):
        assert np.array_equal(fdx.upsample2d(x, fy, fx), np.stack([oracle.upsample2d(x[i], fy, fx) for i in range(3)]))
        want = np.stack([oracle.upsample2d(x[i], fy, fx, True) for i in range(3)])
        assert rel(fdx.upsample2d(x, fy, fx, True), want) <= 1e-6


def test_model_with_resampling_layers(fdx, oracle, modelgen):
    """An encoder / decoder shaped model: Conv, MaxPooling, UpSampling2D (nearest and bilinear), Cropping2D, Concatenate
    skip connection, Permute, and the 1-D forms (Conv1D, ZeroPadding1D, MaxPooling1D, AveragePooling1D, UpSampling1D,
    Cropping1D) on a sequence."""
    say("resampling model")
    b = modelgen.Builder("unet_like", 81)
    img = b.input((12, 12, 3), "img")
    e1 = b.conv2d(img, 8, 3, "enc1", padding="same", activation="relu", bias_std=0.1)
    p1 = b.pool(e1, "pool1", 2, 2)
    e2 = b.conv2d(p1, 12, 3, "enc2", padding="same", activation="relu", bias_std=0.1)
    u1 = b._add("UpSampling2D", "up_nearest", {"size": [2, 2], "interpolation": "nearest"}, [e2], (12, 12, 12))
    cat = b.concatenate([u1, e1], "skip", axis=-1)
    d1 = b.conv2d(cat, 6, 3, "dec1", padding="same", bias_std=0.1)
    u2 = b._add("UpSampling2D", "up_bilinear", {"size": [2, 3], "interpolation": "bilinear"}, [d1], (24, 36, 6))
    cr = b._add("Cropping2D", "crop", {"cropping": [[2, 1], [0, 5]]}, [u2], (21, 31, 6))
    pm = b._add("Permute", "perm", {"dims": [2, 1, 3]}, [cr], (31, 21, 6))
    seq = b.input((10, 4), "seq")
    z1 = b._add("ZeroPadding1D", "pad1d", {"padding": [2, 1]}, [seq], (13, 4))
    c1 = b._add("Conv1D", "conv1d", {"filters": 6, "kernel_size": [3], "strides": [1], "dilation_rate": [1], "padding": "valid",
                                      "use_bias": True}, [z1], (11, 6))
    b.params["conv1d"] = {"weights": b.he((6, 1, 3, 4), 12), "bias": b.normal((6,), 0.1)}
    m1 = b._add("MaxPooling1D", "mp1d", {"pool_size": [2], "strides": [2], "padding": "valid"}, [c1], (5, 6))
    a1 = b._add("AveragePooling1D", "ap1d", {"pool_size": [2], "strides": [1], "padding": "same"}, [m1], (5, 6))
    us = b._add("UpSampling1D", "up1d", {"size": 3}, [a1], (15, 6))
    c1d = b._add("Cropping1D", "crop1d", {"cropping": [2, 4]}, [us], (9, 6))
    spec = b.finish([pm, c1d, u1])
    r = np.random.default_rng(19)
    xi, xs = r.standard_normal((3, 12, 12, 3)).astype(np.float32), r.standard_normal((3, 10, 4)).astype(np.float32)
    js = modelgen.dumps(spec)
    ref = oracle.OracleModel(js)
    want = [ref.predict([xi[i], xs[i]]) for i in range(3)]
    want = [np.stack([w[k] for w in want]) for k in range(3)]
    got = fdx.Model(js).predict([xi, xs])
    errs = [rel(g, w) for g, w in zip(got, want)]
    say("  rel errors:", ["%.2e" % e for e in errs])
    assert max(errs) <= TOL


def test_dilate_kernel(fdx):
    say("dilate2d kernel")
    r = np.random.default_rng(20)
    x = r.standard_normal((2, 3, 4, 5)).astype(np.float32)
    for ry, rx, trailing in ((2, 2, False), (2, 2, True), (3, 2, True), (1, 4, True), (4, 1, False), (1, 1, True)):
        ey, ex = ((ry - 1, rx - 1) if trailing and (ry, rx) != (1, 1) else (0, 0))
        want = np.zeros((2, 2 * ry + 1 + ey, 3 * rx + 1 + ex, 5), np.float32)
        want[:, ey - ey // 2::ry, ex - ex // 2::rx][:, :3, :4] = x
        assert np.array_equal(fdx.dilate2d(x, ry, rx, trailing), want), (ry, rx, trailing)


@pytest.mark.parametrize("case", [
    # h, w, cin, cout, k, strides, padding, dilation, activation
    (6, 7, 5, 8, 3, 2, "same", 1, "relu"),
    (6, 7, 5, 8, 3, 2, "valid", 1, None),
    (5, 5, 16, 32, (4, 2), (2, 3), "same", 1, None),
    (5, 6, 16, 16, 3, 1, "valid", 1, "tanh"),
    (5, 6, 3, 4, 3, 1, "same", 2, None),
    (4, 4, 6, 5, 2, 3, "same", 1, None),   # kernel smaller than the stride
    (4, 5, 6, 5, (3, 2), 2, "valid", (2, 1), "sigmoid"),
])
def test_conv2d_transpose_layer(fdx, oracle, modelgen, case):
    h, w, cin, cout, k, strides, padding, dilation, activation = case
    say("Conv2DTranspose", case)
    b = modelgen.Builder("deconv", 90)
    x = b.input((h, w, cin), "img")
    y = b.conv2d_transpose(x, cout, k, "up", strides=strides, padding=padding, dilation=dilation, activation=activation)
    js = modelgen.dumps(b.finish([y]))
    r = np.random.default_rng(21)
    xi = r.standard_normal((3, h, w, cin)).astype(np.float32)
    ref = oracle.OracleModel(js)
    want = np.stack([ref.predict([xi[i]])[0] for i in range(3)])
    got = fdx.Model(js).predict([xi])[0]
    assert got.shape == want.shape == (3,) + tuple(y.shape)
    assert rel(got, want) <= TOL


def test_decoder_model_with_transposed_convolutions(fdx, oracle, modelgen):
    """Autoencoder shape: strided convolutions down, Conv2DTranspose up with a skip Add, BatchNormalization behind a
    transposed convolution (folded at load), ZeroPadding2D in front of one, and Conv1DTranspose on a sequence."""
    say("transposed-convolution decoder model")
    b = modelgen.Builder("autoencoder", 91)
    img = b.input((16, 16, 3), "img")
    e1 = b.conv2d(img, 16, 3, "e1", strides=2, padding="same", activation="relu", bias_std=0.1)
    e2 = b.conv2d(e1, 32, 3, "e2", strides=2, padding="same", activation="relu", bias_std=0.1)
    d1 = b.conv2d_transpose(e2, 16, 3, "d1", strides=2, padding="same")
    d1 = b.batchnorm(d1, "d1_bn", random_stats=True)
    d1 = b.relu(d1, "d1_relu")
    s1 = b.add([d1, e1], "skip")
    d2 = b.conv2d_transpose(s1, 8, 4, "d2", strides=2, padding="same", activation="relu")
    zp = b._add("ZeroPadding2D", "zp", {"padding": [[1, 0], [0, 2]]}, [d2], (17, 18, 8))
    d3 = b.conv2d_transpose(zp, 3, 3, "d3", strides=1, padding="valid", activation="sigmoid")
    seq = b.input((9, 4), "seq")
    t1 = b.conv2d_transpose(seq, 6, 3, "t1", strides=2, padding="same", activation="relu")
    t2 = b.conv2d_transpose(t1, 2, 2, "t2", strides=3, padding="valid")
    spec = b.finish([d3, t2])
    r = np.random.default_rng(22)
    xi, xs = r.standard_normal((4, 16, 16, 3)).astype(np.float32), r.standard_normal((4, 9, 4)).astype(np.float32)
    js = modelgen.dumps(spec)
    ref = oracle.OracleModel(js)
    want = [ref.predict([xi[i], xs[i]]) for i in range(4)]
    want = [np.stack([w[k] for w in want]) for k in range(2)]
    got = fdx.Model(js).predict([xi, xs])
    assert got[0].shape == (4, 19, 20, 3) and got[1].shape == (4, 18 * 3 - 3 + 2, 2)
    errs = [rel(g, w) for g, w in zip(got, want)]
    say("  rel errors:", ["%.2e" % e for e in errs])
    assert max(errs) <= TOL


def test_model_with_rescaling_normalization_and_passthrough_layers(fdx, oracle, modelgen):
    """Preprocessing layers in front of a small CNN: Rescaling (one pair), Normalization on the channel axis (plain
    and inverted), axis-less Normalization, augmentation layers that pass their input through; the Normalization behind
    a convolution folds into it, the one behind an activation runs as its own launch."""
    say("Rescaling / Normalization / passthrough model")
    b = modelgen.Builder("prep_cnn", 92)
    img = b.input((12, 10, 3), "img")
    x = b.rescaling(img, "scale", 1 / 127.5, -1.0)
    x = b._add("RandomFlip", "flip", {}, [x], x.shape)
    x = b._add("RandAugment", "ra", {}, [x], x.shape)
    x = b.normalization(x, "norm", axis=-1)
    c = b.conv2d(x, 8, 3, "c1", padding="same", bias_std=0.1)
    c = b.normalization(c, "norm_folded", axis=-1)
    c = b.relu(c, "r1")
    c = b.normalization(c, "norm_alone", axis=3, invert=True)
    c = b.normalization(c, "norm_all", axis=None)
    seq = b.input((7, 6), "seq")
    s = b.normalization(seq, "norm_seq", axis=-1)
    s = b.rescaling(s, "scale_seq", -0.5, 3.0)
    js = modelgen.dumps(b.finish([c, s]))
    r = np.random.default_rng(23)
    xi = r.uniform(0, 255, (5, 12, 10, 3)).astype(np.float32)
    xs = r.standard_normal((5, 7, 6)).astype(np.float32)
    ref = oracle.OracleModel(js)
    want = [ref.predict([xi[i], xs[i]]) for i in range(5)]
    want = [np.stack([w[k] for w in want]) for k in range(2)]
    got = fdx.Model(js).predict([xi, xs])
    for g, w in zip(got, want):
        assert g.shape == w.shape
        assert rel(g, w) <= TOL
    # on another axis than the last the launch is refused, not approximated
    b2 = modelgen.Builder("prep_bad", 93)
    x2 = b2.input((4, 5, 6), "x")
    y2 = b2.normalization(x2, "n", axis=2)
    with pytest.raises(Exception, match="last axis"):
        fdx.Model(modelgen.dumps(b2.finish([y2]))).predict([np.zeros((1, 4, 5, 6), np.float32)])
