"""Randomly assembled models against the oracle: image graphs (convolutions of every kind, normalisation, pooling,
activations, merges with skip connections, resampling) and sequence graphs (Dense, EinsumDense, LayerNormalization /
RMSNormalization, attention, merges), each from a seed, each run batched on the GPU and sample by sample through the
oracle.  What the fixed-architecture tests cannot cover is the load-time fusion meeting arbitrary neighbours: a folded
BatchNormalization behind a depthwise convolution that also feeds a skip, an activation with two consumers, a
ZeroPadding2D in front of a pooling layer, an Add whose operands come from the same producer.
Tolerance per output: max|gpu - ref| / max|ref| <= 1e-4."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-4

ACTS = ["relu", "relu6", "tanh", "sigmoid", "swish", "gelu", "elu", "softplus", "hard_sigmoid", "selu", "linear"]


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    assert a.shape == b.shape, (a.shape, b.shape)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def image_graph(modelgen, seed):
    r = np.random.default_rng(seed)
    b = modelgen.Builder("rand_img_%d" % seed, seed)
    h, w, c = int(r.integers(9, 20)), int(r.integers(9, 20)), int(r.choice([3, 4, 8, 16]))
    x = b.input((h, w, c), "img")
    live = [x]       # tensors that may still be consumed
    n = [0]

    def name(kind):
        n[0] += 1
        return "%s_%d" % (kind, n[0])

    def same_shape_partner(t):
        for u in live[::-1]:
            if u is not t and tuple(u.shape) == tuple(t.shape):
                return u
        return None

    for _ in range(int(r.integers(6, 14))):
        t = live[int(r.integers(max(0, len(live) - 3), len(live)))]
        hh, ww, cc = t.shape
        op = r.choice(["conv", "conv", "dw", "sep", "bn", "act", "pool", "zpad", "add", "concat", "up", "tconv", "prelu", "mul"])
        act = r.choice(ACTS) if r.random() < 0.6 else None
        pad = str(r.choice(["same", "valid"]))
        k = int(r.choice([1, 2, 3, 5]))
        s = int(r.choice([1, 1, 2]))
        if op in ("conv", "dw", "sep", "pool", "tconv") and pad == "valid" and (hh < k + 1 or ww < k + 1):
            pad = "same"
        if op == "conv":
            d = int(r.choice([1, 1, 2])) if s == 1 else 1
            if pad == "valid" and (hh <= (k - 1) * d + 1 or ww <= (k - 1) * d + 1):
                d = 1
            y = b.conv2d(t, int(r.choice([4, 8, 16, 24, 64])), k, name("conv"), strides=s, padding=pad, activation=act,
                         dilation=d, use_bias=bool(r.random() < 0.8), bias_std=0.2)
        elif op == "dw":
            y = b.depthwise_conv2d(t, int(r.choice([3, 5])) if min(hh, ww) > 5 else 3, name("dw"), strides=s, padding="same",
                                   use_bias=bool(r.random() < 0.5), bias_std=0.2)
        elif op == "sep":
            y = b.separable_conv2d(t, int(r.choice([8, 16, 32])), 3, name("sep"), strides=s, padding="same", activation=act)
        elif op == "bn":
            y = b.batchnorm(t, name("bn"), random_stats=True)
        elif op == "act":
            y = b.activation(t, name("act"), str(r.choice(ACTS[:-1])))
        elif op == "pool":
            y = b.pool(t, name("pool"), 2 if min(hh, ww) < 6 else int(r.choice([2, 3])), int(r.choice([1, 2])), padding=pad,
                       kind=str(r.choice(["max", "avg"])))
        elif op == "zpad":
            y = b.zero_pad(t, name("zpad"), ((int(r.integers(0, 3)), int(r.integers(0, 3))), (int(r.integers(0, 3)), int(r.integers(0, 3)))))
        elif op in ("add", "mul"):
            u = same_shape_partner(t)
            if u is None:
                u = b.conv2d(t, cc, 1, name("proj"), bias_std=0.2)
            y = b.add([t, u], name("add")) if op == "add" else b.merge([t, u], str(r.choice(["Multiply", "Maximum", "Average", "Subtract"])), name("merge"))
        elif op == "concat":
            u = same_shape_partner(t)
            y = b.concatenate([t, u if u is not None else t], name("cat"), axis=-1)
        elif op == "up":
            if hh * ww > 400:
                continue
            f = [int(r.choice([1, 2])), int(r.choice([2, 3]))]
            y = b._add("UpSampling2D", name("up"), {"size": f, "interpolation": str(r.choice(["nearest", "bilinear"]))}, [t],
                       (hh * f[0], ww * f[1], cc))
        elif op == "tconv":
            if hh * ww > 300:
                continue
            y = b.conv2d_transpose(t, int(r.choice([4, 8, 16])), int(r.choice([2, 3, 4])), name("tconv"), strides=int(r.choice([1, 2])),
                                   padding=pad, activation=act)
        else:
            y = b.prelu(t, name("prelu"), shared_axes=[[1, 2], None, [1], [1, 2, 3]][int(r.integers(0, 4))])
        if min(y.shape[0], y.shape[1]) < 2:
            continue
        live.append(y)
    outs = [live[-1]]
    if len(live) > 3 and r.random() < 0.7:
        outs.append(live[int(r.integers(1, len(live) - 1))])
    if r.random() < 0.5:
        g = b.gap(live[-1], name("gap"))
        outs.append(b.dense(g, 7, name("fc"), activation="softmax", bias_std=0.2))
    return b.finish(outs), [(h, w, c)]


def sequence_graph(modelgen, seed):
    r = np.random.default_rng(seed)
    b = modelgen.Builder("rand_seq_%d" % seed, seed)
    t_len, d = int(r.integers(3, 40)), int(r.choice([8, 16, 32, 64]))
    x = b.input((t_len, d), "seq")
    n = [0]

    def name(kind):
        n[0] += 1
        return "%s_%d" % (kind, n[0])

    cur = x
    outs = []
    for _ in range(int(r.integers(4, 10))):
        op = r.choice(["dense", "ln", "rms", "mha", "gqa", "ffn", "einsum", "act", "conv1d"])
        if op == "dense":
            y = b.dense(cur, d, name("dense"), activation=str(r.choice(ACTS)), bias_std=0.2)
        elif op == "ln":
            y = b.layernorm(cur, name("ln"), random_affine=True)
        elif op == "rms":
            y = b.rmsnorm(cur, name("rms"))
        elif op == "mha":
            heads = int(r.choice([1, 2, 4]))
            kd = int(r.choice([4, 8, 32, 64]))
            y = b.add([cur, b.mha(cur, cur, name("mha"), heads, kd, value_dim=kd if r.random() < 0.7 else int(r.choice([4, 16])),
                                  use_bias=bool(r.random() < 0.7), std=0.2, bias_std=0.1)], name("res"))
        elif op == "gqa":
            hd, hq = int(r.choice([4, 8, 32])), int(r.choice([2, 4]))
            y = b.add([cur, b.gqa(cur, cur, name("gqa"), hd, hq, int(r.choice([1, 2])), use_bias=bool(r.random() < 0.5),
                                  use_gate=bool(r.random() < 0.5))], name("res"))
        elif op == "ffn":
            hid = b.dense(cur, 2 * d, name("ffn_in"), activation="gelu", bias_std=0.2)
            y = b.add([cur, b.dense(hid, d, name("ffn_out"), bias_std=0.2)], name("res"))
        elif op == "einsum":
            y = b.einsum_dense(cur, "abc,cd->abd", (d, d), name("ein"), bias_axes="d", activation=str(r.choice(["relu", "tanh", "linear"])))
        elif op == "act":
            y = b.activation(cur, name("act"), str(r.choice(ACTS[:-1])))
        else:
            k = int(r.choice([1, 3]))
            y = b._add("Conv1D", name("c1d"), {"filters": d, "kernel_size": [k], "strides": [1], "dilation_rate": [1],
                                               "padding": str(r.choice(["same", "causal"])), "use_bias": True}, [cur], (t_len, d))
            b.params[y.layer] = {"weights": b.he((d, 1, k, d), k * d), "bias": b.normal((d,), 0.2)}
        if r.random() < 0.25:
            outs.append(y)
        cur = y
    outs.append(cur)
    return b.finish(outs), [(t_len, d)]


@pytest.mark.parametrize("seed", range(64))
def test_random_image_graph(fdx, oracle, modelgen, seed):
    spec, shapes = image_graph(modelgen, 1000 + seed)
    print("random image graph", seed, [l["class_name"] for l in spec["architecture"]["config"]["layers"]], flush=True)
    js = modelgen.dumps(spec)
    r = np.random.default_rng(seed)
    xs = [r.standard_normal((3,) + s).astype(np.float32) for s in shapes]
    ref = oracle.OracleModel(js)
    want = [ref.predict([x[i] for x in xs]) for i in range(3)]
    want = [np.stack([w[k] for w in want]) for k in range(len(want[0]))]
    got = fdx.Model(js).predict(xs)
    errs = [rel(g, w) for g, w in zip(got, want)]
    assert max(errs) <= TOL, errs


@pytest.mark.parametrize("seed", range(48))
def test_random_sequence_graph(fdx, oracle, modelgen, seed):
    spec, shapes = sequence_graph(modelgen, 2000 + seed)
    print("random sequence graph", seed, [l["class_name"] for l in spec["architecture"]["config"]["layers"]], flush=True)
    js = modelgen.dumps(spec)
    r = np.random.default_rng(seed)
    xs = [r.standard_normal((3,) + s).astype(np.float32) for s in shapes]
    ref = oracle.OracleModel(js)
    want = [ref.predict([x[i] for x in xs]) for i in range(3)]
    want = [np.stack([w[k] for w in want]) for k in range(len(want[0]))]
    got = fdx.Model(js).predict(xs)
    errs = [rel(g, w) for g, w in zip(got, want)]
    assert max(errs) <= TOL, errs
