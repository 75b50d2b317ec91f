"""Writers for frugally-deep's converted-JSON model format (numpy only).

The reference's exporter (keras_export/convert_model.py:971-1001) needs Keras; this
module emits the same file layout directly -- exactly the fields the loader
dereferences (include/fdeep/model.hpp:226-267, include/fdeep/import_model.hpp) -- for
seeded, randomly initialised networks of the benchmark shapes:

  small_cnn()      32x32x3 conv/pool/conv/GAP/dense(softmax)
  resnet50()       keras-applications ResNet50 v1 layout
  mobilenet_v2()   keras-applications MobileNetV2 layout
  encoder()        pre-LayerNorm transformer encoder stack
  gpt2()           GPT-2-small-shaped decoder (ids + positions inputs)

Weight axis orders follow convert_model.py:197-206 (conv [Cout][kh][kw][Cin],
depthwise [C][kh][kw]), :457-469 (dense [in][out]), :492-499 (embedding [vocab][dim]),
:600-607 (MultiHeadAttention q_w,q_b,k_w,k_b,v_w,v_b,o_w,o_b with their Keras shapes).
"""
import base64
import json

import numpy as np

CHUNK = 1024  # characters per base64 string, convert_model.py:187-194


def encode_floats(arr):
    """fp32 little-endian -> list of base64 strings of at most 1024 chars."""
    b = base64.b64encode(np.ascontiguousarray(arr, dtype="<f4").tobytes()).decode("ascii")
    return [b[i:i + CHUNK] for i in range(0, len(b), CHUNK)] or [""]


def _encode_floats_json(arr):
    """Same as json.dumps(encode_floats(arr)) but vectorised for 100 MB+ tensors."""
    b = base64.b64encode(np.ascontiguousarray(arr, dtype="<f4").tobytes())
    n, rem = divmod(len(b), CHUNK)
    parts = [b"["]
    if n:
        body = np.empty((n, CHUNK + 3), np.uint8)
        body[:, 0] = ord('"')
        body[:, 1:CHUNK + 1] = np.frombuffer(b, np.uint8, n * CHUNK).reshape(n, CHUNK)
        body[:, CHUNK + 1] = ord('"')
        body[:, CHUNK + 2] = ord(",")
        parts.append(body.tobytes()[:-1] if not rem else body.tobytes())
    if rem or not n:
        parts.append(b'"' + b[n * CHUNK:] + b'"')
    parts.append(b"]")
    return b"".join(parts)


class T:
    """Symbolic tensor: producing layer name + shape without batch dim."""

    def __init__(self, layer, shape):
        self.layer = layer
        self.shape = tuple(shape)


def _kt(t):
    return {"class_name": "__keras_tensor__",
            "config": {"keras_history": [t.layer, getattr(t, "node", 0), getattr(t, "tensor", 0)]}}


class Builder:
    def __init__(self, name, seed=0):
        self.name = name
        self.rng = np.random.default_rng(seed)
        self.layers = []
        self.params = {}
        self.inputs = []
        self.names = set()

    # ---- helpers
    def _add(self, cls, name, cfg, ins, shape, merge=False):
        assert name not in self.names, name
        self.names.add(name)
        args = [_kt(t) for t in ins]
        nodes = [] if cls == "InputLayer" else [{"args": [args] if merge else args, "kwargs": {}}]
        self.layers.append({"class_name": cls, "name": name, "config": cfg, "inbound_nodes": nodes})
        return T(name, shape)

    def he(self, shape, fan_in):
        return (self.rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)

    def normal(self, shape, std):
        return (self.rng.standard_normal(shape) * std).astype(np.float32)

    @staticmethod
    def _win(n, k, s, padding):
        if padding == "same":
            return -(-n // s)
        return -(-(n - k + 1) // s)

    # ---- layers
    def input(self, shape, name=None):
        name = name or "input_%d" % len(self.inputs)
        t = self._add("InputLayer", name, {"batch_shape": [None] + list(shape)}, [], shape)
        self.inputs.append(t)
        return t

    def conv2d(self, x, filters, k, name, strides=1, padding="valid", use_bias=True, activation=None,
               dilation=1, init="he", bias_std=0.0):
        kh, kw = (k, k) if isinstance(k, int) else k
        sy, sx = (strides, strides) if isinstance(strides, int) else strides
        dy, dx = (dilation, dilation) if isinstance(dilation, int) else dilation
        h, w, cin = x.shape
        fan_in = kh * kw * cin
        wts = self.he((filters, kh, kw, cin), fan_in) if init == "he" else self.normal((filters, kh, kw, cin), init)
        self.params[name] = {"weights": wts}
        if use_bias:
            self.params[name]["bias"] = self.normal((filters,), bias_std) if bias_std else np.zeros(filters, np.float32)
        cfg = {"filters": filters, "kernel_size": [kh, kw], "strides": [sy, sx], "dilation_rate": [dy, dx],
               "padding": padding, "use_bias": use_bias}
        if activation is not None:
            cfg["activation"] = activation
        oh = self._win(h, (kh - 1) * dy + 1, sy, padding)
        ow = self._win(w, (kw - 1) * dx + 1, sx, padding)
        return self._add("Conv2D", name, cfg, [x], (oh, ow, filters))

    def conv2d_transpose(self, x, filters, k, name, strides=1, padding="valid", use_bias=True, activation=None, dilation=1,
                         bias_std=0.2):
        """Conv2DTranspose (Conv1DTranspose for a rank-2 input); weights in the exporter's [filters][kh][kw][cin] order."""
        one_d = len(x.shape) == 2
        kh, kw = (k, k) if isinstance(k, int) else k
        sy, sx = (strides, strides) if isinstance(strides, int) else strides
        dy, dx = (dilation, dilation) if isinstance(dilation, int) else dilation
        h, w, cin = (1,) + tuple(x.shape) if one_d else x.shape
        if one_d:
            kh, sy, dy = 1, 1, 1
        self.params[name] = {"weights": self.he((filters, kh, kw, cin), kh * kw * cin)}
        if use_bias:
            self.params[name]["bias"] = self.normal((filters,), bias_std)
        cfg = {"filters": filters, "padding": padding, "use_bias": use_bias,
               "kernel_size": [kw] if one_d else [kh, kw], "strides": [sx] if one_d else [sy, sx],
               "dilation_rate": [dx] if one_d else [dy, dx]}
        if activation is not None:
            cfg["activation"] = activation
        if padding == "same":
            oh, ow = h * sy, w * sx
        else:
            oh, ow = (h - 1) * sy + (kh - 1) * dy + 1, (w - 1) * sx + (kw - 1) * dx + 1
        return self._add("Conv1DTranspose" if one_d else "Conv2DTranspose", name, cfg, [x], (ow, filters) if one_d else (oh, ow, filters))

    def depthwise_conv2d(self, x, k, name, strides=1, padding="valid", use_bias=False, dilation=1, bias_std=0.0):
        kh, kw = (k, k) if isinstance(k, int) else k
        sy, sx = (strides, strides) if isinstance(strides, int) else strides
        dy, dx = (dilation, dilation) if isinstance(dilation, int) else dilation
        h, w, c = x.shape
        self.params[name] = {"slice_weights": self.he((c, kh, kw), kh * kw)}
        if use_bias:
            self.params[name]["bias"] = self.normal((c,), bias_std) if bias_std else np.zeros(c, np.float32)
        cfg = {"kernel_size": [kh, kw], "strides": [sy, sx], "dilation_rate": [dy, dx], "padding": padding,
               "use_bias": use_bias, "depth_multiplier": 1}
        oh = self._win(h, (kh - 1) * dy + 1, sy, padding)
        ow = self._win(w, (kw - 1) * dx + 1, sx, padding)
        return self._add("DepthwiseConv2D", name, cfg, [x], (oh, ow, c))

    def batchnorm(self, x, name, eps=1.001e-5, random_stats=False):
        c = x.shape[-1]
        if random_stats:
            p = {"moving_mean": self.normal((c,), 0.1), "moving_variance": (0.5 + self.rng.random(c)).astype(np.float32),
                 "gamma": (0.5 + self.rng.random(c)).astype(np.float32), "beta": self.normal((c,), 0.1)}
        else:
            p = {"moving_mean": np.zeros(c, np.float32), "moving_variance": np.ones(c, np.float32),
                 "gamma": np.ones(c, np.float32), "beta": np.zeros(c, np.float32)}
        self.params[name] = p
        cfg = {"axis": len(x.shape), "epsilon": eps, "center": True, "scale": True}
        return self._add("BatchNormalization", name, cfg, [x], x.shape)

    def rescaling(self, x, name, scale, offset=0.0):
        return self._add("Rescaling", name, {"scale": float(scale), "offset": float(offset)}, [x], x.shape)

    def normalization(self, x, name, axis=-1, invert=False):
        """Keras Normalization with random statistics; axis None = one mean / variance for the whole tensor."""
        n = 1 if axis is None else x.shape[axis if axis < 0 else axis - 1]
        self.params[name] = {"mean": self.normal((n,), 0.5), "variance": (0.25 + self.rng.random(n)).astype(np.float32)}
        cfg = {"axis": [] if axis is None else [axis], "invert": bool(invert)}
        return self._add("Normalization", name, cfg, [x], x.shape)

    def layernorm(self, x, name, eps=1e-3, random_affine=False):
        d = x.shape[-1]
        if random_affine:
            p = {"gamma": (0.5 + self.rng.random(d)).astype(np.float32), "beta": self.normal((d,), 0.1)}
        else:
            p = {"gamma": np.ones(d, np.float32), "beta": np.zeros(d, np.float32)}
        self.params[name] = p
        return self._add("LayerNormalization", name, {"axis": [-1], "epsilon": eps, "center": True, "scale": True},
                         [x], x.shape)

    def relu(self, x, name, max_value=None):
        cfg = {"max_value": max_value, "negative_slope": 0.0, "threshold": 0.0}
        return self._add("ReLU", name, cfg, [x], x.shape)

    def activation(self, x, name, kind):
        return self._add("Activation", name, {"activation": kind}, [x], x.shape)

    def separable_conv2d(self, x, filters, k, name, strides=1, padding="valid", use_bias=True, activation=None, dilation=1):
        h, w, cin = x.shape
        self.params[name] = {"slice_weights": self.he((cin, k, k), k * k), "stack_weights": self.he((filters, 1, 1, cin), cin)}
        if use_bias:
            self.params[name]["bias"] = self.normal((filters,), 0.2)
        cfg = {"filters": filters, "kernel_size": [k, k], "strides": [strides, strides], "dilation_rate": [dilation, dilation],
               "padding": padding, "use_bias": use_bias}
        if activation is not None:
            cfg["activation"] = activation
        ek = (k - 1) * dilation + 1
        return self._add("SeparableConv2D", name, cfg, [x], (self._win(h, ek, strides, padding), self._win(w, ek, strides, padding), filters))

    def rmsnorm(self, x, name, axes=(-1,), eps=1e-6):
        rank = len(x.shape)
        pos = sorted(set(a + rank + 1 if a < 0 else a for a in axes))
        n = int(np.prod([x.shape[a - 1] for a in pos]))
        self.params[name] = {"scale": (0.5 + self.rng.random(n)).astype(np.float32)}
        return self._add("RMSNormalization", name, {"axis": list(axes), "epsilon": eps}, [x], x.shape)

    def gqa(self, q, v, name, head_dim, num_query_heads, num_kv_heads, use_bias=True, use_gate=False, k=None, std=0.2):
        """GroupQueryAttention; weights in Keras order Q, K, [Gate], V, Out, each bias right after its kernel."""
        d = q.shape[-1]
        shapes, vals = [], []

        def put(kshape, bshape):
            shapes.append(list(kshape))
            vals.append(self.normal(kshape, std))
            if use_bias:
                shapes.append(list(bshape))
                vals.append(self.normal(bshape, 0.2))

        put((d, num_query_heads, head_dim), (num_query_heads, head_dim))
        put((d, num_kv_heads, head_dim), (num_kv_heads, head_dim))
        if use_gate:
            put((d, num_query_heads, head_dim), (num_query_heads, head_dim))
        put((d, num_kv_heads, head_dim), (num_kv_heads, head_dim))
        put((num_query_heads, head_dim, d), (d,))
        self.params[name] = {"weight_shapes": shapes, "weights": vals}
        cfg = {"head_dim": head_dim, "num_query_heads": num_query_heads, "num_key_value_heads": num_kv_heads,
               "use_bias": use_bias, "use_gate": use_gate}
        return self._add("GroupedQueryAttention", name, cfg, [q, v] + ([k] if k is not None else []), q.shape[:-1] + (d,))

    def activation_layer(self, x, cls, name, cfg=None):
        """A layer class that is one element-wise activation (LeakyReLU, ELU, Softmax, Threshold, ...)."""
        return self._add(cls, name, dict(cfg or {}), [x], x.shape)

    def prelu(self, x, name, shared_axes=None):
        dims = [1 if (shared_axes and a + 1 in shared_axes) else d for a, d in enumerate(x.shape)]
        self.params[name] = {"alpha": self.rng.uniform(-0.5, 0.9, int(np.prod(dims))).astype(np.float32)}
        return self._add("PReLU", name, {"shared_axes": list(shared_axes) if shared_axes else None}, [x], x.shape)

    def merge(self, xs, cls, name):
        """Multiply / Subtract / Average / Maximum / Minimum (same shape rules as Add)."""
        t = self.add(xs, name)
        self.layers[-1]["class_name"] = cls
        return t

    def zero_pad(self, x, name, pad):
        (pt, pb), (pl, pr) = pad
        h, w, c = x.shape
        return self._add("ZeroPadding2D", name, {"padding": [[pt, pb], [pl, pr]]}, [x], (h + pt + pb, w + pl + pr, c))

    def pool(self, x, name, size, strides, padding="valid", kind="max"):
        h, w, c = x.shape
        cfg = {"pool_size": [size, size], "strides": [strides, strides], "padding": padding}
        shape = (self._win(h, size, strides, padding), self._win(w, size, strides, padding), c)
        return self._add("MaxPooling2D" if kind == "max" else "AveragePooling2D", name, cfg, [x], shape)

    def gap(self, x, name, kind="avg"):
        cls = "GlobalAveragePooling2D" if kind == "avg" else "GlobalMaxPooling2D"
        return self._add(cls, name, {"keepdims": False}, [x], (x.shape[-1],))

    def layernorm_axes(self, x, name, axes, eps=1e-3, center=True, scale=True):
        """LayerNormalization over arbitrary axes (1-based in the sample's rank, negative from the end);
        gamma / beta are shaped like the normalised axes in storage order."""
        rank = len(x.shape)
        pos = sorted(set(a + rank + 1 if a < 0 else a for a in axes))
        n = int(np.prod([x.shape[a - 1] for a in pos]))
        p = {}
        if scale:
            p["gamma"] = (0.5 + self.rng.random(n)).astype(np.float32)
        if center:
            p["beta"] = self.normal((n,), 0.3)
        self.params[name] = p
        return self._add("LayerNormalization", name, {"axis": list(axes), "epsilon": eps, "center": center, "scale": scale},
                         [x], x.shape)

    def add(self, xs, name):
        rank = max(len(t.shape) for t in xs)
        shape = [1] * rank
        for t in xs:  # size-1 broadcasting on right-aligned axes
            for i, d in enumerate(reversed(t.shape)):
                cur = shape[rank - 1 - i]
                shape[rank - 1 - i] = None if d is None or cur is None else max(cur, d)  # None = variable extent
        return self._add("Add", name, {}, xs, tuple(shape), merge=True)

    def concatenate(self, xs, name, axis=-1):
        rank = len(xs[0].shape)
        a = (axis + rank + 1 if axis < 0 else axis) - 1
        shape = list(xs[0].shape)
        shape[a] = sum(t.shape[a] for t in xs)
        return self._add("Concatenate", name, {"axis": axis}, xs, tuple(shape), merge=True)

    def einsum_dense(self, x, equation, kernel_shape, name, bias_axes=None, output_shape=None, activation=None, std=None):
        """EinsumDense; the bias is stored over the bias axes in rhs order whatever the order of the
        bias_axes string (include/fdeep/layers/einsum_dense_layer.hpp:197-222)."""
        lhs, rest = equation.split(",")
        ker, rhs = rest.split("->")
        size = dict(zip(ker, kernel_shape))
        for c, d in zip(lhs[len(lhs) - len(x.shape):], x.shape):
            assert size.setdefault(c, d) == d, (equation, c)
        summed = [c for c in lhs if c not in rhs and c in ker]
        fan_in = int(np.prod([size[c] for c in summed])) if summed else 1
        kernel = self.he(tuple(kernel_shape), fan_in) if std is None else self.normal(tuple(kernel_shape), std)
        p = {"kernel": kernel, "kernel_shape": [int(v) for v in kernel_shape]}
        if bias_axes:
            bshape = [size[c] for c in rhs if c in bias_axes]
            p["bias"] = self.normal(tuple(bshape), 0.5)
            p["bias_shape"] = [int(v) for v in bshape]
        self.params[name] = p
        out_shape = tuple(size[c] for c in rhs[1:])
        cfg = {"equation": equation, "bias_axes": bias_axes,
               "output_shape": list(output_shape) if output_shape is not None else list(out_shape)}
        if activation is not None:
            cfg["activation"] = activation
        return self._add("EinsumDense", name, cfg, [x], out_shape)

    def nested(self, inner_spec, xs, name):
        """Applies a finished model (Builder.finish) as one Functional layer; its parameters are stored under
        "<name>_<inner layer>" (keras_export/convert_model.py:907-918).  Returns one tensor per inner output."""
        arch = inner_spec["architecture"]
        for lname, prm in inner_spec["trainable_params"].items():
            self.params[name + "_" + lname] = prm
        assert name not in self.names, name
        self.names.add(name)
        node = {"args": [_kt(t) for t in xs], "kwargs": {}}
        self.layers.append({"class_name": "Functional", "name": name, "config": arch["config"], "inbound_nodes": [node]})
        outs = []
        for i, shp in enumerate(inner_spec["output_shapes"]):
            t = T(name, shp)
            t.node, t.tensor = 1, i  # Keras numbers the first outer call of a nested model as node 1
            outs.append(t)
        return outs

    def dense(self, x, units, name, activation=None, use_bias=True, init="he", bias_std=0.0):
        n_in = x.shape[-1]
        w = self.he((n_in, units), n_in) if init == "he" else self.normal((n_in, units), init)
        self.params[name] = {"weights": w}
        if use_bias:
            self.params[name]["bias"] = self.normal((units,), bias_std) if bias_std else np.zeros(units, np.float32)
        cfg = {"units": units, "use_bias": use_bias}
        if activation is not None:
            cfg["activation"] = activation
        return self._add("Dense", name, cfg, [x], x.shape[:-1] + (units,))

    def embedding(self, x, input_dim, output_dim, name, std=0.02):
        self.params[name] = {"weights": self.normal((input_dim, output_dim), std)}
        return self._add("Embedding", name, {"input_dim": input_dim, "output_dim": output_dim}, [x],
                         (x.shape[0], output_dim))

    def mha(self, q, v, name, heads, key_dim, value_dim=None, use_bias=True, std=0.02, k=None, bias_std=0.0):
        value_dim = value_dim or key_dim
        d, dout = q.shape[-1], q.shape[-1]
        shapes, vals = [], []

        def put(shape, is_bias):
            shapes.append(list(shape))
            vals.append(self.normal(shape, bias_std) if is_bias and bias_std else
                        (np.zeros(shape, np.float32) if is_bias else self.normal(shape, std)))

        for dim in (key_dim, key_dim, value_dim):
            put((d, heads, dim), False)
            if use_bias:
                put((heads, dim), True)
        put((heads, value_dim, dout), False)
        if use_bias:
            put((dout,), True)
        self.params[name] = {"weight_shapes": shapes, "weights": vals}
        cfg = {"num_heads": heads, "key_dim": key_dim, "value_dim": value_dim, "use_bias": use_bias}
        ins = [q, v] + ([k] if k is not None else [])
        return self._add("MultiHeadAttention", name, cfg, ins, q.shape[:-1] + (dout,))

    # ---- output
    def finish(self, outputs, tests=None):
        spec = {
            "image_data_format": "channels_last",
            "input_shapes": [list(t.shape) for t in self.inputs],
            "output_shapes": [list(t.shape) for t in outputs],
            "architecture": {"class_name": "Functional", "config": {
                "name": self.name, "layers": self.layers,
                "input_layers": [[t.layer, 0, 0] for t in self.inputs],
                "output_layers": [[t.layer, getattr(t, "node", 0), getattr(t, "tensor", 0)] for t in outputs]}},
            "trainable_params": self.params,
            "hash": "",
        }
        if tests is not None:
            spec["tests"] = tests
        return spec


def dumps(spec):
    """Serialise a model spec (as returned by Builder.finish) to converted-JSON bytes."""
    head = {k: v for k, v in spec.items() if k not in ("trainable_params", "tests")}
    out = [json.dumps(head)[:-1].encode(), b', "trainable_params": {']
    first_layer = True
    for lname, params in spec["trainable_params"].items():
        out.append((b"" if first_layer else b", ") + json.dumps(lname).encode() + b": {")
        first_layer = False
        first = True
        for key, val in params.items():
            out.append((b"" if first else b", ") + json.dumps(key).encode() + b": ")
            first = False
            if key == "weight_shapes" or key.endswith("_shape"):
                out.append(json.dumps(val).encode())
            elif isinstance(val, list):  # list of tensors (MultiHeadAttention)
                out.append(b"[" + b", ".join(_encode_floats_json(v) for v in val) + b"]")
            else:
                out.append(_encode_floats_json(val))
        out.append(b"}")
    out.append(b"}")
    if spec.get("tests") is not None:
        tests = []
        for t in spec["tests"]:
            enc = lambda xs: [{"shape": list(np.shape(x)), "values": encode_floats(x)} for x in xs]
            tests.append({"inputs": enc(t["inputs"]), "outputs": enc(t["outputs"])})
        out.append(b', "tests": ' + json.dumps(tests).encode())
    out.append(b"}")
    return b"".join(out)


# ------------------------------------------------------------------ the five configurations

def small_cnn(seed=1):
    """Input 32x32x3 -> Conv 3x3x16 same relu -> MaxPool 2 -> Conv 3x3x32 valid relu -> GAP ->
    Dense 10 softmax; He-normal weights, zero biases."""
    b = Builder("small_cnn", seed)
    x = b.input((32, 32, 3), "image")
    x = b.conv2d(x, 16, 3, "conv1", padding="same", activation="relu")
    x = b.pool(x, "pool1", 2, 2)
    x = b.conv2d(x, 32, 3, "conv2", padding="valid", activation="relu")
    x = b.gap(x, "gap")
    x = b.dense(x, 10, "fc", activation="softmax")
    return b.finish([x])


def resnet50(seed=2, input_size=224, width=64, blocks=(3, 4, 6, 3), classes=1000, random_bn=False):
    """keras-applications ResNet50 v1: conv stem, bottleneck stages, BN after every conv, GAP, FC softmax."""
    b = Builder("resnet50", seed)
    x = b.input((input_size, input_size, 3), "input_image")
    x = b.zero_pad(x, "conv1_pad", ((3, 3), (3, 3)))
    x = b.conv2d(x, width, 7, "conv1_conv", strides=2)
    x = b.batchnorm(x, "conv1_bn", random_stats=random_bn)
    x = b.relu(x, "conv1_relu")
    x = b.zero_pad(x, "pool1_pad", ((1, 1), (1, 1)))
    x = b.pool(x, "pool1_pool", 3, 2)

    def block(x, filters, name, stride=1, conv_shortcut=True):
        if conv_shortcut:
            sc = b.conv2d(x, 4 * filters, 1, name + "_0_conv", strides=stride)
            sc = b.batchnorm(sc, name + "_0_bn", random_stats=random_bn)
        else:
            sc = x
        y = b.conv2d(x, filters, 1, name + "_1_conv", strides=stride)
        y = b.batchnorm(y, name + "_1_bn", random_stats=random_bn)
        y = b.relu(y, name + "_1_relu")
        y = b.conv2d(y, filters, 3, name + "_2_conv", padding="same")
        y = b.batchnorm(y, name + "_2_bn", random_stats=random_bn)
        y = b.relu(y, name + "_2_relu")
        y = b.conv2d(y, 4 * filters, 1, name + "_3_conv")
        y = b.batchnorm(y, name + "_3_bn", random_stats=random_bn)
        y = b.add([sc, y], name + "_add")
        return b.relu(y, name + "_out")

    for si, (n, f) in enumerate(zip(blocks, (width, 2 * width, 4 * width, 8 * width))):
        for bi in range(n):
            x = block(x, f, "conv%d_block%d" % (si + 2, bi + 1), stride=(1 if si == 0 else 2) if bi == 0 else 1,
                      conv_shortcut=bi == 0)
    x = b.gap(x, "avg_pool")
    x = b.dense(x, classes, "predictions", activation="softmax")
    return b.finish([x])


def mobilenet_v2(seed=3, input_size=224, alpha=1.0, classes=1000, random_bn=False, truncate=None):
    """keras-applications MobileNetV2: inverted residuals with DepthwiseConv2D 3x3 and ReLU6."""
    def mk(v, divisor=8):
        nv = max(divisor, int(v + divisor / 2) // divisor * divisor)
        return nv + divisor if nv < 0.9 * v else nv

    b = Builder("mobilenetv2", seed)
    x = b.input((input_size, input_size, 3), "input_image")
    first = mk(32 * alpha)
    x = b.conv2d(x, first, 3, "Conv1", strides=2, padding="same", use_bias=False)
    x = b.batchnorm(x, "bn_Conv1", eps=1e-3, random_stats=random_bn)
    x = b.relu(x, "Conv1_relu", 6.0)

    def inv_res(x, expansion, stride, filters, block_id):
        cin = x.shape[-1]
        pw = mk(int(filters * alpha))
        prefix = "block_%d_" % block_id if block_id else "expanded_conv_"
        inp = x
        if block_id:
            x = b.conv2d(x, expansion * cin, 1, prefix + "expand", padding="same", use_bias=False)
            x = b.batchnorm(x, prefix + "expand_BN", eps=1e-3, random_stats=random_bn)
            x = b.relu(x, prefix + "expand_relu", 6.0)
        if stride == 2:
            k = 3
            h, w = x.shape[0], x.shape[1]
            adj = (1 - h % 2, 1 - w % 2)
            cor = (k // 2, k // 2)
            x = b.zero_pad(x, prefix + "pad", ((cor[0] - adj[0], cor[0]), (cor[1] - adj[1], cor[1])))
        x = b.depthwise_conv2d(x, 3, prefix + "depthwise", strides=stride, padding="same" if stride == 1 else "valid")
        x = b.batchnorm(x, prefix + "depthwise_BN", eps=1e-3, random_stats=random_bn)
        x = b.relu(x, prefix + "depthwise_relu", 6.0)
        x = b.conv2d(x, pw, 1, prefix + "project", padding="same", use_bias=False)
        x = b.batchnorm(x, prefix + "project_BN", eps=1e-3, random_stats=random_bn)
        if cin == pw and stride == 1:
            x = b.add([inp, x], prefix + "add")
        return x

    cfgs = [(1, 1, 16), (6, 2, 24), (6, 1, 24), (6, 2, 32), (6, 1, 32), (6, 1, 32), (6, 2, 64), (6, 1, 64),
            (6, 1, 64), (6, 1, 64), (6, 1, 96), (6, 1, 96), (6, 1, 96), (6, 2, 160), (6, 1, 160), (6, 1, 160),
            (6, 1, 320)]
    if truncate:
        cfgs = cfgs[:truncate]
    for i, (e, s, f) in enumerate(cfgs):
        x = inv_res(x, e, s, f, i)
    last = mk(1280 * alpha) if alpha > 1.0 else 1280
    x = b.conv2d(x, last, 1, "Conv_1", use_bias=False)
    x = b.batchnorm(x, "Conv_1_bn", eps=1e-3, random_stats=random_bn)
    x = b.relu(x, "out_relu", 6.0)
    x = b.gap(x, "global_average_pooling2d")
    x = b.dense(x, classes, "predictions", activation="softmax")
    return b.finish([x])


def encoder(seed=4, layers=6, seq=256, d_model=512, heads=8, ffn=2048, bias_std=0.0, random_affine=False):
    """Pre-LayerNorm transformer encoder: [LN -> MHA -> Add -> LN -> Dense gelu -> Dense -> Add] x layers."""
    b = Builder("encoder", seed)
    x = b.input((seq, d_model), "tokens")
    for i in range(layers):
        h = b.layernorm(x, "ln1_%d" % i, 1e-3, random_affine)
        h = b.mha(h, h, "mha_%d" % i, heads, d_model // heads, bias_std=bias_std)
        x = b.add([x, h], "add1_%d" % i)
        h = b.layernorm(x, "ln2_%d" % i, 1e-3, random_affine)
        h = b.dense(h, ffn, "ffn1_%d" % i, activation="gelu", init=0.02, bias_std=bias_std)
        h = b.dense(h, d_model, "ffn2_%d" % i, init=0.02, bias_std=bias_std)
        x = b.add([x, h], "add2_%d" % i)
    return b.finish([x])


def gpt2(seed=5, layers=12, d_model=768, heads=12, vocab=50257, max_pos=1024, ffn=None, bias_std=0.0,
         random_affine=False, std=0.02):
    """GPT-2-small-shaped decoder built from Keras layers: token + position Embedding, Add, pre-LN blocks with
    self-attention MultiHeadAttention and an erf-GELU FFN, final LN, untied Dense LM head.  Sequence length is
    variable (inputs are (T,) float id vectors)."""
    ffn = ffn or 4 * d_model
    b = Builder("gpt2", seed)
    ids = b.input((None,), "ids")
    pos = b.input((None,), "positions")
    te = b.embedding(ids, vocab, d_model, "wte", std)
    pe = b.embedding(pos, max_pos, d_model, "wpe", std)
    x = b.add([te, pe], "embed_add")
    for i in range(layers):
        h = b.layernorm(x, "h%d_ln1" % i, 1e-5, random_affine)
        h = b.mha(h, h, "h%d_attn" % i, heads, d_model // heads, std=std, bias_std=bias_std)
        x = b.add([x, h], "h%d_add1" % i)
        h = b.layernorm(x, "h%d_ln2" % i, 1e-5, random_affine)
        h = b.dense(h, ffn, "h%d_fc" % i, activation="gelu", init=std, bias_std=bias_std)
        h = b.dense(h, d_model, "h%d_proj" % i, init=std, bias_std=bias_std)
        x = b.add([x, h], "h%d_add2" % i)
    x = b.layernorm(x, "ln_f", 1e-5, random_affine)
    x = b.dense(x, vocab, "lm_head", init=std, bias_std=bias_std)
    return b.finish([x])


def model_flops(spec):
    """2 x MACs of every Conv2D / Dense layer, recomputed by tracing shapes through the layer list."""
    shapes = {}
    total = 0
    for ld in spec["architecture"]["config"]["layers"]:
        name, cls, cfg = ld["name"], ld["class_name"], ld["config"]
        if cls == "InputLayer":
            shapes[name] = tuple(cfg["batch_shape"][1:])
            continue
        args = ld["inbound_nodes"][0]["args"]
        args = args[0] if isinstance(args[0], list) else args
        ins = [shapes[a["config"]["keras_history"][0]] for a in args]
        s = ins[0]
        if cls == "Conv2D":
            kh, kw = cfg["kernel_size"]
            oh = Builder._win(s[0], (kh - 1) * cfg["dilation_rate"][0] + 1, cfg["strides"][0], cfg["padding"])
            ow = Builder._win(s[1], (kw - 1) * cfg["dilation_rate"][1] + 1, cfg["strides"][1], cfg["padding"])
            total += 2 * oh * ow * kh * kw * s[2] * cfg["filters"]
            s = (oh, ow, cfg["filters"])
        elif cls == "DepthwiseConv2D":
            kh, kw = cfg["kernel_size"]
            oh = Builder._win(s[0], kh, cfg["strides"][0], cfg["padding"])
            ow = Builder._win(s[1], kw, cfg["strides"][1], cfg["padding"])
            s = (oh, ow, s[2])
        elif cls == "Dense":
            rows = int(np.prod(s[:-1])) if len(s) > 1 else 1
            total += 2 * rows * s[-1] * cfg["units"]
            s = s[:-1] + (cfg["units"],)
        elif cls == "ZeroPadding2D":
            (pt, pb), (pl, pr) = cfg["padding"]
            s = (s[0] + pt + pb, s[1] + pl + pr, s[2])
        elif cls in ("MaxPooling2D", "AveragePooling2D"):
            k, st = cfg["pool_size"], cfg["strides"]
            s = (Builder._win(s[0], k[0], st[0], cfg["padding"]), Builder._win(s[1], k[1], st[1], cfg["padding"]), s[2])
        elif cls.startswith("Global"):
            s = (s[-1],)
        shapes[name] = s
    return total
