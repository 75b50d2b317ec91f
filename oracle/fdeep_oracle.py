"""TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.

CPU oracle for the forward path of frugally-deep's ``fdeep::model::predict``:
a converted-JSON reader and a per-sample graph walker written in Python that
calls the plain-C layer functions of ``oracle.c`` (built as ``liboracle.so``).
Only tests, the smoke check and the bench's cpu_baseline leg may import this.

The walker mirrors the reference's pull-based evaluation: every layer output is
computed once per predict call and memoised by (layer, node)
(include/fdeep/layers/model_layer.hpp:51-66, layers/layer.hpp:63-80,
node.hpp:60-78); a layer's fused ``activation`` runs after the layer itself
(include/fdeep/import_model.hpp:1953-1962, layers/layer.hpp:54-61).

The reference has no attention mask and no key/value cache
(layers/multi_head_attention_layer.hpp:74-95).  ``predict_causal`` therefore
*defines* causal self-attention through calls the reference does support: row t
of the result is ``MHA(query = x[t:t+1], value = x[0:t+1])``
(multi_head_attention_layer.hpp:98-103).
"""
import base64
import ctypes
import json
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_c_float_p = ctypes.POINTER(ctypes.c_float)
_c_int_p = ctypes.POINTER(ctypes.c_int)

PAD = {"valid": 0, "same": 1, "causal": 2}

# Layer class names the reference maps to the identity at inference
# (include/fdeep/import_model.hpp:1796-1838).
IDENTITY_LAYERS = {
    "Identity", "Dropout", "Masking", "ActivityRegularization", "AlphaDropout", "FixedDropout",
    "SpatialDropout1D", "SpatialDropout2D", "SpatialDropout3D", "GaussianDropout", "GaussianNoise",
    "RandomBrightness", "RandomContrast", "RandomCrop", "RandomFlip", "RandomHeight",
    "RandomRotation", "RandomTranslation", "RandomWidth", "RandomZoom",
    "RandomColorDegeneration", "RandomColorJitter", "RandomElasticTransform", "RandomErasing", "RandomGaussianBlur",
    "RandomGrayscale", "RandomHue", "RandomInvert", "RandomPerspective", "RandomPosterization", "RandomSaturation",
    "RandomSharpness", "RandomShear", "AugMix", "CutMix", "Equalization", "MaxNumBoundingBoxes", "MixUp", "Pipeline",
    "RandAugment", "Solarization",
}


def build(force=False):
    """Compile liboracle.so with the Makefile next to this file."""
    so = os.path.join(_HERE, "liboracle.so")
    src = os.path.join(_HERE, "oracle.c")
    stale = os.path.exists(so) and os.path.exists(src) and os.path.getmtime(src) > os.path.getmtime(so)
    if force or stale or not os.path.exists(so):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return so


def use_native_build():
    """Builds the oracle for the CPU of this host (-march=native) and makes every later call use it: for the timed
    CPU-baseline leg, which should not run an AVX2 build on an AVX-512 host.  Returns the compiler flags in use;
    keeps the portable build when no compiler is at hand."""
    global _LIB
    so = os.path.join(_HERE, "liboracle_native.so")
    try:
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle_native.so"], stdout=subprocess.DEVNULL,
                              stderr=subprocess.DEVNULL)
        native = ctypes.CDLL(so)
        native.fdo_argmax.restype = ctypes.c_size_t
        _LIB = native
        return "-O3 -march=native, built on the measuring host"
    except (OSError, subprocess.CalledProcessError):
        lib()
        return "-O3 -march=x86-64-v3 (AVX2 + FMA), prebuilt"


def lib():
    global _LIB
    if _LIB is None:
        _LIB = ctypes.CDLL(build())
        _LIB.fdo_argmax.restype = ctypes.c_size_t
    return _LIB


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return None if a is None else a.ctypes.data_as(_c_float_p)


def _ip(a):
    return a.ctypes.data_as(_c_int_p)


# ---------------------------------------------------------------- layer functions

def window_geometry(in_h, in_w, k_h, k_w, s_h, s_w, padding):
    g = (ctypes.c_int * 6)()
    rc = lib().fdo_window_geometry(in_h, in_w, k_h, k_w, s_h, s_w, PAD[padding], g)
    if rc != 0:
        raise RuntimeError("invalid window geometry")
    return dict(pad_top=g[0], pad_bottom=g[1], pad_left=g[2], pad_right=g[3], out_h=g[4], out_w=g[5])


def conv2d_prepare(w_json, cout, kh, kw, cin):
    w_json = _f32(w_json).reshape(-1)
    out = np.empty(kh * kw * cin * cout, np.float32)
    lib().fdo_conv2d_prepare(_p(w_json), cout, kh, kw, cin, _p(out))
    return out


def conv2d(x, w_hwio, bias, cout, kh, kw, strides=(1, 1), dilation=(1, 1), padding="valid"):
    x = _f32(x)
    h, w, cin = x.shape
    hw = (ctypes.c_int * 2)()
    args = (h, w, cin, _p(w_hwio), _p(bias), cout, kh, kw, strides[0], strides[1],
            dilation[0], dilation[1], PAD[padding])
    if lib().fdo_conv2d(_p(x), *args, None, hw) != 0:
        raise RuntimeError("conv2d geometry error")
    out = np.empty((hw[0], hw[1], cout), np.float32)
    if lib().fdo_conv2d(_p(x), *args, _p(out), hw) != 0:
        raise RuntimeError("conv2d failed")
    return out


def conv2d_transpose_prepare(w_json, cout, kh, kw, cin):
    """Filter of a transposed convolution: mirrored in height and width at load (filter.hpp:94-97)."""
    w = _f32(w_json).reshape(cout, kh, kw, cin)[:, ::-1, ::-1, :]
    return conv2d_prepare(np.ascontiguousarray(w), cout, kh, kw, cin)


def conv2d_transpose(x, w_hwio_flipped, bias, cout, kh, kw, strides=(1, 1), dilation=(1, 1), padding="valid"):
    x = _f32(x)
    h, w, cin = x.shape
    hw = (ctypes.c_int * 2)()
    args = (h, w, cin, _p(w_hwio_flipped), _p(bias), cout, kh, kw, strides[0], strides[1],
            dilation[0], dilation[1], PAD[padding])
    if lib().fdo_conv2d_transpose(_p(x), *args, None, hw) != 0:
        raise RuntimeError("transposed convolution: output width does not match")
    out = np.empty((hw[0], hw[1], cout), np.float32)
    if lib().fdo_conv2d_transpose(_p(x), *args, _p(out), hw) != 0:
        raise RuntimeError("conv2d_transpose failed")
    return out


def depthwise_conv2d(x, w_json, bias, kh, kw, strides=(1, 1), dilation=(1, 1), padding="valid"):
    x = _f32(x)
    h, w, c = x.shape
    w_json = _f32(w_json).reshape(-1)
    hw = (ctypes.c_int * 2)()
    args = (h, w, c, _p(w_json), _p(bias), kh, kw, strides[0], strides[1],
            dilation[0], dilation[1], PAD[padding])
    if lib().fdo_depthwise_conv2d(_p(x), *args, None, hw) != 0:
        raise RuntimeError("depthwise geometry error")
    out = np.empty((hw[0], hw[1], c), np.float32)
    if lib().fdo_depthwise_conv2d(_p(x), *args, _p(out), hw) != 0:
        raise RuntimeError("depthwise failed")
    return out


def dense(x, w, bias, n_out):
    x = _f32(x)
    n_in = x.shape[-1]
    rows = x.size // n_in
    out = np.empty(x.shape[:-1] + (n_out,), np.float32)
    lib().fdo_dense(_p(x), rows, n_in, _p(w), _p(bias), n_out, _p(out))
    return out


def softmax(x):
    x = _f32(x)
    out = np.empty_like(x)
    depth = x.shape[-1]
    lib().fdo_softmax(_p(x), x.size // depth, depth, _p(out))
    return out


def layernorm(x, gamma, beta, eps, n_axes=1):
    x = _f32(x)
    depth = int(np.prod(x.shape[x.ndim - n_axes:]))
    out = np.empty_like(x)
    lib().fdo_layernorm(_p(x), x.size // depth, depth, _p(gamma), _p(beta), ctypes.c_float(eps), _p(out))
    return out


def layernorm_axes(x, axes, gamma, beta, eps):
    """LayerNormalization over `axes` (1-based in x's rank, negative from the end): moments over those
    axes, gamma / beta shaped like them in storage order (layers/layer_normalization_layer.hpp:37-61).
    The axes are brought to the end, rows are normalised by the C routine, and the move is undone."""
    x = _f32(x)
    axes = sorted(set(a + x.ndim + 1 if a < 0 else a for a in axes))
    src = [a - 1 for a in axes]
    dst = list(range(x.ndim - len(axes), x.ndim))
    xm = np.ascontiguousarray(np.moveaxis(x, src, dst))
    return np.ascontiguousarray(np.moveaxis(layernorm(xm, gamma, beta, eps, len(axes)), dst, src))


def batchnorm(x, mean, var, gamma, beta, eps):
    x = _f32(x)
    c = x.shape[-1]
    out = np.empty_like(x)
    lib().fdo_batchnorm(_p(x), ctypes.c_size_t(x.size // c), c, _p(mean), _p(var), _p(gamma), _p(beta),
                        ctypes.c_float(eps), _p(out))
    return out


FLT_MAX = float(np.finfo(np.float32).max)


def relu(x, max_value=FLT_MAX, negative_slope=0.0, threshold=0.0):
    x = _f32(x)
    out = np.empty_like(x)
    lib().fdo_relu(_p(x), ctypes.c_size_t(x.size), ctypes.c_float(max_value), ctypes.c_float(negative_slope),
                   ctypes.c_float(threshold), _p(out))
    return out


def gelu(x):
    x = _f32(x)
    out = np.empty_like(x)
    lib().fdo_gelu(_p(x), ctypes.c_size_t(x.size), _p(out))
    return out


def activation(name, x, p0=0.0, p1=0.0):
    """Any of the reference's element-wise activations by its config name (import_model.hpp:1649-1700)."""
    x = _f32(x)
    out = np.empty_like(x)
    if lib().fdo_activation(name.encode(), ctypes.c_float(p0), ctypes.c_float(p1), _p(x), ctypes.c_size_t(x.size), _p(out)) != 0:
        raise RuntimeError("unknown activation type: " + name)
    return out


def combine(op, a, b):
    """mul / sub / max / min of two tensors; size-1 axes are expanded first (tensor.hpp:642-660)."""
    a, b = np.broadcast_arrays(_f32(a), _f32(b)) if np.shape(a) != np.shape(b) else (_f32(a), _f32(b))
    a, b = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
    out = np.empty_like(a)
    lib().fdo_combine({"mul": 1, "sub": 2, "max": 3, "min": 4}[op], _p(a), _p(b), ctypes.c_size_t(a.size), _p(out))
    return out


def prelu(x, alpha, shared_axes):
    """layers/prelu_layer.hpp:29-70, including the shift of the shared axis numbers for samples without a height
    (and width) axis of their own."""
    x = _f32(x)
    h, w, c = ((1, 1, 1) + x.shape)[-3:]
    shifted, shift = [], 0
    for a in shared_axes:
        if (a == 1 and h == 1) or (a == 2 and w == 1):
            shift += 1
        shifted.append(a + shift)
    out = np.empty_like(x)
    lib().fdo_prelu(_p(x), h, w, c, _p(_f32(alpha)), int(1 in shifted), int(2 in shifted), int(3 in shifted), _p(out))
    return out


def pool2d(x, pool_size, strides, padding, mode):
    x = _f32(x)
    h, w, c = x.shape
    hw = (ctypes.c_int * 2)()
    m = 0 if mode == "max" else 1
    args = (h, w, c, pool_size[0], pool_size[1], strides[0], strides[1], PAD[padding], m)
    if lib().fdo_pool2d(_p(x), *args, None, hw) != 0:
        raise RuntimeError("pool geometry error")
    out = np.empty((hw[0], hw[1], c), np.float32)
    lib().fdo_pool2d(_p(x), *args, _p(out), hw)
    return out


def global_pool(x, mode, keepdims=False):
    x = _f32(x)
    c = x.shape[-1]
    out = np.empty(c, np.float32)
    lib().fdo_global_pool(_p(x), ctypes.c_size_t(x.size // c), c, 0 if mode == "max" else 1, _p(out))
    return out.reshape((1,) * (x.ndim - 1) + (c,)) if keepdims else out


def add(a, b):
    a, b = _f32(a), _f32(b)
    if a.shape != b.shape:
        # numpy-style broadcasting of size-1 dims on right-aligned shapes,
        # include/fdeep/tensor.hpp:642-676
        return (a + b).astype(np.float32)
    out = np.empty_like(a)
    lib().fdo_add(_p(a), _p(b), ctypes.c_size_t(a.size), _p(out))
    return out


def embedding(ids, table, input_dim, output_dim):
    ids = _f32(ids).reshape(-1)
    out = np.empty((ids.size, output_dim), np.float32)
    if lib().fdo_embedding(_p(ids), ids.size, _p(table), input_dim, output_dim, _p(out)) != 0:
        raise RuntimeError("vocabulary item indices must all be strictly less than the value of input_dim")
    return out


def argmax(x):
    x = _f32(x).reshape(-1)
    return int(lib().fdo_argmax(_p(x), ctypes.c_size_t(x.size)))


def mha(query, value, key, heads, dk, dv, weights, use_bias):
    """weights: list in Keras order q_w,q_b,k_w,k_b,v_w,v_b,o_w,o_b (no-bias: 4 kernels)."""
    query, value = _f32(query), _f32(value)
    key = value if key is None else _f32(key)
    if query.ndim != 2 or value.ndim != 2 or key.ndim != 2:
        raise RuntimeError("Invalid shapes; need a query tensor of shape (B, T, dim) and a value/key tensor of "
                           "shape (B, S, dim).")
    if use_bias:
        qw, qb, kw, kb, vw, vb, ow, ob = weights
    else:
        qw, kw, vw, ow = weights
        qb = kb = vb = ob = None
    t, d = query.shape
    s = value.shape[0]
    dout = ow.size // (heads * dv)
    out = np.empty((t, dout), np.float32)
    rc = lib().fdo_mha(_p(query), t, _p(value), _p(key), s, d, heads, dk, dv, dout,
                       _p(qw), _p(qb), _p(kw), _p(kb), _p(vw), _p(vb), _p(ow), _p(ob), _p(out))
    if rc != 0:
        raise RuntimeError("mha failed")
    return out


def gqa(query, value, key, head_dim, hq, hkv, weights, use_bias, use_gate):
    """GroupQueryAttention; weights in Keras order Q, K, [Gate], V, Out with each bias right after its kernel
    (include/fdeep/layers/group_query_attention_layer.hpp:45-60)."""
    q, v = _f32(query), _f32(value)
    k = v if key is None else _f32(key)
    step = 2 if use_bias else 1
    w = [_f32(a).reshape(-1) for a in weights]
    def kern(i):
        return w[i * step]
    def bias(i):
        return w[i * step + 1] if use_bias else None
    vi, oi = (3, 4) if use_gate else (2, 3)
    dout = kern(oi).size // (hq * head_dim)
    out = np.empty((q.shape[0], dout), np.float32)
    rc = lib().fdo_gqa(_p(q), q.shape[0], _p(v), _p(k), v.shape[0], q.shape[1], head_dim, hq, hkv, _p(kern(0)), _p(bias(0)),
                       _p(kern(1)), _p(bias(1)), _p(kern(2)) if use_gate else None, _p(bias(2)) if use_gate else None,
                       _p(kern(vi)), _p(bias(vi)), _p(kern(oi)), _p(bias(oi)), dout, _p(out))
    if rc != 0:
        raise RuntimeError("num_query_heads must be divisible by num_key_value_heads.")
    return out


def rmsnorm_axes(x, axes, scale, eps):
    """RMSNormalization over `axes` (1-based, negative from the end), scale shaped like those axes
    (layers/rms_normalization_layer.hpp:37-69); the axes are brought to the end around the row routine."""
    x = _f32(x)
    axes = sorted(set(a + x.ndim + 1 if a < 0 else a for a in axes))
    src, dst = [a - 1 for a in axes], list(range(x.ndim - len(axes), x.ndim))
    xm = np.ascontiguousarray(np.moveaxis(x, src, dst))
    depth = int(np.prod(xm.shape[xm.ndim - len(axes):]))
    out = np.empty_like(xm)
    lib().fdo_rmsnorm(_p(xm), ctypes.c_size_t(xm.size // depth), depth, _p(scale), ctypes.c_float(eps), _p(out))
    return np.ascontiguousarray(np.moveaxis(out, dst, src))


def upsample2d(x, factor_y, factor_x, bilinear=False):
    """UpSampling2D on an (h, w, c) sample by integer factors (layers/upsampling_2d_layer.hpp)."""
    x = _f32(x)
    h, w, c = x.shape
    out = np.empty((h * factor_y, w * factor_x, c), np.float32)
    lib().fdo_upsample2d(_p(x), h, w, c, int(factor_y), int(factor_x), int(bool(bilinear)), _p(out))
    return out


def einsum_dense(x, equation, kernel, kernel_shape, bias, bias_axes):
    """EinsumDense on one sample; x excludes the batch dim (size-1 batch char is re-added)."""
    x = _f32(x)
    lhs, rest = equation.split(",")
    rk, rhs = rest.split("->")
    chars = sorted(set(lhs + rk + rhs))
    cid = {c: i for i, c in enumerate(chars)}
    sizes = {}
    for c, n in zip(rk, kernel_shape[len(kernel_shape) - len(rk):]):
        sizes[c] = int(n)
    lead = len(lhs) - x.ndim
    for i, c in enumerate(lhs):
        sz = 1 if i < lead else x.shape[i - lead]
        if c in sizes and sizes[c] != sz:
            raise RuntimeError("EinsumDense: inconsistent char size in equation.")
        sizes[c] = sz
    summed = [c for c in lhs if c not in rhs and c in rk]
    bias_chars = [c for c in rhs if c in (bias_axes or "")]
    sz_arr = np.array([sizes[c] for c in chars], np.int32)
    idx = lambda s: np.array([cid[c] for c in s], np.int32)
    in_idx, k_idx, o_idx, s_idx, b_idx = idx(lhs), idx(rk), idx(rhs), idx(summed), idx(bias_chars)
    out_shape = [sizes[c] for c in rhs]
    out = np.empty(out_shape, np.float32)
    kernel = _f32(kernel).reshape(-1)
    b = _f32(bias).reshape(-1) if bias_axes else None
    rc = lib().fdo_einsum_dense(_p(x), _ip(in_idx), len(lhs), _p(kernel), _ip(k_idx), len(rk),
                                _p(b), _ip(b_idx), len(bias_chars), _ip(o_idx), len(rhs),
                                _ip(s_idx), len(summed), _ip(sz_arr), len(chars), _p(out))
    if rc != 0:
        raise RuntimeError("einsum_dense failed")
    return out.reshape(out_shape[1:])


# ---------------------------------------------------------------- file format

def decode_floats(data):
    """Base64 chunks (fp32 little-endian) or a plain number array.
    include/fdeep/import_model.hpp:274-297, include/fdeep/base64.hpp:65-108."""
    if isinstance(data, list) and data and isinstance(data[0], (int, float)):
        return np.array(data, np.float32)
    if isinstance(data, str):
        data = [data]
    raw = b"".join(base64.b64decode(s.replace("-", "+").replace("_", "/")) for s in data)
    if len(raw) % 4:
        raise RuntimeError("invalid float vector data")
    return np.frombuffer(raw, "<f4").astype(np.float32)


def _connections(data):
    # a single connection may be a flat triple, import_model.hpp:352-360
    if data and not isinstance(data[0], list):
        return [tuple(data[:3])]
    return [tuple(d[:3]) for d in data]


def _node_inputs(node):
    args = node["args"]
    if args and isinstance(args[0], list):  # merge layers wrap their inputs once more
        args = args[0]
    res = []
    for a in args:
        hist = a["config"].get("keras_history") if isinstance(a, dict) and "config" in a else None
        if hist is None:
            raise RuntimeError("No keras_history on node connection. Constant-value tensors are not supported.")
        res.append((hist[0], int(hist[1]), int(hist[2])))
    return res


def _activation(name, cfg, x):
    if name == "linear":
        return x
    if name == "relu":
        # relu layer parameters are honoured only when max_value is present and non-null,
        # import_model.hpp:1289-1302
        if cfg.get("max_value") is not None:
            return relu(x, cfg["max_value"], cfg["negative_slope"], cfg["threshold"])
        return relu(x)
    if name == "relu6":
        return relu(x, 6.0, 0.0, 0.0)
    if name == "gelu":
        if cfg.get("approximate"):
            raise RuntimeError("Gelu with approximate = True is not supported.")
        return gelu(x)
    if name == "softmax":
        return softmax(x)
    if name == "log_softmax":
        return activation("log", softmax(x))
    # parameters and their defaults: import_model.hpp:1200-1385
    if name in ("elu", "celu"):
        return activation(name, x, cfg.get("alpha", 1.0))
    if name == "leaky_relu":
        return activation(name, x, cfg.get("negative_slope", 0.2))
    if name in ("hard_shrink", "soft_shrink"):
        return activation(name, x, cfg["threshold"])
    if name == "squareplus":
        b = cfg.get("b")
        return activation(name, x, 4.0 if b is None else b)
    if name == "threshold":
        thr = cfg["threshold"] if "threshold" in cfg else cfg["threshold_value"]
        dv = cfg["default_value"] if "default_value" in cfg else cfg["value"]
        return activation(name, x, thr, dv)
    return activation(name, x)


ACTIVATION_LAYERS = {"LeakyReLU": "leaky_relu", "LeakyRelu": "leaky_relu", "ELU": "elu", "Elu": "elu", "Celu": "celu",
                     "Relu6": "relu6", "Exp": "exponential", "Gelu": "gelu", "Selu": "selu", "Silu": "silu", "Tanh": "tanh",
                     "TanhShrink": "tanh_shrink", "Threshold": "threshold", "Sigmoid": "sigmoid", "HardShrink": "hard_shrink",
                     "HardSigmoid": "hard_sigmoid", "HardTanh": "hard_tanh", "SoftShrink": "soft_shrink", "Softplus": "softplus",
                     "Softsign": "softsign", "SparsePlus": "sparse_plus", "Squareplus": "squareplus",
                     "LogSigmoid": "log_sigmoid", "LogSoftmax": "log_softmax"}  # import_model.hpp:1839-1865


def _pair(v):
    """create_shape2 (import_model.hpp): two values, or one value for the width of a 1-D layer (height 1)."""
    if isinstance(v, (list, tuple)):
        return (int(v[0]), int(v[1])) if len(v) == 2 else (1, int(v[0]))
    return (1, int(v))  # a bare number is a width


class _Layer:
    def __init__(self, data, get_param):
        self.name = data["name"]
        self.cls = data["class_name"]
        self.cfg = data.get("config", {})
        self.nodes = [_node_inputs(n) for n in data.get("inbound_nodes", [])]
        self.p = {}
        c, cls, name = self.cfg, self.cls, self.name
        if cls in ("Conv2D", "Conv1D", "Conv2DTranspose", "Conv1DTranspose"):
            self.kh, self.kw = _pair(c["kernel_size"])
            self.cout = int(c["filters"])
            w = decode_floats(get_param(name, "weights"))
            self.cin = w.size // (self.kh * self.kw * self.cout)
            prepare = conv2d_transpose_prepare if cls.endswith("Transpose") else conv2d_prepare
            self.p["w"] = prepare(w, self.cout, self.kh, self.kw, self.cin)
            self.p["b"] = decode_floats(get_param(name, "bias")) if c["use_bias"] else np.zeros(self.cout, np.float32)
        elif cls == "DepthwiseConv2D":
            self.kh, self.kw = c["kernel_size"]
            self.p["w"] = decode_floats(get_param(name, "slice_weights"))
            ch = self.p["w"].size // (self.kh * self.kw)
            self.p["b"] = decode_floats(get_param(name, "bias")) if c["use_bias"] else np.zeros(ch, np.float32)
        elif cls == "Dense":
            self.p["w"] = decode_floats(get_param(name, "weights"))
            units = int(c["units"])
            self.p["b"] = decode_floats(get_param(name, "bias")) if c["use_bias"] else np.zeros(units, np.float32)
        elif cls == "BatchNormalization":
            self.p["mean"] = decode_floats(get_param(name, "moving_mean"))
            self.p["var"] = decode_floats(get_param(name, "moving_variance"))
            self.p["gamma"] = decode_floats(get_param(name, "gamma")) if c["scale"] else None
            self.p["beta"] = decode_floats(get_param(name, "beta")) if c["center"] else None
        elif cls == "Normalization":
            self.p["mean"] = decode_floats(get_param(name, "mean"))
            self.p["var"] = decode_floats(get_param(name, "variance"))
        elif cls == "LayerNormalization":
            self.p["gamma"] = decode_floats(get_param(name, "gamma")) if c["scale"] else None
            self.p["beta"] = decode_floats(get_param(name, "beta")) if c["center"] else None
        elif cls == "Embedding":
            self.p["w"] = decode_floats(get_param(name, "weights"))
        elif cls == "MultiHeadAttention":
            shapes = get_param(name, "weight_shapes")
            vals = [decode_floats(v) for v in get_param(name, "weights")]
            assert len(shapes) == len(vals)
            self.p["w"] = vals
        elif cls == "PReLU":
            self.p["alpha"] = decode_floats(get_param(name, "alpha"))
        elif cls in ("SeparableConv2D", "SeparableConv1D"):
            self.kh, self.kw = c["kernel_size"] if len(c["kernel_size"]) == 2 else (1, c["kernel_size"][0])
            self.p["slice"] = decode_floats(get_param(name, "slice_weights"))
            self.p["stack"] = decode_floats(get_param(name, "stack_weights"))
            self.cout = int(c["filters"])
            self.p["b"] = decode_floats(get_param(name, "bias")) if c["use_bias"] else np.zeros(self.cout, np.float32)
        elif cls == "RMSNormalization":
            self.p["scale"] = decode_floats(get_param(name, "scale"))
        elif cls in ("GroupQueryAttention", "GroupedQueryAttention"):
            self.p["w"] = [decode_floats(v) for v in get_param(name, "weights")]
        elif cls == "EinsumDense":
            self.p["kernel"] = decode_floats(get_param(name, "kernel"))
            self.p["kernel_shape"] = [int(v) for v in get_param(name, "kernel_shape")]
            self.p["bias"] = decode_floats(get_param(name, "bias")) if c.get("bias_axes") else None

    def apply(self, ins):
        cls, c, p = self.cls, self.cfg, self.p
        if cls == "InputLayer":
            raise AssertionError("input layers are seeded, never applied")
        if cls in IDENTITY_LAYERS:
            out = ins[0]
        elif cls in ("Conv2D", "Conv1D"):
            x = _f32(ins[0])
            one_d = x.ndim == 2  # a (width, depth) sequence is a height-1 image
            out = conv2d(x[None] if one_d else x, p["w"], p["b"], self.cout, self.kh, self.kw, _pair(c["strides"]),
                         _pair(c["dilation_rate"]), c["padding"])
            out = out[0] if one_d else out
        elif cls in ("Conv2DTranspose", "Conv1DTranspose"):
            x = _f32(ins[0])
            one_d = x.ndim == 2
            out = conv2d_transpose(x[None] if one_d else x, p["w"], p["b"], self.cout, self.kh, self.kw,
                                   _pair(c["strides"]), _pair(c["dilation_rate"]), c["padding"])
            out = out[0] if one_d else out
        elif cls == "DepthwiseConv2D":
            out = depthwise_conv2d(ins[0], p["w"], p["b"], self.kh, self.kw, c["strides"],
                                   c["dilation_rate"], c["padding"])
        elif cls == "Dense":
            out = dense(ins[0], p["w"], p["b"], int(c["units"]))
        elif cls == "Rescaling":
            # layers/rescaling_layer.hpp:30-40
            out = (np.float32(c["scale"]) * ins[0] + np.float32(c["offset"])).astype(np.float32)
        elif cls == "Normalization":
            # layers/normalization_layer.hpp:36-75: per slice of the axis, (x - mean) / max(sqrt(var), 1e-7) or,
            # inverted, mean + x * max(sqrt(var), 1e-7); no axis: one pair for the whole tensor
            x = ins[0]
            axes = c["axis"] if isinstance(c["axis"], (list, tuple)) else ([] if c["axis"] is None else [c["axis"]])
            if len(axes) > 1:
                raise ValueError("Unsupported number of axes for Normalization layer")
            sd = np.maximum(np.sqrt(p["var"]), np.float32(1e-7)).astype(np.float32)
            mean = p["mean"]
            if not axes:
                if sd.size != 1:
                    raise ValueError("Invalid number of variance values in Normalization layer.")
            else:
                axis = axes[0] if axes[0] >= 0 else axes[0] + x.ndim + 1  # Keras axes count the batch dimension
                if x.shape[axis - 1] != sd.size:
                    raise ValueError("Invalid number of variance values in Normalization layer.")
                shape = [1] * x.ndim
                shape[axis - 1] = sd.size
                sd, mean = sd.reshape(shape), mean.reshape(shape)
            out = ((mean + x * sd) if c.get("invert", False) else ((x - mean) / sd)).astype(np.float32)
        elif cls == "BatchNormalization":
            axis = c["axis"][0] if isinstance(c["axis"], list) else c["axis"]
            x = ins[0]
            if axis < 0:
                axis += x.ndim + 1
            if axis != x.ndim:  # Keras axes count the batch dim; move the axis last
                xm = np.moveaxis(x, axis - 1, -1)
                out = np.moveaxis(batchnorm(xm, p["mean"], p["var"], p["gamma"], p["beta"], c["epsilon"]), -1,
                                  axis - 1)
            else:
                out = batchnorm(x, p["mean"], p["var"], p["gamma"], p["beta"], c["epsilon"])
        elif cls == "LayerNormalization":
            x = ins[0]
            axes = c["axis"] if isinstance(c["axis"], list) else [c["axis"]]
            out = layernorm_axes(x, axes, p["gamma"], p["beta"], c["epsilon"])
        elif cls == "ReLU":
            out = _activation("relu", c, ins[0])
        elif cls == "Activation":
            return _activation(c["activation"], c, ins[0])
        elif cls in ACTIVATION_LAYERS:
            return _activation(ACTIVATION_LAYERS[cls], c, ins[0])
        elif cls == "PReLU":
            out = prelu(ins[0], p["alpha"], c.get("shared_axes") or [])
        elif cls == "Softmax":
            out = softmax(ins[0])
        elif cls == "ZeroPadding2D":
            pad = c["padding"]
            (pt, pb), (pl, pr) = pad
            x = _f32(ins[0])
            out = np.zeros((x.shape[0] + pt + pb, x.shape[1] + pl + pr, x.shape[2]), np.float32)
            out[pt:pt + x.shape[0], pl:pl + x.shape[1]] = x
        elif cls in ("MaxPooling2D", "AveragePooling2D"):
            strides = c["strides"] if c.get("strides") is not None else c["pool_size"]
            out = pool2d(ins[0], c["pool_size"], strides, c["padding"], "max" if cls[0] == "M" else "avg")
        elif cls in ("MaxPooling1D", "AveragePooling1D"):
            # the 1-D layers are the 2-D ones on a height-1 tensor (import_model.hpp:866-905)
            size = c["pool_size"][0] if isinstance(c["pool_size"], list) else c["pool_size"]
            st = c["strides"] if c.get("strides") is not None else size
            st = st[0] if isinstance(st, list) else st
            out = pool2d(_f32(ins[0])[None], (1, size), (1, st), c["padding"], "max" if cls[0] == "M" else "avg")[0]
        elif cls == "ZeroPadding1D":
            pad = c["padding"]
            left, right = (pad, pad) if isinstance(pad, int) else pad
            x = _f32(ins[0])
            out = np.zeros((x.shape[0] + left + right, x.shape[1]), np.float32)
            out[left:left + x.shape[0]] = x
        elif cls in ("Cropping2D", "Cropping1D"):
            cr = c["cropping"]  # crop_tensor, tensor.hpp:586-610
            x = _f32(ins[0])
            if isinstance(cr[0], list):
                (t, b), (l, r) = cr
                out = np.ascontiguousarray(x[t:x.shape[0] - b, l:x.shape[1] - r])
            else:
                out = np.ascontiguousarray(x[cr[0]:x.shape[0] - cr[1]])
        elif cls == "UpSampling2D":
            if c["interpolation"] not in ("nearest", "bilinear"):
                raise RuntimeError("Invalid interpolation method: " + c["interpolation"])
            out = upsample2d(ins[0], c["size"][0], c["size"][1], c["interpolation"] == "bilinear")
        elif cls == "UpSampling1D":
            out = upsample2d(_f32(ins[0])[None], 1, c["size"])[0]  # x_in = x / size, layers/upsampling_1d_layer.hpp
        elif cls == "Permute":
            out = np.ascontiguousarray(np.transpose(_f32(ins[0]), [d - 1 for d in c["dims"]]))  # tensor.hpp:526-549
        elif cls in ("GlobalAveragePooling2D", "GlobalMaxPooling2D", "GlobalAveragePooling1D", "GlobalMaxPooling1D"):
            out = global_pool(ins[0], "max" if "Max" in cls else "avg", bool(c.get("keepdims", False)))
        elif cls == "Add":
            out = ins[0]
            for other in ins[1:]:  # left fold, tensor.hpp:677-680
                out = add(out, other)
        elif cls in ("Multiply", "Maximum", "Minimum"):
            out = ins[0]
            for other in ins[1:]:  # left folds (tensor.hpp:687-690, 893-929)
                out = combine({"Multiply": "mul", "Maximum": "max", "Minimum": "min"}[cls], out, other)
        elif cls == "Subtract":
            if len(ins) != 2:
                raise RuntimeError("subtract layer needs exactly two input tensors")
            out = combine("sub", ins[0], ins[1])
        elif cls == "Average":
            out = ins[0]
            for other in ins[1:]:
                out = add(out, other)
            out = (out * np.float32(1.0 / len(ins))).astype(np.float32)  # sum times 1 / n, tensor.hpp:886-891
        elif cls == "Concatenate":
            # the axis counts from the first input's rank, batch axis = 0 (tensor.hpp:459-483)
            axis = int(c["axis"])
            rank = _f32(ins[0]).ndim
            axis = axis + rank + 1 if axis < 0 else axis
            if not 1 <= axis <= rank:
                raise RuntimeError("Invalid axis (%d) for tensor concatenation." % axis)
            out = np.concatenate([_f32(t) for t in ins], axis=axis - 1)
        elif cls == "Embedding":
            out = embedding(ins[0], p["w"], int(c["input_dim"]), int(c["output_dim"]))
        elif cls == "MultiHeadAttention":
            key = ins[2] if len(ins) > 2 else None
            out = mha(ins[0], ins[1], key, int(c["num_heads"]), int(c["key_dim"]), int(c["value_dim"]),
                      p["w"], bool(c["use_bias"]))
        elif cls in ("SeparableConv2D", "SeparableConv1D"):
            # depthwise part without bias, then a 1x1 valid convolution (layers/separable_conv_2d_layer.hpp:26-55)
            ch = p["slice"].size // (self.kh * self.kw)
            tmp = depthwise_conv2d(ins[0], p["slice"], np.zeros(ch, np.float32), self.kh, self.kw, c["strides"],
                                   c["dilation_rate"], c["padding"])
            out = conv2d(tmp, conv2d_prepare(p["stack"], self.cout, 1, 1, ch), p["b"], self.cout, 1, 1, (1, 1), (1, 1), "valid")
        elif cls == "RMSNormalization":
            axes = c["axis"] if isinstance(c["axis"], list) else [c["axis"]]
            out = rmsnorm_axes(ins[0], axes, p["scale"] if p["scale"].size else None, c["epsilon"])
        elif cls in ("GroupQueryAttention", "GroupedQueryAttention"):
            out = gqa(ins[0], ins[1], ins[2] if len(ins) > 2 else None, int(c["head_dim"]), int(c["num_query_heads"]),
                      int(c["num_key_value_heads"]), p["w"], bool(c["use_bias"]), bool(c.get("use_gate", False)))
        elif cls == "EinsumDense":
            out = einsum_dense(ins[0], c["equation"], p["kernel"], p["kernel_shape"], p["bias"],
                               c.get("bias_axes"))
        elif cls == "Flatten":
            out = _f32(ins[0]).reshape(-1)
        elif cls == "Reshape":
            out = _f32(ins[0]).reshape(c["target_shape"])
        else:
            raise RuntimeError("unknown layer type: " + cls)
        act = c.get("activation")
        if act is not None:
            out = _activation(act, {}, out)
        return out


class _Graph:
    """One level of the layer graph: the model itself or a nested Functional model, whose layers
    read their parameters under "<outer layer names>_<layer>" (import_model.hpp:397-424)."""

    def __init__(self, config, get_param):
        self.layers = {}
        self.nested = {}
        for ld in config["layers"]:
            if ld["name"] in self.layers or ld["name"] in self.nested:
                raise RuntimeError("layer names must be unique")
            if ld["class_name"] in ("Functional", "Model"):
                prefix = ld["name"] + "_"
                inner = _Graph(ld["config"], lambda layer, key, pf=prefix: get_param(pf + layer, key))
                inner.nodes = [_node_inputs(n) for n in ld.get("inbound_nodes", [])]
                self.nested[ld["name"]] = inner
            else:
                self.layers[ld["name"]] = _Layer(ld, get_param)
        self.inputs = _connections(config["input_layers"])
        self.outputs = _connections(config["output_layers"])

    def run(self, inputs, causal=False, taps=None):
        if len(inputs) != len(self.inputs):
            raise RuntimeError("invalid number of input tensors for this model: %d required but %d provided"
                               % (len(self.inputs), len(inputs)))
        memo = {}
        for (lname, node, tidx), x in zip(self.inputs, inputs):
            memo[(lname, node)] = [x]

        def get(conn):
            lname, node, tidx = conn
            if lname in self.nested:
                inner = self.nested[lname]
                # a nested model counts its construction as node 0 (layers/model_layer.hpp:36-44)
                node = node - 1 if node >= 1 else node
                key = (lname, node)
                if key not in memo:
                    memo[key] = inner.run([get(cn) for cn in inner.nodes[node]], causal)
                return memo[key][tidx]
            key = (lname, node)
            if key not in memo:
                layer = self.layers[lname]
                ins = [get(cn) for cn in layer.nodes[node]]
                if causal and layer.cls == "MultiHeadAttention":
                    hook = causal if callable(causal) else OracleModel._causal_mha
                    memo[key] = [hook(layer, ins)]
                else:
                    memo[key] = [layer.apply(ins)]
            return memo[key][0]

        outs = [get(cn) for cn in self.outputs]
        if taps is not None:
            taps.update({k: v[0] for k, v in memo.items()})
        return outs


class OracleModel:
    """One converted-JSON model evaluated sample by sample on the CPU."""

    def __init__(self, source):
        if isinstance(source, (str, bytes)) and not (isinstance(source, str) and os.path.exists(source)):
            data = json.loads(source)
        elif isinstance(source, str):
            with open(source, "rb") as f:
                data = json.load(f)
        else:
            data = source
        if data.get("image_data_format") != "channels_last":
            raise RuntimeError("only channels_last data format supported")
        self.data = data
        arch = data["architecture"]
        params = data.get("trainable_params", {})
        get_param = lambda layer, key: params[layer][key]
        self.name = arch["config"]["name"]
        self.graph = _Graph(arch["config"], get_param)
        self.layers = self.graph.layers
        self.inputs = self.graph.inputs
        self.outputs = self.graph.outputs
        self.input_shapes = data["input_shapes"]
        self.output_shapes = data["output_shapes"]

    def _check_inputs(self, inputs):
        if len(inputs) != len(self.input_shapes):
            raise RuntimeError("Invalid inputs shape.")
        for x, shp in zip(inputs, self.input_shapes):
            if x.ndim != len(shp) or any(s is not None and s != d for s, d in zip(shp, x.shape)):
                raise RuntimeError("Invalid inputs shape.")

    def predict(self, inputs, causal=False, taps=None):
        """inputs: list of arrays without batch dim.  taps: optional dict that receives
        every intermediate (layer name, node) -> array of the top-level graph."""
        inputs = [_f32(x) for x in inputs]
        self._check_inputs(inputs)
        return self.graph.run(inputs, causal, taps)

    @staticmethod
    def _causal_mha(layer, ins):
        # row t = reference MHA(query = x[t:t+1], value = x[0:t+1]), the 2-input call of
        # include/fdeep/layers/multi_head_attention_layer.hpp:98-103
        q, v = ins[0], ins[1]
        k = ins[2] if len(ins) > 2 else None
        rows = []
        for t in range(q.shape[0]):
            sub = [q[t:t + 1], v[:t + 1]] + ([k[:t + 1]] if k is not None else [])
            rows.append(layer.apply(sub))
        return np.concatenate(rows, axis=0)

    def predict_class(self, inputs):
        out = self.predict(inputs)
        return argmax(out[0])


    def run_embedded_tests(self, eps=1e-4):
        """Replays the file's own test cases, absolute tolerance, NaN == NaN passes.
        include/fdeep/model.hpp:254-267, import_model.hpp:1990-2021"""
        for t in self.data.get("tests") or []:
            ins = [decode_floats(i["values"]).reshape(i["shape"]) for i in t["inputs"]]
            outs = self.predict(ins)
            for o, ref in zip(outs, t["outputs"]):
                r = decode_floats(ref["values"]).reshape(ref["shape"])
                bad = ~((np.abs(o.reshape(r.shape) - r) <= eps) | (np.isnan(o.reshape(r.shape)) & np.isnan(r)))
                if bad.any():
                    raise RuntimeError("test failed")
        return True


class CachedDecoder:
    """One sequence decoded token by token with the projected keys / values of every self-attention layer
    kept between steps: the CPU counterpart of a KV-cache decode session, used as the timed CPU baseline of
    the decode benchmark and as a second statement of the causal definition.

    Step t feeds (id, position t) through the layer graph as a one-row sample.  Every layer other than
    attention works on rows independently; a self-attention layer projects the new row with the layer's
    per-head Dense kernels (multi_head_attention_layer.hpp:47-59: q_w (D, H, dk) read as a Dense kernel
    [D][H*dk], o_w (H, dv, D) as [H*dv][D]), appends k and v to its cache and evaluates
    softmax(q K^T * 1/sqrt(dk)) V per head over the cached rows (same file :74-95, scale applied to the
    scores, softmax in the reference's exp(x - m - log sum) form), which is what the reference computes
    for MultiHeadAttention(query = x[t:t+1], value = x[0:t+1])."""

    def __init__(self, model):
        self.model = model
        self.cache = {}
        self.t = 0

    def _attend(self, layer, ins):
        c, w = layer.cfg, layer.p["w"]
        heads, dk = int(c["num_heads"]), int(c["key_dim"])
        dv = int(c.get("value_dim") or dk)
        if c["use_bias"]:
            qw, qb, kw, kb, vw, vb, ow, ob = w
        else:
            (qw, kw, vw, ow), qb, kb, vb, ob = w, None, None, None, None
        x = ins[0]
        assert x.shape[0] == 1 and all(i is ins[0] or np.array_equal(i, x) for i in ins[1:]), "self-attention on one new row"
        zk, zv = np.zeros(heads * dk, np.float32), np.zeros(heads * dv, np.float32)
        q = dense(x, qw, qb if qb is not None else zk, heads * dk)[0]
        k = dense(x, kw, kb if kb is not None else zk, heads * dk)[0]
        v = dense(x, vw, vb if vb is not None else zv, heads * dv)[0]
        ks, vs = self.cache.setdefault(layer.name, ([], []))
        ks.append(k)
        vs.append(v)
        K = np.stack(ks).reshape(len(ks), heads, dk)
        V = np.stack(vs).reshape(len(vs), heads, dv)
        scale = np.float32(1.0 / np.sqrt(float(dk)))
        merged = np.empty(heads * dv, np.float32)
        for h in range(heads):
            scores = (K[:, h, :] @ q[h * dk:(h + 1) * dk]).astype(np.float32) * scale
            merged[h * dv:(h + 1) * dv] = softmax(scores[None, :])[0] @ V[:, h, :]
        dout = ow.size // (heads * dv)
        return dense(merged[None, :], ow, ob if ob is not None else np.zeros(dout, np.float32), dout)

    def step(self, token):
        """Feeds one token id; returns the logits row for the next position."""
        ids = np.array([token], np.float32)
        pos = np.array([self.t], np.float32)
        out = self.model.graph.run([ids, pos], self._attend)[0]
        self.t += 1
        return out[-1]
