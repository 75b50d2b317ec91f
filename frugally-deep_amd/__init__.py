"""ctypes binding of libfdx.so, the C ABI declared in include/fdx.h.

The forward path runs only on the GPU through the HIP library; there is no CPU
fallback.  Importing this module without a built libfdx.so raises ImportError with the
build command (``python -c "import __graft_entry__ as g; g.build()"`` or
``make -C frugally-deep_amd/csrc``).
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# FDX_LIBRARY names another build of the same library (for comparing two builds in one session on one machine)
LIB_PATH = os.environ.get("FDX_LIBRARY") or os.path.join(_HERE, "libfdx.so")

c_float_p = ctypes.POINTER(ctypes.c_float)
c_void_pp = ctypes.POINTER(ctypes.c_void_p)

ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2
# config name -> FDX_ACT_* (include/fdx.h)
ACT_KINDS = {"tanh": 3, "sigmoid": 4, "swish": 5, "silu": 5, "hard_sigmoid": 6, "selu": 7, "elu": 8, "celu": 8, "exponential": 9,
             "softsign": 10, "softplus": 11, "leaky_relu": 12, "hard_shrink": 13, "soft_shrink": 14, "sparse_plus": 15,
             "squareplus": 16, "tanh_shrink": 17, "threshold": 18, "log_sigmoid": 19, "hard_tanh": 20, "log": 21}
COMBINE = {"add": 0, "mul": 1, "sub": 2, "max": 3, "min": 4, "prelu": 5}
FLT_MAX = float(np.finfo(np.float32).max)
PAD = {"valid": 0, "same": 1, "causal": 2}


class Act(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int), ("max_value", ctypes.c_float), ("negative_slope", ctypes.c_float),
                ("threshold", ctypes.c_float)]


class GemmBatch(ctypes.Structure):
    _fields_ = [("batch", ctypes.c_int), ("inner", ctypes.c_int)] + [
        (n, ctypes.c_int64) for n in ("a_outer", "a_inner", "b_outer", "b_inner", "c_outer", "c_inner")]


class FdxError(RuntimeError):
    pass


def build_library():
    import subprocess
    subprocess.check_call(["make", "-C", os.path.join(_HERE, "csrc"), "-j8"])


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError("libfdx.so is not built (run `make -C %s`); the fdx forward path has no fallback"
                          % os.path.join(_HERE, "csrc"))
    return ctypes.CDLL(LIB_PATH)


lib = _load()
lib.fdx_last_error.restype = ctypes.c_char_p
lib.fdx_set_last_error.restype = None
lib.fdx_mha_scratch_bytes.restype = ctypes.c_size_t


def check(status):
    if status != 0:
        raise FdxError(lib.fdx_last_error().decode("utf-8", "replace"))


def relu_act(max_value=None, negative_slope=0.0, threshold=0.0):
    return Act(ACT_RELU, FLT_MAX if max_value is None else max_value, negative_slope, threshold)


def named_act(name, p0=0.0, p1=0.0):
    """fdx_act for an activation by its config name; p0 / p1 as the oracle's activation(): alpha, slope, threshold, b,
    (threshold, default value)."""
    kind = ACT_KINDS[name]
    if name in ("elu", "celu", "leaky_relu"):
        return Act(kind, FLT_MAX, p0, 0.0)
    if name in ("hard_shrink", "soft_shrink"):
        return Act(kind, FLT_MAX, 0.0, p0)
    if name == "squareplus":
        return Act(kind, p0, 0.0, 0.0)
    if name == "threshold":
        return Act(kind, p1, 0.0, p0)
    return Act(kind, FLT_MAX, 0.0, 0.0)


def gelu_act():
    return Act(ACT_GELU, FLT_MAX, 0.0, 0.0)


def _act_ref(act):
    return None if act is None else ctypes.byref(act)


def tuner_export():
    """The per-shape tuning table of this process as text (fdx_tuner_export)."""
    need = ctypes.c_size_t()
    check(lib.fdx_tuner_export(None, ctypes.c_size_t(0), ctypes.byref(need)))
    buf = ctypes.create_string_buffer(need.value)
    check(lib.fdx_tuner_export(buf, ctypes.c_size_t(need.value), ctypes.byref(need)))
    return buf.value.decode()


def tuner_import(text):
    check(lib.fdx_tuner_import(text.encode()))


def model_check(json_text, unknown_extent=7):
    """The host half of loading a model file (parse, graph, parameter arrays, shapes) without touching a GPU
    (fdx_model_check); raises FdxError with the loader's message for a defective file."""
    data = json_text if isinstance(json_text, bytes) else json_text.encode()
    check(lib.fdx_model_check(data, ctypes.c_size_t(len(data)), ctypes.c_int64(unknown_extent)))


def tuner_timing(on=True):
    """Timing runs on the first sight of a shape (off unless asked for; FDX_AUTOTUNE=1 asks for them too)."""
    check(lib.fdx_tuner_timing(1 if on else 0))


def tuner_freeze(on=True):
    check(lib.fdx_tuner_freeze(1 if on else 0))


class DevBuf:
    """Device buffer owned by the library's allocator; holds fp32 (or raw bytes)."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = ctypes.c_void_p()
        check(lib.fdx_dev_alloc(ctypes.c_size_t(max(self.nbytes, 4)), ctypes.byref(p)))
        self.ptr = p

    @classmethod
    def from_host(cls, arr, dtype=np.float32):
        arr = np.ascontiguousarray(arr, dtype=dtype)
        buf = cls(arr.nbytes)
        if arr.nbytes:
            check(lib.fdx_h2d(buf.ptr, arr.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(arr.nbytes)))
        return buf

    def to_host(self, shape, dtype=np.float32):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes, (out.nbytes, self.nbytes)
        check(lib.fdx_d2h(out.ctypes.data_as(ctypes.c_void_p), self.ptr, ctypes.c_size_t(out.nbytes)))
        return out

    def free(self):
        if self.ptr:
            check(lib.fdx_dev_free(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _dp(buf):
    return None if buf is None else ctypes.cast(buf.ptr, c_float_p)


def sync():
    check(lib.fdx_sync())


def window_geometry(in_h, in_w, k_h, k_w, s_h, s_w, padding):
    g = (ctypes.c_int * 6)()
    check(lib.fdx_window_geometry(in_h, in_w, k_h, k_w, s_h, s_w, PAD[padding], g))
    return dict(pad_top=g[0], pad_bottom=g[1], pad_left=g[2], pad_right=g[3], out_h=g[4], out_w=g[5])


# ------------------------------------------------------------------ host-array conveniences
# Each takes numpy arrays, stages them in HBM, launches the kernel through the C ABI and returns numpy.

def conv2d(x, w, bias, strides=(1, 1), dilation=(1, 1), padding="valid", residual=None, act=None, extra_pad=None):
    """x [n,h,w,cin]; w in converted-JSON order [cout,kh,kw,cin]."""
    x = np.ascontiguousarray(x, np.float32)
    n, h, wd, cin = x.shape
    cout, kh, kw, _ = w.shape
    g = window_geometry(h, wd, (kh - 1) * dilation[0] + 1, (kw - 1) * dilation[1] + 1, strides[0], strides[1], padding)
    dx, dw = DevBuf.from_host(x), DevBuf.from_host(w)
    db = None if bias is None else DevBuf.from_host(bias)
    dr = None if residual is None else DevBuf.from_host(residual)
    out = DevBuf(4 * n * g["out_h"] * g["out_w"] * cout)
    check(lib.fdx_conv2d_nhwc_f32(_dp(dx), n, h, wd, cin, _dp(dw), _dp(db), cout, kh, kw, strides[0], strides[1],
                                  dilation[0], dilation[1], g["pad_top"], g["pad_left"], g["out_h"], g["out_w"],
                                  _dp(dr), _act_ref(act), _dp(out)))
    return out.to_host((n, g["out_h"], g["out_w"], cout))


def dwconv2d(x, w_chw, bias, strides=(1, 1), dilation=(1, 1), padding="valid", act=None):
    """x [n,h,w,c]; w in converted-JSON order [c,kh,kw] (re-laid to [kh,kw,c] here, as the loader does)."""
    x = np.ascontiguousarray(x, np.float32)
    n, h, wd, c = x.shape
    _, kh, kw = w_chw.shape
    g = window_geometry(h, wd, (kh - 1) * dilation[0] + 1, (kw - 1) * dilation[1] + 1, strides[0], strides[1], padding)
    dx, dw = DevBuf.from_host(x), DevBuf.from_host(np.transpose(w_chw, (1, 2, 0)))
    db = None if bias is None else DevBuf.from_host(bias)
    out = DevBuf(4 * n * g["out_h"] * g["out_w"] * c)
    check(lib.fdx_dwconv2d_nhwc_f32(_dp(dx), n, h, wd, c, _dp(dw), _dp(db), kh, kw, strides[0], strides[1],
                                    dilation[0], dilation[1], g["pad_top"], g["pad_left"], g["out_h"], g["out_w"],
                                    _act_ref(act), _dp(out)))
    return out.to_host((n, g["out_h"], g["out_w"], c))


def dwconv_pointwise(x, dw_w_chw, dw_bias, stride, padding, dw_act, pw_w_nc, pw_bias, residual=None, act=None):
    """Depthwise 3x3 then 1x1 convolution in one launch.  x [n,h,w,c]; dw_w_chw [c,3,3]; pw_w_nc [n_out,c]."""
    x = np.ascontiguousarray(x, np.float32)
    n, h, wd, c = x.shape
    g = window_geometry(h, wd, 3, 3, stride, stride, padding)
    n_out = pw_w_nc.shape[0]
    dx, dw = DevBuf.from_host(x), DevBuf.from_host(np.transpose(dw_w_chw, (1, 2, 0)))
    db = None if dw_bias is None else DevBuf.from_host(dw_bias)
    pw, pb = DevBuf.from_host(pw_w_nc), (None if pw_bias is None else DevBuf.from_host(pw_bias))
    dr = None if residual is None else DevBuf.from_host(residual)
    out = DevBuf(4 * n * g["out_h"] * g["out_w"] * n_out)
    check(lib.fdx_dwconv_pointwise_nhwc_f32(_dp(dx), n, h, wd, c, _dp(dw), _dp(db), stride, g["pad_top"], g["pad_left"],
                                            g["out_h"], g["out_w"], _act_ref(dw_act), _dp(pw), _dp(pb), n_out, _dp(dr),
                                            _act_ref(act), _dp(out)))
    return out.to_host((n, g["out_h"], g["out_w"], n_out))


def inverted_residual(x, exp_w_ec, exp_bias, exp_act, dw_w_chw, dw_bias, stride, padding, dw_act, pw_w_nc, pw_bias,
                      residual=None, act=None, zero_frame=(0, 0, 0, 0)):
    """1x1 expansion, depthwise 3x3, 1x1 projection in one launch.  x [n,h,w,cin]; exp_w_ec [ce,cin]; dw_w_chw [ce,3,3];
    pw_w_nc [n_out,ce]; zero_frame = (top, left, bottom, right) of an explicit ZeroPadding2D in front of the depthwise layer."""
    x = np.ascontiguousarray(x, np.float32)
    n, h, wd, cin = x.shape
    zt, zl, zb, zr = zero_frame
    g = window_geometry(h + zt + zb, wd + zl + zr, 3, 3, stride, stride, padding)
    ce, n_out = exp_w_ec.shape[0], pw_w_nc.shape[0]
    dx, ew = DevBuf.from_host(x), DevBuf.from_host(exp_w_ec)
    eb = None if exp_bias is None else DevBuf.from_host(exp_bias)
    dw = DevBuf.from_host(np.transpose(dw_w_chw, (1, 2, 0)))
    db = None if dw_bias is None else DevBuf.from_host(dw_bias)
    pw, pb = DevBuf.from_host(pw_w_nc), (None if pw_bias is None else DevBuf.from_host(pw_bias))
    dr = None if residual is None else DevBuf.from_host(residual)
    out = DevBuf(4 * n * g["out_h"] * g["out_w"] * n_out)
    check(lib.fdx_inverted_residual_nhwc_f32(_dp(dx), n, h, wd, cin, _dp(ew), _dp(eb), _act_ref(exp_act), ce, _dp(dw), _dp(db),
                                             stride, g["pad_top"] + zt, g["pad_left"] + zl, g["out_h"], g["out_w"], _act_ref(dw_act),
                                             _dp(pw), _dp(pb), n_out, _dp(dr), _act_ref(act), _dp(out)))
    return out.to_host((n, g["out_h"], g["out_w"], n_out))


def conv2d_winograd(x, w, bias, padding="same", residual=None, act=None):
    """3x3 stride-1 convolution in the Winograd F(2x2, 3x3) form.  x [n,h,w,cin]; w in converted-JSON order [cout,3,3,cin]."""
    x, w = np.ascontiguousarray(x, np.float32), np.ascontiguousarray(w, np.float32)
    n, h, wd, cin = x.shape
    cout = w.shape[0]
    assert w.shape[1:] == (3, 3, cin)
    g = window_geometry(h, wd, 3, 3, 1, 1, padding)
    lib.fdx_conv2d_winograd_weight_floats.restype = ctypes.c_size_t
    u = np.empty(lib.fdx_conv2d_winograd_weight_floats(cout, cin), np.float32)
    check(lib.fdx_conv2d_winograd_prepare(w.ctypes.data_as(c_float_p), cout, cin, u.ctypes.data_as(c_float_p)))
    dx, du = DevBuf.from_host(x), DevBuf.from_host(u)
    db = None if bias is None else DevBuf.from_host(bias)
    dr = None if residual is None else DevBuf.from_host(residual)
    out = DevBuf(4 * n * g["out_h"] * g["out_w"] * cout)
    check(lib.fdx_conv2d_winograd_nhwc_f32(_dp(dx), n, h, wd, cin, _dp(du), _dp(db), cout, g["pad_top"], g["pad_left"], g["out_h"],
                                           g["out_w"], _dp(dr), _act_ref(act), _dp(out)))
    return out.to_host((n, g["out_h"], g["out_w"], cout))


def stem_block(x, conv_w_nkkc, conv_bias, conv_act, conv_stride, conv_padding, dw_w_chw, dw_bias, stride, padding, dw_act,
               pw_w_nc, pw_bias, residual=None, act=None, conv_zero_frame=(0, 0, 0, 0), zero_frame=(0, 0, 0, 0)):
    """Small convolution on the image, depthwise 3x3, 1x1 projection in one launch.  x [n,ih,iw,ic]; conv_w_nkkc
    [ce,ek,ek,ic]; dw_w_chw [ce,3,3]; pw_w_nc [n_out,ce]; the zero frames = (top, left, bottom, right) of explicit
    ZeroPadding2D layers in front of the convolution / the depthwise layer."""
    x = np.ascontiguousarray(x, np.float32)
    n, ih, iw, ic = x.shape
    ce, ek = conv_w_nkkc.shape[0], conv_w_nkkc.shape[1]
    ct, cl, cb, cr = conv_zero_frame
    gc = window_geometry(ih + ct + cb, iw + cl + cr, ek, ek, conv_stride, conv_stride, conv_padding)
    h, w = gc["out_h"], gc["out_w"]
    zt, zl, zb, zr = zero_frame
    g = window_geometry(h + zt + zb, w + zl + zr, 3, 3, stride, stride, padding)
    n_out = pw_w_nc.shape[0]
    dx, cw = DevBuf.from_host(x), DevBuf.from_host(conv_w_nkkc)
    cbias = None if conv_bias is None else DevBuf.from_host(conv_bias)
    dw = DevBuf.from_host(np.transpose(dw_w_chw, (1, 2, 0)))
    db = None if dw_bias is None else DevBuf.from_host(dw_bias)
    pw, pb = DevBuf.from_host(pw_w_nc), (None if pw_bias is None else DevBuf.from_host(pw_bias))
    dr = None if residual is None else DevBuf.from_host(residual)
    out = DevBuf(4 * n * g["out_h"] * g["out_w"] * n_out)
    check(lib.fdx_stem_block_nhwc_f32(_dp(dx), n, ih, iw, ic, _dp(cw), _dp(cbias), _act_ref(conv_act), ce, ek, conv_stride,
                                      gc["pad_top"] + ct, gc["pad_left"] + cl, h, w, _dp(dw), _dp(db), stride, g["pad_top"] + zt,
                                      g["pad_left"] + zl, g["out_h"], g["out_w"], _act_ref(dw_act), _dp(pw), _dp(pb), n_out, _dp(dr),
                                      _act_ref(act), _dp(out)))
    return out.to_host((n, g["out_h"], g["out_w"], n_out))


def gemm(a, b_nk, bias=None, alpha=1.0, bias_per_row=False, residual=None, act=None):
    a, b_nk = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b_nk, np.float32)
    m, k = a.shape
    n = b_nk.shape[0]
    da, dbm = DevBuf.from_host(a), DevBuf.from_host(b_nk)
    dbias = None if bias is None else DevBuf.from_host(bias)
    dr = None if residual is None else DevBuf.from_host(residual)
    out = DevBuf(4 * m * n)
    check(lib.fdx_gemm_bias_act_f32(_dp(da), ctypes.c_int64(k), _dp(dbm), ctypes.c_int64(k), m, n, k,
                                    ctypes.c_float(alpha), _dp(dbias), int(bias_per_row), _dp(dr), _act_ref(act),
                                    _dp(out), ctypes.c_int64(n), None))
    return out.to_host((m, n))


def pool2d(x, pool, strides, padding, mode, zero_frame=(0, 0, 0, 0)):
    """zero_frame = (top, left, bottom, right) of an explicit ZeroPadding2D folded into the pool."""
    x = np.ascontiguousarray(x, np.float32)
    n, h, w, c = x.shape
    zt, zl, zb, zr = zero_frame
    g = window_geometry(h + zt + zb, w + zl + zr, pool[0], pool[1], strides[0], strides[1], padding)
    dx = DevBuf.from_host(x)
    out = DevBuf(4 * n * g["out_h"] * g["out_w"] * c)
    check(lib.fdx_pool2d_nhwc_f32(_dp(dx), n, h, w, c, pool[0], pool[1], strides[0], strides[1],
                                  g["pad_top"] + zt, g["pad_left"] + zl, zt, zl, zb, zr, g["out_h"], g["out_w"],
                                  0 if mode == "max" else 1, _dp(out)))
    return out.to_host((n, g["out_h"], g["out_w"], c))


def global_pool(x, mode):
    x = np.ascontiguousarray(x, np.float32)
    n, c = x.shape[0], x.shape[-1]
    pos = x.size // (n * c)
    dx, out = DevBuf.from_host(x), DevBuf(4 * n * c)
    check(lib.fdx_global_pool_f32(_dp(dx), n, pos, c, 0 if mode == "max" else 1, _dp(out)))
    return out.to_host((n, c))


def add(a, b, act=None):
    a, b = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
    da, db, out = DevBuf.from_host(a), DevBuf.from_host(b), DevBuf(a.nbytes)
    check(lib.fdx_eltwise_add_f32(_dp(da), _dp(db), ctypes.c_size_t(a.size), ctypes.c_size_t(b.size), _act_ref(act),
                                  _dp(out)))
    return out.to_host(a.shape)


def activation(x, act):
    x = np.ascontiguousarray(x, np.float32)
    dx, out = DevBuf.from_host(x), DevBuf(x.nbytes)
    check(lib.fdx_activation_f32(_dp(dx), ctypes.c_size_t(x.size), _act_ref(act), _dp(out)))
    return out.to_host(x.shape)


def channel_affine(x, scale, shift, act=None):
    x = np.ascontiguousarray(x, np.float32)
    c = x.shape[-1]
    dx, ds, dh, out = DevBuf.from_host(x), DevBuf.from_host(scale), DevBuf.from_host(shift), DevBuf(x.nbytes)
    check(lib.fdx_channel_affine_f32(_dp(dx), ctypes.c_size_t(x.size // c), c, _dp(ds), _dp(dh), _act_ref(act),
                                     _dp(out)))
    return out.to_host(x.shape)


def zero_pad2d(x, pt, pb, pl, pr):
    x = np.ascontiguousarray(x, np.float32)
    n, h, w, c = x.shape
    dx, out = DevBuf.from_host(x), DevBuf(4 * n * (h + pt + pb) * (w + pl + pr) * c)
    check(lib.fdx_zero_pad2d_nhwc_f32(_dp(dx), n, h, w, c, pt, pb, pl, pr, _dp(out)))
    return out.to_host((n, h + pt + pb, w + pl + pr, c))


def layernorm(x, gamma, beta, eps):
    x = np.ascontiguousarray(x, np.float32)
    d = x.shape[-1]
    dx, out = DevBuf.from_host(x), DevBuf(x.nbytes)
    dg = None if gamma is None else DevBuf.from_host(gamma)
    db = None if beta is None else DevBuf.from_host(beta)
    check(lib.fdx_layernorm_f32(_dp(dx), ctypes.c_int64(x.size // d), d, _dp(dg), _dp(db), ctypes.c_float(eps),
                                _dp(out)))
    return out.to_host(x.shape)


def _dims5(shape):
    shape = tuple(int(v) for v in shape)
    return (ctypes.c_int64 * 5)(*((1,) * (5 - len(shape)) + shape))


def layernorm_axes(x, axes, gamma, beta, eps):
    """x: (batch, ...sample dims); axes: 1-based positions in the sample's rank, negative from the end."""
    x = np.ascontiguousarray(x, np.float32)
    rank = x.ndim - 1
    mask = 0
    for a in axes:
        a = a + rank + 1 if a < 0 else a
        mask |= 1 << (5 - rank + a - 1)
    dx, out = DevBuf.from_host(x), DevBuf(x.nbytes)
    dg = None if gamma is None else DevBuf.from_host(gamma)
    db = None if beta is None else DevBuf.from_host(beta)
    check(lib.fdx_layernorm_axes_f32(_dp(dx), x.shape[0], _dims5(x.shape[1:]), ctypes.c_uint(mask), _dp(dg), _dp(db),
                                     ctypes.c_float(eps), _dp(out)))
    return out.to_host(x.shape)


def rmsnorm_axes(x, axes, scale, eps):
    x = np.ascontiguousarray(x, np.float32)
    rank = x.ndim - 1
    mask = 0
    for a in axes:
        a = a + rank + 1 if a < 0 else a
        mask |= 1 << (5 - rank + a - 1)
    dx, out = DevBuf.from_host(x), DevBuf(x.nbytes)
    ds = None if scale is None else DevBuf.from_host(scale)
    check(lib.fdx_rmsnorm_axes_f32(_dp(dx), x.shape[0], _dims5(x.shape[1:]), ctypes.c_uint(mask), _dp(ds), ctypes.c_float(eps),
                                   _dp(out)))
    return out.to_host(x.shape)


def conv2d_s2d(x, w, bias, padding="valid", residual=None, act=None, extra_pad=(0, 0)):
    """Stride-2 stem convolution through the space-to-depth path; x [n,h,w,c], w [cout,k,k,c]; extra_pad = (top, left)
    zero rows / columns of a folded ZeroPadding2D."""
    x, w = np.ascontiguousarray(x, np.float32), np.ascontiguousarray(w, np.float32)
    n, h, wd, cin = x.shape
    cout, k = w.shape[0], w.shape[1]
    if not lib.fdx_conv2d_s2d_eligible(cin, k, w.shape[2], 2, 2, 1, 1, cout):
        raise FdxError("shape not eligible for the space-to-depth path")
    g = window_geometry(h + 2 * extra_pad[0], wd + 2 * extra_pad[1], k, k, 2, 2, padding)
    lib.fdx_conv2d_s2d_weight_floats.restype = ctypes.c_size_t
    lib.fdx_conv2d_s2d_scratch_bytes.restype = ctypes.c_size_t
    w2 = np.empty(lib.fdx_conv2d_s2d_weight_floats(cout, cin, k), np.float32)
    check(lib.fdx_conv2d_s2d_prepare(w.ctypes.data_as(c_float_p), cout, cin, k, w2.ctypes.data_as(c_float_p)))
    dx, dw = DevBuf.from_host(x), DevBuf.from_host(w2)
    db = None if bias is None else DevBuf.from_host(np.ascontiguousarray(bias, np.float32))
    dr = None if residual is None else DevBuf.from_host(np.ascontiguousarray(residual, np.float32))
    oh, ow = g["out_h"], g["out_w"]
    scratch = DevBuf(lib.fdx_conv2d_s2d_scratch_bytes(n, oh, ow, cin, k))
    out = DevBuf(4 * n * oh * ow * cout)
    check(lib.fdx_conv2d_s2d_nhwc_f32(_dp(dx), n, h, wd, cin, _dp(dw), _dp(db), cout, k, g["pad_top"] + extra_pad[0], g["pad_left"] + extra_pad[1],
                                      oh, ow, _dp(dr), _act_ref(act), _dp(scratch), _dp(out)))
    return out.to_host((n, oh, ow, cout))


def permute(x, dims):
    """x: (batch, ...); dims: the Permute layer's 1-based axis list."""
    x = np.ascontiguousarray(x, np.float32)
    rank = x.ndim - 1
    d = (ctypes.c_int64 * rank)(*x.shape[1:])
    perm = (ctypes.c_int * rank)(*[v - 1 for v in dims])
    dx, out = DevBuf.from_host(x), DevBuf(x.nbytes)
    check(lib.fdx_permute_f32(_dp(dx), x.shape[0], rank, d, perm, _dp(out)))
    return out.to_host((x.shape[0],) + tuple(x.shape[v] for v in dims))


def crop2d(x, top, bottom, left, right):
    x = np.ascontiguousarray(x, np.float32)
    n, h, w, c = x.shape
    dx, out = DevBuf.from_host(x), DevBuf(4 * n * (h - top - bottom) * (w - left - right) * c)
    check(lib.fdx_crop2d_nhwc_f32(_dp(dx), n, h, w, c, top, bottom, left, right, _dp(out)))
    return out.to_host((n, h - top - bottom, w - left - right, c))


def upsample2d(x, factor_y, factor_x, bilinear=False):
    x = np.ascontiguousarray(x, np.float32)
    n, h, w, c = x.shape
    dx, out = DevBuf.from_host(x), DevBuf(4 * x.size * factor_y * factor_x)
    check(lib.fdx_upsample2d_nhwc_f32(_dp(dx), n, h, w, c, factor_y, factor_x, int(bilinear), _dp(out)))
    return out.to_host((n, h * factor_y, w * factor_x, c))


def dilate2d(x, rate_y, rate_x, trailing_zeros=False):
    x = np.ascontiguousarray(x, np.float32)
    n, h, w, c = x.shape
    extra = (rate_y - 1, rate_x - 1) if trailing_zeros and (rate_y, rate_x) != (1, 1) else (0, 0)
    oh, ow = (h - 1) * rate_y + 1 + extra[0], (w - 1) * rate_x + 1 + extra[1]
    dx, out = DevBuf.from_host(x), DevBuf(4 * n * oh * ow * c)
    check(lib.fdx_dilate2d_nhwc_f32(_dp(dx), n, h, w, c, rate_y, rate_x, int(trailing_zeros), _dp(out)))
    return out.to_host((n, oh, ow, c))


def broadcast_add(a, b, act=None):
    """a, b: (batch, ...sample dims) with right-aligned size-1 broadcasting between the samples."""
    a, b = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
    batch = a.shape[0]
    od = (ctypes.c_int64 * 5)()
    rank = max(a.ndim, b.ndim) - 1
    pa, pb = (1,) * (rank - a.ndim + 1) + a.shape[1:], (1,) * (rank - b.ndim + 1) + b.shape[1:]
    out = DevBuf(4 * batch * int(np.prod([max(x, y) for x, y in zip(pa, pb)])))
    da, db = DevBuf.from_host(a), DevBuf.from_host(b)
    check(lib.fdx_broadcast_add_f32(_dp(da), _dims5(a.shape[1:]), _dp(db), _dims5(b.shape[1:]), batch, _act_ref(act),
                                    _dp(out), od))
    got = tuple(od)[5 - rank:]
    return out.to_host((batch,) + got)


def broadcast_combine(op, a, b, b_shared=False, scale=1.0, act=None):
    """a: (batch, ...); b: (batch, ...) or, with b_shared, one tensor without a batch axis used for every sample."""
    a, b = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
    batch = a.shape[0]
    bs = b.shape if b_shared else b.shape[1:]
    rank = max(a.ndim - 1, len(bs))
    pa, pb = (1,) * (rank - a.ndim + 1) + a.shape[1:], (1,) * (rank - len(bs)) + tuple(bs)
    od = (ctypes.c_int64 * 5)()
    out = DevBuf(4 * batch * int(np.prod([max(x, y) for x, y in zip(pa, pb)])))
    da, db = DevBuf.from_host(a), DevBuf.from_host(b)
    check(lib.fdx_broadcast_combine_f32(COMBINE[op], _dp(da), _dims5(a.shape[1:]), _dp(db), _dims5(bs), int(b_shared), batch,
                                        ctypes.c_float(scale), _act_ref(act), _dp(out), od))
    return out.to_host((batch,) + tuple(od)[5 - rank:])


def concat(xs, axis):
    """xs: arrays of shape (batch, ...); axis: 1-based in the sample's rank (batch = 0), negative from the end."""
    xs = [np.ascontiguousarray(x, np.float32) for x in xs]
    rank = xs[0].ndim - 1
    a = axis + rank + 1 if axis < 0 else axis
    outer = int(np.prod(xs[0].shape[:a]))
    inner = (ctypes.c_int64 * len(xs))(*[int(np.prod(x.shape[a:])) for x in xs])
    bufs = [DevBuf.from_host(x) for x in xs]
    ptrs = (ctypes.c_void_p * len(xs))(*[b.ptr.value for b in bufs])
    shape = list(xs[0].shape)
    shape[a] = sum(x.shape[a] for x in xs)
    out = DevBuf(4 * int(np.prod(shape)))
    check(lib.fdx_concat_f32(ptrs, len(xs), inner, ctypes.c_int64(outer), _dp(out)))
    return out.to_host(tuple(shape))


def einsum_dense(x, equation, kernel, bias=None, bias_axes=None, full_output_shape=None, act=None):
    """x carries every lhs character it has (a leading batch is just the first one); returns the full rhs array."""
    x, kernel = np.ascontiguousarray(x, np.float32), np.ascontiguousarray(kernel, np.float32)
    rhs = equation.split("->")[1]
    dx, dk = DevBuf.from_host(x), DevBuf.from_host(kernel)
    db = None if bias is None else DevBuf.from_host(np.ascontiguousarray(bias, np.float32))
    lhs, ker = equation.split("->")[0].split(",")
    size = dict(zip(ker[len(ker) - kernel.ndim:], kernel.shape))
    size.update(zip(lhs[len(lhs) - x.ndim:], x.shape))
    for i, c in enumerate(rhs):
        if c not in size:
            size[c] = 1 if c in lhs else int(full_output_shape[i])
    out = DevBuf(4 * int(np.prod([size[c] for c in rhs])))
    in_dims = (ctypes.c_int64 * x.ndim)(*x.shape)
    k_dims = (ctypes.c_int64 * kernel.ndim)(*kernel.shape)
    full = None if full_output_shape is None else (ctypes.c_int64 * len(rhs))(*[int(v) for v in full_output_shape])
    orank, odims = ctypes.c_int(0), (ctypes.c_int64 * 6)()
    check(lib.fdx_einsum_dense_f32(equation.encode(), (bias_axes or "").encode(), _dp(dx), x.ndim, in_dims, _dp(dk),
                                   kernel.ndim, k_dims, _dp(db), full, _act_ref(act), _dp(out), ctypes.byref(orank), odims))
    return out.to_host(tuple(odims)[:orank.value])


def softmax(x, causal_period=0, causal_offset=0):
    x = np.ascontiguousarray(x, np.float32)
    d = x.shape[-1]
    dx, out = DevBuf.from_host(x), DevBuf(x.nbytes)
    check(lib.fdx_softmax_f32(_dp(dx), ctypes.c_int64(x.size // d), d, causal_period, causal_offset, _dp(out)))
    return out.to_host(x.shape)


def embedding(ids, table):
    ids = np.ascontiguousarray(ids, np.float32).reshape(-1)
    table = np.ascontiguousarray(table, np.float32)
    di, dt, out = DevBuf.from_host(ids), DevBuf.from_host(table), DevBuf(4 * ids.size * table.shape[1])
    flag = DevBuf.from_host(np.zeros(1, np.int32), np.int32)
    check(lib.fdx_embedding_f32(_dp(di), ctypes.c_int64(ids.size), _dp(dt), table.shape[0], table.shape[1], _dp(out),
                                ctypes.cast(flag.ptr, ctypes.POINTER(ctypes.c_int))))
    if flag.to_host((1,), np.int32)[0]:
        raise FdxError("vocabulary item indices must all be strictly less than the value of input_dim")
    return out.to_host((ids.size, table.shape[1]))


def argmax(x):
    x = np.ascontiguousarray(x, np.float32)
    d = x.shape[-1]
    rows = x.size // d
    dx, oi, ov = DevBuf.from_host(x), DevBuf(4 * rows), DevBuf(4 * rows)
    check(lib.fdx_argmax_f32(_dp(dx), ctypes.c_int64(rows), d, ctypes.cast(oi.ptr, ctypes.POINTER(ctypes.c_int32)),
                             _dp(ov)))
    return oi.to_host((rows,), np.int32), ov.to_host((rows,))


def mha_prefill(q, k, v, heads, dk, dv, causal=False):
    """q [b,t,heads*dk], k [b,s,heads*dk], v [b,s,heads*dv] (already projected)."""
    q, k, v = (np.ascontiguousarray(a, np.float32) for a in (q, k, v))
    b, t, _ = q.shape
    s = k.shape[1]
    dq, dk_, dv_ = DevBuf.from_host(q), DevBuf.from_host(k), DevBuf.from_host(v)
    scratch = DevBuf(lib.fdx_mha_scratch_bytes(b, heads, t, s, dv))
    out = DevBuf(4 * b * t * heads * dv)
    check(lib.fdx_mha_prefill_f32(_dp(dq), _dp(dk_), _dp(dv_), b, t, s, heads, dk, dv, int(causal), _dp(out),
                                  scratch.ptr))
    return out.to_host((b, t, heads * dv))


def mha_decode(q, k_cache, v_cache, heads, dk, dv, length):
    """q [b,heads*dk]; caches [b,max_len,heads*dk|dv]."""
    q, k_cache, v_cache = (np.ascontiguousarray(a, np.float32) for a in (q, k_cache, v_cache))
    b, max_len = k_cache.shape[0], k_cache.shape[1]
    dq, dkc, dvc = DevBuf.from_host(q), DevBuf.from_host(k_cache), DevBuf.from_host(v_cache)
    out = DevBuf(4 * b * heads * dv)
    check(lib.fdx_mha_decode_f32(_dp(dq), _dp(dkc), _dp(dvc), b, heads, dk, dv, length, max_len, _dp(out)))
    return out.to_host((b, heads * dv))


# ------------------------------------------------------------------ whole models

_PARAM_GETTER = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p,
                                 ctypes.POINTER(ctypes.POINTER(ctypes.c_float)), ctypes.POINTER(ctypes.c_size_t))
_CREATE_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_void_p, ctypes.c_size_t, _PARAM_GETTER,
                              ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p))
_APPLY_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.POINTER(ctypes.c_float)),
                             ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_float),
                             ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int64))
_DESTROY_FN = ctypes.CFUNCTYPE(None, ctypes.c_void_p)


class _CustomLayerStruct(ctypes.Structure):
    _fields_ = [("class_name", ctypes.c_char_p), ("create", _CREATE_FN), ("apply", _APPLY_FN), ("destroy", _DESTROY_FN),
                ("user", ctypes.c_void_p)]


class _CustomLayers:
    """ctypes glue for fdx_custom_layer: `creators` maps a class name to creator(get_param, layer_dict, name) -> callable
    that takes the list of input arrays (no batch axis) and returns one array."""

    def __init__(self, creators):
        import json as _json
        self.instances = {}
        self.keep = []
        self.errors = []
        structs = []
        for cls_name, creator in creators.items():
            def create(user, lname, cfg, cfg_len, getter, gctx, inst, creator=creator):
                try:
                    def get_param(layer, key):
                        vals, cnt = ctypes.POINTER(ctypes.c_float)(), ctypes.c_size_t()
                        check(getter(gctx, layer.encode(), key.encode(), ctypes.byref(vals), ctypes.byref(cnt)))
                        return np.ctypeslib.as_array(vals, (cnt.value,)).copy()
                    fn = creator(get_param, _json.loads(ctypes.string_at(cfg, cfg_len)), lname.decode())
                    handle = len(self.instances) + 1
                    self.instances[handle] = fn
                    inst[0] = handle
                    return 0
                except Exception as e:  # noqa: BLE001 - reported through the status code
                    self.errors.append(e)
                    lib.fdx_set_last_error(str(e).encode())
                    return 1

            def apply(inst, n, ins, ranks, dims5, out, orank, odims):
                try:
                    arrs = []
                    for i in range(n):
                        shape = tuple(int(dims5[i * 5 + k]) for k in range(5 - ranks[i], 5))
                        arrs.append(np.ctypeslib.as_array(ins[i], shape).copy())
                    y = np.ascontiguousarray(self.instances[inst](arrs), np.float32)
                    orank[0] = y.ndim
                    for k in range(5):
                        odims[k] = 1 if k < 5 - y.ndim else y.shape[k - (5 - y.ndim)]
                    if out:
                        ctypes.memmove(out, y.ctypes.data, y.nbytes)
                    return 0
                except Exception as e:  # noqa: BLE001
                    self.errors.append(e)
                    lib.fdx_set_last_error(str(e).encode())
                    return 1

            def destroy(inst):
                self.instances.pop(inst, None)

            fns = (_CREATE_FN(create), _APPLY_FN(apply), _DESTROY_FN(destroy))
            self.keep.append(fns)
            structs.append(_CustomLayerStruct(cls_name.encode(), fns[0], fns[1], fns[2], None))
        self.array = (_CustomLayerStruct * len(structs))(*structs)
        self.count = len(structs)


class Model:
    """A converted-JSON model resident on the GPU (fdx_model_*).  `source` is the file's bytes or a path."""

    def __init__(self, source, verify=True, verify_epsilon=1e-4, custom_layers=None):
        if isinstance(source, str):
            if not os.path.exists(source):
                raise FdxError("Can not open " + source)
            with open(source, "rb") as f:
                source = f.read()
        self._h = ctypes.c_void_p()
        self._custom = _CustomLayers(custom_layers) if custom_layers else None
        if self._custom:
            check(lib.fdx_model_create_custom(source, ctypes.c_size_t(len(source)), int(verify), ctypes.c_float(verify_epsilon),
                                              self._custom.array, self._custom.count, ctypes.byref(self._h)))
        else:
            check(lib.fdx_model_create(source, ctypes.c_size_t(len(source)), int(verify), ctypes.c_float(verify_epsilon),
                                       ctypes.byref(self._h)))
        ni, no = ctypes.c_int(), ctypes.c_int()
        check(lib.fdx_model_io_count(self._h, ctypes.byref(ni), ctypes.byref(no)))
        self.n_inputs, self.n_outputs = ni.value, no.value
        self.input_shapes = [self._io_shape(0, i) for i in range(self.n_inputs)]
        self.output_shapes = [self._io_shape(1, i) for i in range(self.n_outputs)]
        name, hsh = ctypes.c_char_p(), ctypes.c_char_p()
        check(lib.fdx_model_name(self._h, ctypes.byref(name), ctypes.byref(hsh)))
        self.name, self.hash = name.value.decode(), hsh.value.decode()

    def _io_shape(self, is_output, index):
        rank, dims = ctypes.c_int(), (ctypes.c_int64 * 5)()
        check(lib.fdx_model_io_shape(self._h, is_output, index, ctypes.byref(rank), dims))
        return tuple(None if d < 0 else int(d) for d in list(dims)[5 - rank.value:])

    def _dims(self, shapes):
        dims = (ctypes.c_int64 * (5 * len(shapes)))(*([1] * (5 * len(shapes))))
        ranks = (ctypes.c_int * len(shapes))()
        for i, s in enumerate(shapes):
            ranks[i] = len(s)
            for k, d in enumerate(s):
                dims[i * 5 + 5 - len(s) + k] = d
        return dims, ranks

    def infer_shapes(self, sample_shapes):
        dims, ranks = self._dims(sample_shapes)
        od, orank = (ctypes.c_int64 * (5 * self.n_outputs))(), (ctypes.c_int * self.n_outputs)()
        check(lib.fdx_model_infer_shapes(self._h, dims, ranks, od, orank))
        return [tuple(int(d) for d in od[i * 5 + 5 - orank[i]:i * 5 + 5]) for i in range(self.n_outputs)]

    def predict(self, inputs):
        """inputs: one array per model input, shaped [batch, *sample_shape]; returns arrays [batch, *out_shape].
        All samples go through one batched launch sequence (predict_multi semantics)."""
        inputs = [np.ascontiguousarray(x, np.float32) for x in inputs]
        if len(inputs) != self.n_inputs:
            raise FdxError("Invalid inputs shape.\nThe model takes %d inputs" % self.n_inputs)
        batch = inputs[0].shape[0]
        sample_shapes = [x.shape[1:] for x in inputs]
        dims, ranks = self._dims(sample_shapes)
        out_shapes = self.infer_shapes(sample_shapes)
        outs = [np.empty((batch,) + s, np.float32) for s in out_shapes]
        ip = (c_float_p * self.n_inputs)(*[x.ctypes.data_as(c_float_p) for x in inputs])
        op = (c_float_p * self.n_outputs)(*[o.ctypes.data_as(c_float_p) for o in outs])
        check(lib.fdx_model_predict(self._h, batch, ip, dims, ranks, op, None, None))
        return outs

    def predict_samples(self, samples):
        """samples[b][i] = the array of input i of sample b (the form fdeep::model::predict_multi takes): every sample
        stays where it is, the library gathers them on their way to the GPU (fdx_model_predict_samples)."""
        batch = len(samples)
        held = [[np.ascontiguousarray(samples[b][i], np.float32) for b in range(batch)] for i in range(self.n_inputs)]
        sample_shapes = [held[i][0].shape for i in range(self.n_inputs)]
        dims, ranks = self._dims(sample_shapes)
        out_shapes = self.infer_shapes(sample_shapes)
        outs = [np.empty((batch,) + s, np.float32) for s in out_shapes]
        ip = (c_float_p * (self.n_inputs * batch))(*[held[i][b].ctypes.data_as(c_float_p) for i in range(self.n_inputs)
                                                      for b in range(batch)])
        op = (c_float_p * self.n_outputs)(*[o.ctypes.data_as(c_float_p) for o in outs])
        check(lib.fdx_model_predict_samples(self._h, batch, ip, dims, ranks, op, None, None))
        return outs

    def predict_dev(self, batch, in_bufs, sample_shapes, out_bufs):
        """Device-resident variant: in_bufs / out_bufs are DevBuf objects; asynchronous (call sync())."""
        dims, ranks = self._dims(sample_shapes)
        ip = (c_float_p * self.n_inputs)(*[_dp(b) for b in in_bufs])
        op = (c_float_p * self.n_outputs)(*[_dp(b) for b in out_bufs])
        check(lib.fdx_model_predict_dev(self._h, batch, ip, dims, ranks, op, None, None))

    def last_flops(self):
        f = ctypes.c_double()
        check(lib.fdx_model_last_flops(self._h, ctypes.byref(f)))
        return f.value

    def close(self):
        if self._h:
            check(lib.fdx_model_destroy(self._h))
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Session:
    """Autoregressive decoding with a key/value cache over a decoder Model (fdx_session_*)."""

    def __init__(self, model, batch, max_len):
        self.model, self.batch, self.max_len = model, batch, max_len
        self.vocab = model.output_shapes[0][-1]
        self._h = ctypes.c_void_p()
        check(lib.fdx_session_create(model._h, batch, max_len, ctypes.byref(self._h)))

    def length(self):
        n = ctypes.c_int()
        check(lib.fdx_session_length(self._h, ctypes.byref(n)))
        return n.value

    def reset(self):
        check(lib.fdx_session_reset(self._h))

    def prefill(self, ids):
        """ids [batch, t]; returns (logits [batch, vocab] of the last position, greedy next ids [batch])."""
        ids = np.ascontiguousarray(ids, np.float32)
        assert ids.shape[0] == self.batch
        d_ids, d_log, d_next = DevBuf.from_host(ids), DevBuf(4 * self.batch * self.vocab), DevBuf(4 * self.batch)
        check(lib.fdx_session_prefill(self._h, _dp(d_ids), ids.shape[1], _dp(d_log), _dp(d_next)))
        return d_log.to_host((self.batch, self.vocab)), d_next.to_host((self.batch,)).astype(np.int64)

    def decode_step(self, ids):
        ids = np.ascontiguousarray(ids, np.float32).reshape(self.batch)
        d_ids, d_log, d_next = DevBuf.from_host(ids), DevBuf(4 * self.batch * self.vocab), DevBuf(4 * self.batch)
        check(lib.fdx_session_decode_step(self._h, _dp(d_ids), _dp(d_log), _dp(d_next)))
        return d_log.to_host((self.batch, self.vocab)), d_next.to_host((self.batch,)).astype(np.int64)

    def decode_greedy(self, first_ids, steps):
        """Feeds each step's argmax back in; returns (tokens [steps, batch], logits of the last step)."""
        first = np.ascontiguousarray(first_ids, np.float32).reshape(self.batch)
        d_first, d_tok = DevBuf.from_host(first), DevBuf(4 * steps * self.batch)
        d_log = DevBuf(4 * self.batch * self.vocab)
        check(lib.fdx_session_decode_greedy(self._h, _dp(d_first), steps, _dp(d_tok), _dp(d_log)))
        return d_tok.to_host((steps, self.batch)).astype(np.int64), d_log.to_host((self.batch, self.vocab))

    def close(self):
        if self._h:
            check(lib.fdx_session_destroy(self._h))
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
