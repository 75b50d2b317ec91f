"""Pins the CPU oracle (oracle/oracle.c) against independent statements of the same
mathematics: brute-force loops, fp64 numpy/scipy/torch-CPU library routines and closed
forms.  None of these reuse the oracle's own formulas."""
import itertools
import math

import numpy as np
import pytest
import torch
from scipy import special

TOL = 2e-5


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def tf_geometry(n, k, s, padding):
    """TensorFlow's documented rule, written independently of the reference's code path."""
    if padding == "same":
        out = -(-n // s)
        total = max((out - 1) * s + k - n, 0)
        return out, total // 2, total - total // 2
    return (n - k) // s + 1 if n >= k else 0, 0, 0


@pytest.mark.parametrize("padding", ["same", "valid"])
def test_window_geometry_table(oracle, padding):
    for n, k, s in itertools.product(range(1, 12), range(1, 6), range(1, 4)):
        if padding == "valid" and n < k:
            continue
        g = oracle.window_geometry(n, n + 1, k, k, s, s, padding)
        out, before, after = tf_geometry(n, k, s, padding)
        assert (g["out_h"], g["pad_top"], g["pad_bottom"]) == (out, before, after), (n, k, s)
        out, before, after = tf_geometry(n + 1, k, s, padding)
        assert (g["out_w"], g["pad_left"], g["pad_right"]) == (out, before, after), (n, k, s)


def test_window_geometry_causal(oracle):
    g = oracle.window_geometry(7, 9, 3, 5, 1, 1, "causal")
    assert (g["pad_top"], g["pad_bottom"], g["pad_left"], g["pad_right"]) == (2, 0, 4, 0)
    assert (g["out_h"], g["out_w"]) == (7, 9)


def torch_conv(x, w_oihw, b, strides, dilation, padding, groups=1):
    import torch
    import torch.nn.functional as F
    h, w = x.shape[:2]
    kh, kw = w_oihw.shape[2:]
    ek = ((kh - 1) * dilation[0] + 1, (kw - 1) * dilation[1] + 1)
    pads = []
    for n, k, s in ((w, ek[1], strides[1]), (h, ek[0], strides[0])):
        _, before, after = tf_geometry(n, k, s, padding)
        pads += [before, after]
    xt = torch.from_numpy(x.astype(np.float64)).permute(2, 0, 1)[None]
    xt = F.pad(xt, pads)
    y = F.conv2d(xt, torch.from_numpy(w_oihw.astype(np.float64)),
                 None if b is None else torch.from_numpy(b.astype(np.float64)),
                 stride=strides, dilation=dilation, groups=groups)
    return y[0].permute(1, 2, 0).numpy()


CONV_CASES = [
    # h, w, cin, cout, kh, kw, strides, dilation, padding
    (8, 9, 3, 5, 3, 3, (1, 1), (1, 1), "same"),
    (8, 9, 3, 5, 3, 3, (1, 1), (1, 1), "valid"),
    (11, 10, 4, 6, 3, 2, (2, 2), (1, 1), "same"),
    (11, 10, 4, 6, 3, 2, (2, 3), (1, 1), "valid"),
    (12, 12, 2, 3, 3, 3, (1, 1), (2, 2), "same"),
    (12, 13, 2, 3, 2, 3, (1, 1), (2, 3), "valid"),
    (9, 9, 8, 4, 1, 1, (1, 1), (1, 1), "valid"),
    (9, 9, 8, 4, 1, 1, (2, 2), (1, 1), "same"),
    (15, 15, 3, 8, 7, 7, (2, 2), (1, 1), "valid"),
    (6, 7, 5, 7, 5, 5, (1, 1), (1, 1), "same"),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_vs_torch_fp64(oracle, case):
    h, w, cin, cout, kh, kw, strides, dilation, padding = case
    rng = np.random.default_rng(hash(case) % 2**32)
    x = rng.standard_normal((h, w, cin)).astype(np.float32)
    wj = rng.standard_normal((cout, kh, kw, cin)).astype(np.float32)  # converted-JSON order
    b = rng.standard_normal(cout).astype(np.float32)
    got = oracle.conv2d(x, oracle.conv2d_prepare(wj, cout, kh, kw, cin), b, cout, kh, kw, strides, dilation, padding)
    want = torch_conv(x, wj.transpose(0, 3, 1, 2), b, strides, dilation, padding)
    assert got.shape == want.shape
    assert rel(got, want) < TOL


def test_conv2d_brute_force(oracle):
    rng = np.random.default_rng(3)
    h, w, cin, cout, k = 5, 6, 2, 3, 3
    x = rng.standard_normal((h, w, cin)).astype(np.float32)
    wj = rng.standard_normal((cout, k, k, cin)).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    got = oracle.conv2d(x, oracle.conv2d_prepare(wj, cout, k, k, cin), b, cout, k, k, (1, 1), (1, 1), "valid")
    want = np.zeros((h - 2, w - 2, cout))
    for y, xx, n, fy, fx, c in itertools.product(range(h - 2), range(w - 2), range(cout), range(k), range(k), range(cin)):
        want[y, xx, n] += float(wj[n, fy, fx, c]) * float(x[y + fy, xx + fx, c])
    want += b
    assert rel(got, want) < TOL


def test_conv2d_closed_forms(oracle):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((6, 7, 4)).astype(np.float32)
    # 1x1 conv == matmul over channels
    wj = rng.standard_normal((5, 1, 1, 4)).astype(np.float32)
    got = oracle.conv2d(x, oracle.conv2d_prepare(wj, 5, 1, 1, 4), None, 5, 1, 1)
    assert rel(got, x.astype(np.float64) @ wj.reshape(5, 4).T.astype(np.float64)) < TOL
    # all-ones 3x3 kernel on one channel == box sum; same padding keeps size
    x1 = x[:, :, :1]
    got = oracle.conv2d(x1, np.ones(9, np.float32), None, 1, 3, 3, padding="same")
    padded = np.pad(x1[:, :, 0].astype(np.float64), 1)
    want = sum(padded[i:i + 6, j:j + 7] for i in range(3) for j in range(3))
    assert rel(got[:, :, 0], want) < TOL
    # delta kernel at (0, 2) == shift (cross-correlation, no flip)
    delta = np.zeros((1, 3, 3, 1), np.float32)
    delta[0, 0, 2, 0] = 1
    got = oracle.conv2d(x1, oracle.conv2d_prepare(delta, 1, 3, 3, 1), None, 1, 3, 3, padding="valid")
    assert np.array_equal(got[:, :, 0], x1[0:4, 2:7, 0])


def torch_conv_transpose_full(x, wj, b, strides, dilation):
    """Scatter form in fp64: out[y*s + ky*d, x*s + kx*d, co] += in[y, x, ci] * K[co, ky, kx, ci] (+ bias)."""
    import torch.nn.functional as F
    xt = torch.from_numpy(x.astype(np.float64)).permute(2, 0, 1)[None]
    wt = torch.from_numpy(wj.astype(np.float64)).permute(3, 0, 1, 2)  # [cin][cout][kh][kw]
    y = F.conv_transpose2d(xt, wt, None if b is None else torch.from_numpy(b.astype(np.float64)),
                           stride=strides, dilation=dilation)
    return y[0].permute(1, 2, 0).numpy()


TRANSPOSE_CASES = [
    # h, w, cin, cout, kh, kw, strides, dilation
    (5, 6, 3, 4, 3, 3, (1, 1), (1, 1)),
    (5, 6, 3, 4, 3, 3, (2, 2), (1, 1)),
    (4, 7, 2, 5, 4, 2, (2, 3), (1, 1)),
    (6, 5, 4, 3, 5, 5, (3, 2), (1, 1)),
    (5, 5, 2, 3, 3, 2, (2, 2), (2, 2)),
    (1, 9, 3, 4, 1, 3, (1, 2), (1, 1)),   # Conv1DTranspose seen as a height-1 image
    (4, 4, 3, 2, 1, 1, (3, 3), (1, 1)),
    (4, 5, 3, 2, 2, 2, (3, 4), (1, 1)),
]


@pytest.mark.parametrize("case", TRANSPOSE_CASES)
def test_conv2d_transpose_valid_vs_torch_fp64(oracle, case):
    h, w, cin, cout, kh, kw, strides, dilation = case
    rng = np.random.default_rng(hash(case) % 2**32)
    x = rng.standard_normal((h, w, cin)).astype(np.float32)
    wj = rng.standard_normal((cout, kh, kw, cin)).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    got = oracle.conv2d_transpose(x, oracle.conv2d_transpose_prepare(wj, cout, kh, kw, cin), b, cout, kh, kw,
                                  strides, dilation, "valid")
    want = torch_conv_transpose_full(x, wj, b, strides, dilation)
    assert got.shape == want.shape
    assert rel(got, want) < TOL


@pytest.mark.parametrize("case", [c for c in TRANSPOSE_CASES if c[7] == (1, 1) and c[4] >= c[6][0] and c[5] >= c[6][1]])
def test_conv2d_transpose_same_is_input_gradient_of_same_conv(oracle, case):
    # TensorFlow defines the layer as the input gradient of the strided "same" convolution whose output is x:
    # an image of (h*sy, w*sx) pixels convolved with the same kernel (cin and cout swapped) gives (h, w).
    import torch.nn.functional as F
    h, w, cin, cout, kh, kw, strides, _ = case
    rng = np.random.default_rng(hash(case) % 2**32 + 1)
    x = rng.standard_normal((h, w, cin)).astype(np.float32)
    wj = rng.standard_normal((cout, kh, kw, cin)).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    got = oracle.conv2d_transpose(x, oracle.conv2d_transpose_prepare(wj, cout, kh, kw, cin), b, cout, kh, kw,
                                  strides, (1, 1), "same")
    big = torch.zeros(1, cout, h * strides[0], w * strides[1], dtype=torch.float64, requires_grad=True)
    pads = []
    for n, k, s in ((w * strides[1], kw, strides[1]), (h * strides[0], kh, strides[0])):
        _, before, after = tf_geometry(n, k, s, "same")
        pads += [before, after]
    # forward filter of that convolution: [out = cin of the layer][in = cout of the layer][kh][kw]
    fwd = torch.from_numpy(wj.astype(np.float64)).permute(3, 0, 1, 2)
    y = F.conv2d(F.pad(big, pads), fwd, stride=strides)
    assert tuple(y.shape[2:]) == (h, w)
    (grad,) = torch.autograd.grad(y, big, torch.from_numpy(x.astype(np.float64)).permute(2, 0, 1)[None])
    want = grad[0].permute(1, 2, 0).numpy() + b.astype(np.float64)
    assert got.shape == want.shape
    assert rel(got, want) < TOL


@pytest.mark.parametrize("case", TRANSPOSE_CASES)
def test_conv2d_transpose_same_is_a_window_of_the_full_result(oracle, case):
    # "same" keeps h*sy x w*sx pixels of the full ("valid") result; the window starts where the reference's padding
    # puts it (convolution.hpp:366-377 on the zero-stuffed input of tensor.hpp:619-626), which for kernels smaller
    # than the stride lies one zero row / column before the full result.
    h, w, cin, cout, kh, kw, strides, dilation = case
    rng = np.random.default_rng(hash(case) % 2**32 + 2)
    x = rng.standard_normal((h, w, cin)).astype(np.float32)
    wj = rng.standard_normal((cout, kh, kw, cin)).astype(np.float32)
    got = oracle.conv2d_transpose(x, oracle.conv2d_transpose_prepare(wj, cout, kh, kw, cin), None, cout, kh, kw,
                                  strides, dilation, "same")
    full = torch_conv_transpose_full(x, wj, None, strides, dilation)
    assert got.shape == (h * strides[0], w * strides[1], cout)
    starts = []
    for k, d, s in ((kh, dilation[0], strides[0]), (kw, dilation[1], strides[1])):
        ek = (k - 1) * d + 1
        lead = 0 if strides == (1, 1) else (s - 1) - (s - 1) // 2
        starts.append((ek - 1) - lead - (ek - 1) // 2)
    big = np.zeros((full.shape[0] + 2 * 8, full.shape[1] + 2 * 8, cout))
    big[8:8 + full.shape[0], 8:8 + full.shape[1]] = full
    want = big[8 + starts[0]:8 + starts[0] + got.shape[0], 8 + starts[1]:8 + starts[1] + got.shape[1]]
    assert rel(got, want) < TOL


def test_conv2d_transpose_rejects_causal(oracle):
    x = np.ones((4, 4, 1), np.float32)
    with pytest.raises(RuntimeError):
        oracle.conv2d_transpose(x, np.ones(4, np.float32), None, 1, 2, 2, (1, 1), (1, 1), "causal")


@pytest.mark.parametrize("case", [
    (9, 8, 6, 3, 3, (1, 1), (1, 1), "same"), (9, 8, 6, 3, 3, (2, 2), (1, 1), "same"),
    (10, 11, 5, 3, 3, (2, 2), (1, 1), "valid"), (12, 12, 4, 3, 3, (1, 1), (2, 2), "same"),
    (7, 7, 3, 5, 2, (1, 2), (1, 1), "valid")])
def test_depthwise_vs_torch_fp64(oracle, case):
    h, w, c, kh, kw, strides, dilation, padding = case
    rng = np.random.default_rng(hash(case) % 2**32)
    x = rng.standard_normal((h, w, c)).astype(np.float32)
    wj = rng.standard_normal((c, kh, kw)).astype(np.float32)
    b = rng.standard_normal(c).astype(np.float32)
    got = oracle.depthwise_conv2d(x, wj, b, kh, kw, strides, dilation, padding)
    want = torch_conv(x, wj[:, None], b, strides, dilation, padding, groups=c)
    assert got.shape == want.shape
    assert rel(got, want) < TOL


def test_dense_any_rank(oracle):
    rng = np.random.default_rng(5)
    w = rng.standard_normal((7, 4)).astype(np.float32)
    b = rng.standard_normal(4).astype(np.float32)
    for shape in [(7,), (3, 7), (2, 3, 7), (2, 2, 3, 7)]:
        x = rng.standard_normal(shape).astype(np.float32)
        got = oracle.dense(x, w.reshape(-1), b, 4)
        assert got.shape == shape[:-1] + (4,)
        assert rel(got, x.astype(np.float64) @ w.astype(np.float64) + b) < TOL


def test_softmax_vs_scipy(oracle):
    from scipy.special import softmax
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((5, 3, 17)) * 8).astype(np.float32)
    assert rel(oracle.softmax(x), softmax(x.astype(np.float64), axis=-1)) < TOL
    big = np.array([[1000.0, -1000.0, 999.0]], np.float32)
    got = oracle.softmax(big)
    assert np.isfinite(got).all() and abs(got.sum() - 1) < 1e-6


@pytest.mark.parametrize("affine", [True, False])
def test_layernorm_vs_torch(oracle, affine):
    import torch
    rng = np.random.default_rng(7)
    x = (rng.standard_normal((6, 33)) * 3 + 1).astype(np.float32)
    g = rng.standard_normal(33).astype(np.float32) if affine else None
    b = rng.standard_normal(33).astype(np.float32) if affine else None
    want = torch.nn.functional.layer_norm(
        torch.from_numpy(x.astype(np.float64)), (33,),
        None if g is None else torch.from_numpy(g.astype(np.float64)),
        None if b is None else torch.from_numpy(b.astype(np.float64)), eps=1e-3).numpy()
    assert rel(oracle.layernorm(x, g, b, 1e-3), want) < TOL
    # two trailing axes normalised together == layer norm of the flattened rows
    x3 = x.reshape(2, 3, 33)
    got = oracle.layernorm(x3, None, None, 1e-3, n_axes=2)
    flat = x3.reshape(2, 99).astype(np.float64)
    want = (flat - flat.mean(1, keepdims=True)) / np.sqrt(flat.var(1, keepdims=True) + 1e-3)
    assert rel(got.reshape(2, 99), want) < TOL


def test_batchnorm_formula(oracle):
    rng = np.random.default_rng(8)
    x = rng.standard_normal((4, 5, 6)).astype(np.float32)
    mean, beta = rng.standard_normal(6).astype(np.float32), rng.standard_normal(6).astype(np.float32)
    var, gamma = (0.5 + rng.random(6)).astype(np.float32), (0.5 + rng.random(6)).astype(np.float32)
    want = (x.astype(np.float64) - mean) / np.sqrt(var.astype(np.float64) + 1e-3) * gamma + beta
    assert rel(oracle.batchnorm(x, mean, var, gamma, beta, 1e-3), want) < TOL
    want = (x.astype(np.float64) - mean) / np.sqrt(var.astype(np.float64) + 1e-3)
    assert rel(oracle.batchnorm(x, mean, var, None, None, 1e-3), want) < TOL


def test_relu_family_and_gelu(oracle):
    from scipy.special import erf
    x = np.linspace(-8, 8, 161).astype(np.float32)
    assert np.array_equal(oracle.relu(x), np.maximum(x, 0))
    assert np.array_equal(oracle.relu(x, 6.0, 0.0, 0.0), np.clip(x, 0, 6))
    got = oracle.relu(x, 4.0, 0.1, 1.0)  # x>=4 -> 4; 1<=x<4 -> x; else 0.1*(x-1)
    want = np.where(x >= 4, 4, np.where(x >= 1, x, np.float32(0.1) * (x - 1)))
    assert rel(got, want) < 1e-7
    xd = x.astype(np.float64)
    assert rel(oracle.gelu(x), 0.5 * xd * (1 + erf(xd / math.sqrt(2)))) < TOL


@pytest.mark.parametrize("case", [(8, 8, 2, 2, "valid"), (9, 7, 3, 2, "same"), (9, 7, 3, 2, "valid"),
                                  (5, 5, 2, 1, "same"), (7, 10, 3, 3, "same")])
@pytest.mark.parametrize("mode", ["max", "avg"])
def test_pool2d_vs_torch(oracle, case, mode):
    import torch
    import torch.nn.functional as F
    h, w, k, s, padding = case
    rng = np.random.default_rng(9)
    x = rng.standard_normal((h, w, 3)).astype(np.float32)
    got = oracle.pool2d(x, (k, k), (s, s), padding, mode)
    _, pt, pb = tf_geometry(h, k, s, padding)
    _, pl, pr = tf_geometry(w, k, s, padding)
    xt = torch.from_numpy(x.astype(np.float64)).permute(2, 0, 1)[None]
    if mode == "max":
        want = F.max_pool2d(F.pad(xt, (pl, pr, pt, pb), value=-1e30), k, s)
    else:  # padded taps are excluded from the divisor
        ones = F.pad(torch.ones_like(xt), (pl, pr, pt, pb))
        want = F.avg_pool2d(F.pad(xt, (pl, pr, pt, pb)), k, s) / F.avg_pool2d(ones, k, s)
    want = want[0].permute(1, 2, 0).numpy()
    assert got.shape == want.shape
    assert rel(got, want) < TOL


def test_global_pool_add_embedding_argmax(oracle):
    rng = np.random.default_rng(10)
    x = rng.standard_normal((4, 5, 6)).astype(np.float32)
    assert rel(oracle.global_pool(x, "avg"), x.astype(np.float64).mean((0, 1))) < TOL
    assert np.array_equal(oracle.global_pool(x, "max"), x.max((0, 1)))
    assert oracle.global_pool(x, "avg", keepdims=True).shape == (1, 1, 6)
    y = rng.standard_normal((4, 5, 6)).astype(np.float32)
    assert np.array_equal(oracle.add(x, y), x + y)
    assert np.array_equal(oracle.add(x, y[:1, :, :]), x + y[:1])
    table = rng.standard_normal((11, 3)).astype(np.float32)
    ids = np.array([0, 10, 3.7, 3], np.float32)  # floats are truncated
    assert np.array_equal(oracle.embedding(ids, table.reshape(-1), 11, 3), table[[0, 10, 3, 3]])
    with pytest.raises(RuntimeError):
        oracle.embedding(np.array([11], np.float32), table.reshape(-1), 11, 3)
    assert oracle.argmax(np.array([1, 5, 5, 2], np.float32)) == 1  # first maximum wins
    assert oracle.argmax(np.array([-3, -1, -1], np.float32)) == 1


def numpy_mha(q, v, k, heads, dk, dv, w, use_bias):
    q, v, k = (a.astype(np.float64) for a in (q, v, k))
    if use_bias:
        qw, qb, kw, kb, vw, vb, ow, ob = [a.astype(np.float64) for a in w]
    else:
        qw, kw, vw, ow = [a.astype(np.float64) for a in w]
        qb = kb = vb = ob = 0.0
    d = q.shape[1]
    Q = np.einsum("td,dhk->htk", q, qw.reshape(d, heads, dk)) + (np.reshape(qb, (heads, 1, dk)) if use_bias else 0)
    K = np.einsum("sd,dhk->hsk", k, kw.reshape(d, heads, dk)) + (np.reshape(kb, (heads, 1, dk)) if use_bias else 0)
    V = np.einsum("sd,dhk->hsk", v, vw.reshape(d, heads, dv)) + (np.reshape(vb, (heads, 1, dv)) if use_bias else 0)
    S = np.einsum("htk,hsk->hts", Q, K) / math.sqrt(dk)
    P = np.exp(S - S.max(-1, keepdims=True))
    P /= P.sum(-1, keepdims=True)
    O = np.einsum("hts,hsk->thk", P, V).reshape(q.shape[0], heads * dv)
    return O @ ow.reshape(heads * dv, -1) + ob


@pytest.mark.parametrize("heads,dk,dv,use_bias,sep_key", [(1, 4, 4, True, False), (3, 4, 5, True, True),
                                                          (2, 8, 8, False, False), (2, 3, 6, True, False)])
def test_mha_vs_numpy(oracle, heads, dk, dv, use_bias, sep_key):
    rng = np.random.default_rng(11)
    t, s, d = 5, 7, 6
    q = rng.standard_normal((t, d)).astype(np.float32)
    v = rng.standard_normal((s, d)).astype(np.float32)
    k = rng.standard_normal((s, d)).astype(np.float32) if sep_key else None
    shapes = []
    for dim in (dk, dk, dv):
        shapes.append((d, heads, dim))
        if use_bias:
            shapes.append((heads, dim))
    shapes.append((heads, dv, d))
    if use_bias:
        shapes.append((d,))
    w = [rng.standard_normal(sh).astype(np.float32).reshape(-1) * 0.5 for sh in shapes]
    got = oracle.mha(q, v, k, heads, dk, dv, w, use_bias)
    want = numpy_mha(q, v, v if k is None else k, heads, dk, dv, w, use_bias)
    assert rel(got, want) < TOL
    # permuting key/value rows together leaves the output unchanged (no positional term, no mask)
    perm = rng.permutation(s)
    got2 = oracle.mha(q, v[perm], None if k is None else k[perm], heads, dk, dv, w, use_bias)
    assert rel(got2, got) < TOL


def test_mha_torch_sdpa_crosscheck(oracle):
    import torch
    rng = np.random.default_rng(12)
    t, d = 6, 8
    x = rng.standard_normal((t, d)).astype(np.float32)
    eye = np.eye(d, dtype=np.float32)
    # one head, identity projections: plain softmax(x x^T / sqrt(d)) x
    got = oracle.mha(x, x, None, 1, d, d, [eye.reshape(-1)] * 4, False)
    xt = torch.from_numpy(x.astype(np.float64))[None]
    want = torch.nn.functional.scaled_dot_product_attention(xt, xt, xt)[0].numpy()
    assert rel(got, want) < TOL


@pytest.mark.parametrize("eq,xs,ks,bias_axes", [
    ("abc,cd->abd", (3, 4), (4, 5), "d"), ("abc,cde->abde", (3, 4), (4, 2, 5), "de"),
    ("abc,cde->abde", (3, 4), (4, 2, 5), "ed"), ("abcd,cde->abe", (3, 4, 2), (4, 2, 5), "e"),
    ("abc,cd->abd", (3, 4), (4, 5), None)])
def test_einsum_dense_vs_numpy(oracle, eq, xs, ks, bias_axes):
    rng = np.random.default_rng(13)
    x = rng.standard_normal(xs).astype(np.float32)
    k = rng.standard_normal(ks).astype(np.float32)
    lhs, rest = eq.split(",")
    rk, rhs = rest.split("->")
    sizes = dict(zip(lhs, (1,) + xs))
    sizes.update(zip(rk, ks))
    bias = None
    want = np.einsum(eq, x[None].astype(np.float64), k.astype(np.float64))
    if bias_axes:
        # the stored bias follows the order of the output subscripts, whatever order bias_axes spells
        bchars = [c for c in rhs if c in bias_axes]
        bias = rng.standard_normal([sizes[c] for c in bchars]).astype(np.float32)
        want = want + np.einsum("".join(bchars) + "->" + "".join(c if c in bchars else "" for c in rhs),
                                bias.astype(np.float64)).reshape([sizes[c] if c in bchars else 1 for c in rhs])
    got = oracle.einsum_dense(x, eq, k, list(ks), bias, bias_axes)
    assert got.shape == want.shape[1:]
    assert rel(got, want[0]) < TOL


ACTIVATION_PINS = [
    # name, oracle parameters, independent float64 statement (torch / numpy / scipy, none of them the reference)
    ("tanh", (), lambda x: np.tanh(x)),
    ("sigmoid", (), lambda x: special.expit(x)),
    ("swish", (), lambda x: torch.nn.functional.silu(torch.from_numpy(x)).numpy()),
    ("silu", (), lambda x: x * special.expit(x)),
    ("hard_sigmoid", (), lambda x: torch.nn.functional.hardsigmoid(torch.from_numpy(x)).numpy()),
    ("selu", (), lambda x: torch.nn.functional.selu(torch.from_numpy(x)).numpy()),
    ("elu", (0.7,), lambda x: torch.nn.functional.elu(torch.from_numpy(x), 0.7).numpy()),
    ("celu", (1.0,), lambda x: torch.nn.functional.celu(torch.from_numpy(x), 1.0).numpy()),
    ("exponential", (), lambda x: np.exp(x)),
    ("softsign", (), lambda x: torch.nn.functional.softsign(torch.from_numpy(x)).numpy()),
    ("softplus", (), lambda x: np.logaddexp(0.0, x)),
    ("leaky_relu", (0.2,), lambda x: torch.nn.functional.leaky_relu(torch.from_numpy(x), 0.2).numpy()),
    ("hard_shrink", (0.5,), lambda x: torch.nn.functional.hardshrink(torch.from_numpy(x), 0.5).numpy()),
    ("soft_shrink", (0.5,), lambda x: torch.nn.functional.softshrink(torch.from_numpy(x), 0.5).numpy()),
    ("sparse_plus", (), lambda x: np.where(x <= -1, 0.0, np.where(x < 1, 0.25 * (x + 1) ** 2, x))),
    ("squareplus", (4.0,), lambda x: (x + np.sqrt(x * x + 4.0)) / 2),
    ("tanh_shrink", (), lambda x: torch.nn.functional.tanhshrink(torch.from_numpy(x)).numpy()),
    ("threshold", (0.25, -2.0), lambda x: torch.nn.functional.threshold(torch.from_numpy(x), 0.25, -2.0).numpy()),
    ("log_sigmoid", (), lambda x: torch.nn.functional.logsigmoid(torch.from_numpy(x)).numpy()),
    ("hard_tanh", (), lambda x: torch.nn.functional.hardtanh(torch.from_numpy(x)).numpy()),
]


@pytest.mark.parametrize("name,params,ref", ACTIVATION_PINS, ids=[a[0] for a in ACTIVATION_PINS])
def test_activation_vs_float64(oracle, name, params, ref):
    r = np.random.default_rng(3)
    x = np.concatenate([r.standard_normal(500) * 3, [-20.0, -14.0, -13.5, -3.0, -1.0, -0.5, 0.0, 0.25, 0.5, 1.0, 3.0, 13.5, 14.0, 20.0]])  # thresholds exact in float
    x = x.astype(np.float32)
    want = ref(x.astype(np.float64))
    got = oracle.activation(name, x, *params)
    scale = np.maximum(np.abs(want), 1.0)
    assert (np.abs(got - want) / scale).max() <= 3e-6
    with pytest.raises(RuntimeError, match="unknown activation type"):
        oracle.activation("no_such_activation", x)


def test_log_softmax_prelu_and_merges(oracle):
    r = np.random.default_rng(4)
    x = r.standard_normal((5, 7, 6)).astype(np.float32)
    got = oracle._activation("log_softmax", {}, x)
    assert np.abs(got - special.log_softmax(x.astype(np.float64), axis=-1)).max() <= 2e-6
    y = r.standard_normal((5, 7, 6)).astype(np.float32)
    for op, f in (("mul", np.multiply), ("sub", np.subtract), ("max", np.maximum), ("min", np.minimum)):
        assert np.array_equal(oracle.combine(op, x, y), f(x, y))
    assert np.array_equal(oracle.combine("mul", x, y[:, :1, :]), x * y[:, :1, :])  # size-1 broadcasting
    # PReLU: alpha over the axes that are not shared; torch's prelu covers the channel-only case
    alpha = r.uniform(-1, 1, 6).astype(np.float32)
    want = torch.nn.functional.prelu(torch.from_numpy(x).permute(2, 0, 1)[None], torch.from_numpy(alpha))[0].permute(1, 2, 0).numpy()
    assert np.array_equal(oracle.prelu(x, alpha, [1, 2]), want)
    full = r.uniform(-1, 1, x.size).astype(np.float32)
    assert np.array_equal(oracle.prelu(x, full, []), np.where(x > 0, x, full.reshape(x.shape) * x))
    # a (T, D) sample has no height axis: Keras' shared axis 1 (the sequence) is the reference's width axis
    seq = r.standard_normal((7, 6)).astype(np.float32)
    assert np.array_equal(oracle.prelu(seq, alpha, [1]), np.where(seq > 0, seq, alpha[None, :] * seq))
