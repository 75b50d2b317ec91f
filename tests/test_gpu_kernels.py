"""Parity of every HIP kernel launcher of the C ABI against the CPU oracle on the same seeded
inputs.  Tolerance (floating point, summation order differs): per output tensor
max|gpu - ref| / max|ref| <= 1e-4; integer results (argmax) are exact."""
import zlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-4


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    assert a.shape == b.shape, (a.shape, b.shape)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def rng_for(*key):
    return np.random.default_rng(zlib.crc32(repr(key).encode()))


def say(*a):
    print(*a, flush=True)


CONV_CASES = [
    # n, h, w, cin, cout, kh, kw, strides, dilation, padding
    (2, 8, 9, 3, 5, 3, 3, (1, 1), (1, 1), "same"),       # scalar gather path (cin % 4 != 0)
    (2, 32, 32, 3, 16, 3, 3, (1, 1), (1, 1), "same"),    # small-CNN first layer
    (3, 15, 15, 16, 32, 3, 3, (1, 1), (1, 1), "valid"),  # small-CNN second layer
    (1, 30, 30, 3, 64, 7, 7, (2, 2), (1, 1), "valid"),   # ResNet stem shape, K = 147
    (2, 14, 14, 64, 64, 3, 3, (1, 1), (1, 1), "same"),   # bottleneck 3x3
    (2, 14, 14, 64, 256, 1, 1, (1, 1), (1, 1), "valid"),  # pointwise -> plain GEMM path
    (2, 14, 14, 256, 128, 1, 1, (2, 2), (1, 1), "valid"),  # strided pointwise
    (1, 11, 10, 4, 6, 3, 2, (2, 3), (1, 1), "same"),     # cin = 4 < slab, ragged everything
    (1, 12, 13, 8, 12, 2, 3, (1, 1), (2, 3), "same"),    # dilation
    (1, 9, 9, 20, 40, 5, 5, (1, 1), (1, 1), "same"),     # cin not a multiple of the 16-wide slab
    (4, 7, 7, 512, 160, 1, 1, (1, 1), (1, 1), "valid"),  # M = 196, N not a tile multiple
    (1, 5, 5, 8, 8, 3, 3, (1, 1), (1, 1), "causal"),
]


@pytest.mark.parametrize("tile", [-1, 0, 1, 2, 3, 10, 11, 12, 13, 14, 15, 16, 17, 18])
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_vs_oracle(fdx, oracle, case, tile):
    n, h, w, cin, cout, kh, kw, strides, dilation, padding = case
    say("conv2d", case, "tile", tile)
    r = rng_for("conv", case)
    x = r.standard_normal((n, h, w, cin)).astype(np.float32)
    wj = (r.standard_normal((cout, kh, kw, cin)) / np.sqrt(kh * kw * cin)).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    wo = oracle.conv2d_prepare(wj, cout, kh, kw, cin)
    want = np.stack([oracle.conv2d(x[i], wo, b, cout, kh, kw, strides, dilation, padding) for i in range(n)])
    fdx.lib.fdx_debug_force_tile(tile)
    try:
        got = fdx.conv2d(x, wj, b, strides, dilation, padding)
    finally:
        fdx.lib.fdx_debug_force_tile(-1)
    assert rel(got, want) <= TOL


def test_conv2d_epilogue_residual_relu(fdx, oracle):
    say("conv2d epilogue")
    r = rng_for("conv-epi")
    n, h, w, cin, cout = 2, 10, 10, 32, 48
    x = r.standard_normal((n, h, w, cin)).astype(np.float32)
    wj = (r.standard_normal((cout, 3, 3, cin)) / np.sqrt(9 * cin)).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    res = r.standard_normal((n, h, w, cout)).astype(np.float32)
    wo = oracle.conv2d_prepare(wj, cout, 3, 3, cin)
    conv = np.stack([oracle.conv2d(x[i], wo, b, cout, 3, 3, (1, 1), (1, 1), "same") for i in range(n)])
    for act, f in [(fdx.relu_act(), lambda v: oracle.relu(v)), (fdx.relu_act(6.0), lambda v: oracle.relu(v, 6.0, 0.0, 0.0)),
                   (fdx.relu_act(4.0, 0.1, 1.0), lambda v: oracle.relu(v, 4.0, 0.1, 1.0)), (fdx.gelu_act(), oracle.gelu),
                   (None, lambda v: v)]:
        got = fdx.conv2d(x, wj, b, padding="same", residual=res, act=act)
        assert rel(got, f(oracle.add(res, conv))) <= TOL
    got = fdx.conv2d(x, wj, None, padding="same")
    want = np.stack([oracle.conv2d(x[i], wo, None, cout, 3, 3, (1, 1), (1, 1), "same") for i in range(n)])
    assert rel(got, want) <= TOL


@pytest.mark.parametrize("m,n,k", [(1000, 96, 16), (33, 144, 24), (4096, 192, 32), (257, 960, 96), (64, 4, 8), (31, 33, 128),
                                   (500, 256, 64), (129, 576, 96), (70, 100, 40)])
def test_row_streaming_gemm_short_k(fdx, oracle, m, n, k):
    """The row-streaming kernel for K <= 128 (tile configuration 30), forced: rows and columns that end inside a
    32-wide group, every epilogue operand, k counts that fill the register blocks only partly."""
    say("row-streaming gemm", m, n, k)
    r = rng_for("pws", m, n, k)
    a = r.standard_normal((m, k)).astype(np.float32)
    w = (r.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
    b = r.standard_normal(n).astype(np.float32)
    res = r.standard_normal((m, n)).astype(np.float32)
    ref = a.astype(np.float64) @ w.astype(np.float64).T
    fdx.lib.fdx_debug_force_tile(30)
    try:
        got = fdx.gemm(a, w, None)
        got_full = fdx.gemm(a, w, b, alpha=0.75, residual=res, act=fdx.relu_act(6.0))
        got_gelu = fdx.gemm(a, w, b, act=fdx.gelu_act())
    finally:
        fdx.lib.fdx_debug_force_tile(-1)
    assert rel(got, ref) <= TOL
    assert rel(got_full, np.clip(0.75 * ref + b + res, 0.0, 6.0)) <= TOL
    assert rel(got_gelu, oracle.gelu((ref + b).astype(np.float32))) <= TOL


GEMM_CASES = [(1, 10, 32), (16, 768, 768), (37, 50, 29), (256, 2048, 512), (130, 1000, 2048), (5, 3, 7), (64, 64, 16),
              (300, 96, 100)]


@pytest.mark.parametrize("tile", [-1, 0, 1, 2, 3, 10, 11, 12, 13, 14, 15, 16, 17, 18, 30])
@pytest.mark.parametrize("m,n,k", GEMM_CASES)
def test_gemm_vs_oracle_dense(fdx, oracle, m, n, k, tile):
    say("gemm", m, n, k, "tile", tile)
    r = rng_for("gemm", m, n, k)
    a = r.standard_normal((m, k)).astype(np.float32)
    w = (r.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)  # Dense layout [in][out]
    b = r.standard_normal(n).astype(np.float32)
    want = oracle.dense(a, w.reshape(-1), b, n)
    fdx.lib.fdx_debug_force_tile(tile)
    try:
        got = fdx.gemm(a, w.T, b)
        got_gelu = fdx.gemm(a, w.T, b, act=fdx.gelu_act())
        got_row = fdx.gemm(w.T, a, b, bias_per_row=True, alpha=0.5)  # swapped operands: (a w)^T
    finally:
        fdx.lib.fdx_debug_force_tile(-1)
    assert rel(got, want) <= TOL
    assert rel(got_gelu, oracle.gelu(want)) <= TOL
    want_row = 0.5 * (a.astype(np.float64) @ w.astype(np.float64)).T + b[:, None]
    assert rel(got_row, want_row) <= TOL


@pytest.mark.parametrize("case", [
    (2, 9, 8, 8, 3, 3, (1, 1), (1, 1), "same"), (2, 9, 8, 6, 3, 3, (2, 2), (1, 1), "same"),
    (1, 10, 11, 5, 3, 3, (2, 2), (1, 1), "valid"), (2, 12, 12, 4, 3, 3, (1, 1), (2, 2), "same"),
    (3, 28, 28, 96, 3, 3, (2, 2), (1, 1), "valid"), (2, 14, 14, 144, 3, 3, (1, 1), (1, 1), "same"),
    # the column-tiled 3x3 kernel: widths that are not a multiple of its four-column tile, one-column images, same / valid
    (2, 7, 7, 32, 3, 3, (1, 1), (1, 1), "same"), (1, 5, 1, 8, 3, 3, (1, 1), (1, 1), "same"), (2, 9, 13, 16, 3, 3, (2, 2), (1, 1), "same"),
    (1, 8, 10, 12, 3, 3, (1, 1), (1, 1), "valid"), (1, 3, 3, 4, 3, 3, (2, 2), (1, 1), "valid"), (2, 6, 5, 8, 5, 5, (1, 1), (1, 1), "same"),
    # enough items for the sliding-window 3x3 kernel with row tiles of 4: column tiles of 7 and of 8, extents that end inside a tile
    (16, 14, 14, 256, 3, 3, (1, 1), (1, 1), "same"), (32, 7, 7, 480, 3, 3, (1, 1), (1, 1), "same"), (8, 9, 11, 512, 3, 3, (1, 1), (1, 1), "same"),
    (8, 21, 16, 256, 3, 3, (1, 1), (1, 1), "valid")])
def test_dwconv_vs_oracle(fdx, oracle, case):
    n, h, w, c, kh, kw, strides, dilation, padding = case
    say("dwconv", case)
    r = rng_for("dw", case)
    x = r.standard_normal((n, h, w, c)).astype(np.float32)
    wj = r.standard_normal((c, kh, kw)).astype(np.float32)
    b = r.standard_normal(c).astype(np.float32)
    want = np.stack([oracle.depthwise_conv2d(x[i], wj, b, kh, kw, strides, dilation, padding) for i in range(n)])
    assert rel(fdx.dwconv2d(x, wj, b, strides, dilation, padding), want) <= TOL
    got6 = fdx.dwconv2d(x, wj, None, strides, dilation, padding, act=fdx.relu_act(6.0))
    want6 = np.stack([oracle.relu(oracle.depthwise_conv2d(x[i], wj, None, kh, kw, strides, dilation, padding), 6.0, 0.0, 0.0)
                      for i in range(n)])
    assert rel(got6, want6) <= TOL


@pytest.mark.parametrize("case", [(64, 14, 14, 1024, "same"), (64, 16, 16, 1024, "same"), (64, 16, 14, 1024, "same"), (64, 14, 16, 1024, "same"),
                                  (64, 15, 13, 1024, "same"), (64, 18, 18, 1024, "valid")])
def test_dwconv_sliding_window_tall_tiles(fdx, oracle, case):
    """The sliding-window 3x3 kernel with row tiles of 7 and 8 (taken where they leave at least 65536 items): all four
    (column tile, row tile) forms, extents that end inside a tile, both paddings; every image against the oracle."""
    n, h, w, c, padding = case
    say("dwconv sliding window", case)
    r = rng_for("dwslide", case)
    x = r.standard_normal((n, h, w, c)).astype(np.float32)
    wj = r.standard_normal((c, 3, 3)).astype(np.float32)
    b = r.standard_normal(c).astype(np.float32)
    want = np.stack([oracle.relu(oracle.depthwise_conv2d(x[i], wj, b, 3, 3, (1, 1), (1, 1), padding), 6.0, 0.0, 0.0) for i in range(n)])
    assert rel(fdx.dwconv2d(x, wj, b, (1, 1), (1, 1), padding, act=fdx.relu_act(6.0)), want) <= TOL


@pytest.mark.parametrize("case", [
    # n, h, w, c, n_out, stride, padding: the three tile forms (<= 32, <= 96, more channels), widths that are not a
    # multiple of a run of 8, one-column images, channel counts that end inside a slab, 1..3 column tiles
    (2, 9, 8, 32, 16, 1, "same"), (2, 12, 11, 96, 24, 2, "same"), (1, 14, 14, 144, 24, 1, "same"),
    (2, 7, 7, 192, 32, 1, "same"), (1, 15, 13, 64, 96, 2, "valid"), (1, 5, 1, 8, 4, 1, "same"), (3, 3, 3, 4, 5, 2, "valid"),
    (1, 10, 17, 40, 33, 1, "valid"), (2, 6, 9, 20, 70, 1, "same"), (1, 28, 28, 160, 64, 1, "same"), (2, 17, 16, 36, 96, 2, "same"),
    (4, 56, 56, 144, 32, 2, "same"),
    # filters too large for the LDS: fragments straight from memory
    (1, 15, 13, 384, 96, 2, "valid"), (2, 14, 14, 576, 96, 1, "same"), (1, 28, 28, 192, 64, 2, "same"), (1, 9, 9, 388, 70, 1, "same")])
def test_dwconv_pointwise_vs_oracle(fdx, oracle, case):
    """Depthwise 3x3 + ReLU6 + 1x1 convolution (+ residual) in one launch against the oracle's two layers."""
    n, h, w, c, n_out, stride, padding = case
    say("dwconv_pointwise", case)
    r = rng_for("dwpw", case)
    x = r.standard_normal((n, h, w, c)).astype(np.float32)
    wd = r.standard_normal((c, 3, 3)).astype(np.float32) * 0.5
    bd = r.standard_normal(c).astype(np.float32)
    wp = (r.standard_normal((n_out, c)) / np.sqrt(c)).astype(np.float32)
    bp = r.standard_normal(n_out).astype(np.float32)
    mid = [oracle.relu(oracle.depthwise_conv2d(x[i], wd, bd, 3, 3, (stride, stride), (1, 1), padding), 6.0, 0.0, 0.0) for i in range(n)]
    # 1x1 filter in converted-JSON order [cout][1][1][cin] is the [n_out][c] matrix itself
    want = np.stack([oracle.conv2d(m, oracle.conv2d_prepare(wp.reshape(-1), n_out, 1, 1, c), bp, n_out, 1, 1) for m in mid])
    got = fdx.dwconv_pointwise(x, wd, bd, stride, padding, fdx.relu_act(6.0), wp, bp)
    assert got.shape == want.shape
    assert rel(got, want) <= TOL
    res = r.standard_normal(want.shape).astype(np.float32)
    got_r = fdx.dwconv_pointwise(x, wd, None, stride, padding, None, wp, None, residual=res, act=fdx.relu_act())
    mid0 = [oracle.depthwise_conv2d(x[i], wd, None, 3, 3, (stride, stride), (1, 1), padding) for i in range(n)]
    want_r = np.stack([oracle.relu(oracle.conv2d(m, oracle.conv2d_prepare(wp.reshape(-1), n_out, 1, 1, c), None, n_out, 1, 1) + res[i])
                       for i, m in enumerate(mid0)])
    assert rel(got_r, want_r) <= TOL


@pytest.mark.parametrize("case", [
    # n, h, w, cin, ce, n_out, stride, padding, zero_frame: MobileNetV2's first blocks, odd sizes that leave partial tiles,
    # an expansion that does not fill its last 32-channel slab, two projection tiles
    (2, 16, 16, 16, 96, 24, 2, "valid", (0, 0, 1, 1)), (2, 12, 20, 24, 144, 24, 1, "same", (0, 0, 0, 0)),
    (1, 13, 11, 24, 144, 32, 2, "valid", (0, 0, 1, 1)), (3, 9, 7, 32, 192, 32, 1, "same", (0, 0, 0, 0)),
    (1, 10, 10, 32, 192, 64, 1, "same", (0, 0, 0, 0)), (2, 5, 3, 16, 20, 8, 1, "same", (0, 0, 0, 0)),
    (1, 56, 56, 24, 144, 24, 1, "same", (0, 0, 0, 0)), (1, 33, 47, 16, 96, 40, 2, "same", (0, 0, 0, 0))])
def test_inverted_residual_block_vs_oracle(fdx, oracle, case):
    """1x1 expansion + ReLU6, depthwise 3x3 + ReLU6, 1x1 projection (+ residual) as one launch against the oracle's three
    layers; the depthwise padding pads the expanded tensor with zeros (not with expand(0))."""
    n, h, w, cin, ce, n_out, stride, padding, frame = case
    say("inverted_residual", case)
    r = rng_for("irb", case)
    x = r.standard_normal((n, h, w, cin)).astype(np.float32)
    we = (r.standard_normal((ce, cin)) / np.sqrt(cin)).astype(np.float32)
    be = (r.standard_normal(ce) + 1.0).astype(np.float32)  # a bias that survives ReLU6: padding must still read zero
    wd = r.standard_normal((ce, 3, 3)).astype(np.float32) * 0.5
    bd = r.standard_normal(ce).astype(np.float32)
    wp = (r.standard_normal((n_out, ce)) / np.sqrt(ce)).astype(np.float32)
    bp = r.standard_normal(n_out).astype(np.float32)
    zt, zl, zb, zr = frame

    def reference(i, res, with_bias, final_act):
        e = oracle.conv2d(x[i], oracle.conv2d_prepare(we.reshape(-1), ce, 1, 1, cin), be if with_bias else None, ce, 1, 1)
        e = oracle.relu(e, 6.0, 0.0, 0.0)
        e = np.pad(e, ((zt, zb), (zl, zr), (0, 0)))
        d = oracle.relu(oracle.depthwise_conv2d(e, wd, bd if with_bias else None, 3, 3, (stride, stride), (1, 1), padding), 6.0, 0.0, 0.0)
        o = oracle.conv2d(d, oracle.conv2d_prepare(wp.reshape(-1), n_out, 1, 1, ce), bp if with_bias else None, n_out, 1, 1)
        if res is not None:
            o = o + res[i]
        return oracle.relu(o) if final_act else o

    want = np.stack([reference(i, None, True, False) for i in range(n)])
    got = fdx.inverted_residual(x, we, be, fdx.relu_act(6.0), wd, bd, stride, padding, fdx.relu_act(6.0), wp, bp, zero_frame=frame)
    assert got.shape == want.shape
    assert rel(got, want) <= TOL
    res = r.standard_normal(want.shape).astype(np.float32)
    want_r = np.stack([reference(i, res, False, True) for i in range(n)])
    got_r = fdx.inverted_residual(x, we, None, fdx.relu_act(6.0), wd, None, stride, padding, fdx.relu_act(6.0), wp, None, residual=res,
                                  act=fdx.relu_act(), zero_frame=frame)
    assert rel(got_r, want_r) <= TOL


def test_inverted_residual_rejects_what_it_does_not_cover(fdx):
    assert fdx.lib.fdx_inverted_residual_supported(16, 96, 24, 2) == 1 and fdx.lib.fdx_inverted_residual_supported(24, 144, 32, 1) == 1
    assert fdx.lib.fdx_inverted_residual_supported(20, 96, 24, 1) == 0 and fdx.lib.fdx_inverted_residual_supported(16, 96, 24, 3) == 0
    assert fdx.lib.fdx_inverted_residual_supported(32, 192, 65, 1) == 0 and fdx.lib.fdx_inverted_residual_supported(32, 4000, 32, 1) == 0
    x = np.zeros((1, 4, 4, 20), np.float32)
    with pytest.raises(RuntimeError):
        fdx.inverted_residual(x, np.zeros((8, 20), np.float32), None, None, np.zeros((8, 3, 3), np.float32), None, 1, "same", None,
                              np.zeros((8, 8), np.float32), None)


@pytest.mark.parametrize("case", [
    # n, h, w, cin, cout, padding
    (2, 8, 8, 8, 64, "same"), (1, 7, 7, 16, 64, "same"), (3, 9, 6, 24, 128, "same"), (2, 10, 13, 8, 64, "valid"),
    (1, 14, 14, 64, 128, "same"), (5, 5, 5, 32, 192, "same"), (2, 4, 3, 8, 64, "valid"), (1, 3, 3, 8, 64, "valid"),
    (4, 28, 28, 40, 64, "same"), (8, 14, 14, 72, 128, "same"), (6, 20, 20, 104, 256, "same"),  # units shared by two or three workgroups
])
def test_conv2d_winograd_vs_oracle(fdx, oracle, case):
    """3x3 stride-1 convolution through the F(2x2, 3x3) transforms against the oracle's direct sum: odd extents (tiles
    that hang over the output), both paddings, partial tile blocks, bias, residual and activation; twice in a row, since
    the tickets of shared units must be back at zero after a launch."""
    n, h, w, cin, cout, padding = case
    say("conv2d_winograd", case)
    r = rng_for("wino", case)
    x = r.standard_normal((n, h, w, cin)).astype(np.float32)
    wt = (r.standard_normal((cout, 3, 3, cin)) / np.sqrt(9 * cin)).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    prepared = oracle.conv2d_prepare(wt.reshape(-1), cout, 3, 3, cin)
    want = np.stack([oracle.conv2d(x[i], prepared, b, cout, 3, 3, (1, 1), (1, 1), padding) for i in range(n)])
    got = fdx.conv2d_winograd(x, wt, b, padding)
    assert got.shape == want.shape
    assert rel(got, want) <= TOL
    res = r.standard_normal(want.shape).astype(np.float32)
    want_r = np.stack([oracle.relu(oracle.conv2d(x[i], prepared, None, cout, 3, 3, (1, 1), (1, 1), padding) + res[i]) for i in range(n)])
    got_r = fdx.conv2d_winograd(x, wt, None, padding, residual=res, act=fdx.relu_act())
    assert rel(got_r, want_r) <= TOL
    assert np.array_equal(fdx.conv2d_winograd(x, wt, b, padding), got)  # the same shares, added in the same order


def test_conv2d_winograd_rejects_what_it_does_not_cover(fdx):
    assert fdx.lib.fdx_conv2d_winograd_supported(64, 64) == 1 and fdx.lib.fdx_conv2d_winograd_supported(8, 192) == 1
    assert fdx.lib.fdx_conv2d_winograd_supported(3, 64) == 0 and fdx.lib.fdx_conv2d_winograd_supported(64, 32) == 0
    with pytest.raises(RuntimeError):
        fdx.conv2d_winograd(np.zeros((1, 6, 6, 4), np.float32), np.zeros((64, 3, 3, 4), np.float32), None)


@pytest.mark.parametrize("case", [
    # n, ih, iw, ic, ek, conv stride, conv padding, conv frame, ce, n_out, depthwise stride, depthwise padding, depthwise frame
    (2, 32, 32, 3, 3, 2, "same", (0, 0, 0, 0), 32, 16, 1, "same", (0, 0, 0, 0)),     # MobileNetV2's first block
    (2, 33, 29, 3, 3, 2, "valid", (0, 0, 1, 1), 32, 16, 1, "same", (0, 0, 0, 0)),    # explicit bottom / right padding
    (1, 20, 24, 1, 5, 1, "same", (0, 0, 0, 0), 16, 24, 2, "same", (0, 0, 0, 0)),     # 25 taps on one channel, stride-2 stencil
    (2, 17, 19, 4, 2, 2, "valid", (1, 2, 0, 0), 40, 40, 2, "valid", (0, 0, 1, 1)),   # two slabs, two projection tiles
    (1, 9, 40, 2, 3, 1, "same", (0, 0, 0, 0), 64, 8, 1, "valid", (0, 0, 0, 0)),
    (3, 70, 45, 3, 3, 2, "same", (0, 0, 0, 0), 32, 16, 1, "same", (0, 0, 0, 0)),     # tiles whose windows lie inside the image
])
def test_stem_block_vs_oracle(fdx, oracle, case):
    """Small convolution + ReLU6, depthwise 3x3 + ReLU6, 1x1 projection (+ residual) as one launch against the oracle's
    three layers; both paddings (the convolution's on the image, the stencil's on the convolution's output) read zeros."""
    n, ih, iw, ic, ek, cs, cpad, cframe, ce, n_out, stride, padding, frame = case
    say("stem_block", case)
    r = rng_for("stem", case)
    x = r.standard_normal((n, ih, iw, ic)).astype(np.float32)
    wc = (r.standard_normal((ce, ek, ek, ic)) / np.sqrt(ek * ek * ic)).astype(np.float32)
    bc = (r.standard_normal(ce) + 1.0).astype(np.float32)
    wd = r.standard_normal((ce, 3, 3)).astype(np.float32) * 0.5
    bd = r.standard_normal(ce).astype(np.float32)
    wp = (r.standard_normal((n_out, ce)) / np.sqrt(ce)).astype(np.float32)
    bp = r.standard_normal(n_out).astype(np.float32)
    ct, cl, cb, cr = cframe
    zt, zl, zb, zr = frame

    def reference(i, res, with_bias, final_act):
        img = np.pad(x[i], ((ct, cb), (cl, cr), (0, 0)))
        e = oracle.conv2d(img, oracle.conv2d_prepare(wc.reshape(-1), ce, ek, ek, ic), bc if with_bias else None, ce, ek, ek, (cs, cs),
                          (1, 1), cpad)
        e = oracle.relu(e, 6.0, 0.0, 0.0)
        e = np.pad(e, ((zt, zb), (zl, zr), (0, 0)))
        d = oracle.relu(oracle.depthwise_conv2d(e, wd, bd if with_bias else None, 3, 3, (stride, stride), (1, 1), padding), 6.0, 0.0, 0.0)
        o = oracle.conv2d(d, oracle.conv2d_prepare(wp.reshape(-1), n_out, 1, 1, ce), bp if with_bias else None, n_out, 1, 1)
        if res is not None:
            o = o + res[i]
        return oracle.relu(o) if final_act else o

    want = np.stack([reference(i, None, True, False) for i in range(n)])
    got = fdx.stem_block(x, wc, bc, fdx.relu_act(6.0), cs, cpad, wd, bd, stride, padding, fdx.relu_act(6.0), wp, bp,
                         conv_zero_frame=cframe, zero_frame=frame)
    assert got.shape == want.shape
    assert rel(got, want) <= TOL
    res = r.standard_normal(want.shape).astype(np.float32)
    want_r = np.stack([reference(i, res, False, True) for i in range(n)])
    got_r = fdx.stem_block(x, wc, None, fdx.relu_act(6.0), cs, cpad, wd, None, stride, padding, fdx.relu_act(6.0), wp, None, residual=res,
                           act=fdx.relu_act(), conv_zero_frame=cframe, zero_frame=frame)
    assert rel(got_r, want_r) <= TOL


def test_stem_block_rejects_what_it_does_not_cover(fdx):
    assert fdx.lib.fdx_stem_block_supported(3, 3, 32, 16, 1) == 1 and fdx.lib.fdx_stem_block_supported(1, 5, 16, 24, 2) == 1
    assert fdx.lib.fdx_stem_block_supported(4, 3, 32, 16, 1) == 0  # 36 taps
    assert fdx.lib.fdx_stem_block_supported(3, 3, 30, 16, 1) == 0 and fdx.lib.fdx_stem_block_supported(3, 3, 32, 65, 1) == 0
    assert fdx.lib.fdx_stem_block_supported(3, 3, 32, 16, 3) == 0
    x = np.zeros((1, 8, 8, 4), np.float32)
    with pytest.raises(RuntimeError):
        fdx.stem_block(x, np.zeros((8, 3, 3, 4), np.float32), None, None, 1, "same", np.zeros((8, 3, 3), np.float32), None, 1, "same", None,
                       np.zeros((8, 8), np.float32), None)


def test_dwconv_pointwise_rejects_what_it_does_not_cover(fdx):
    x = np.zeros((1, 4, 4, 6), np.float32)
    with pytest.raises(RuntimeError):
        fdx.dwconv_pointwise(x, np.zeros((6, 3, 3), np.float32), None, 1, "same", None, np.zeros((8, 6), np.float32), None)
    x = np.zeros((1, 4, 4, 8), np.float32)
    with pytest.raises(RuntimeError):
        fdx.dwconv_pointwise(x, np.zeros((8, 3, 3), np.float32), None, 1, "same", None, np.zeros((100, 8), np.float32), None)
    assert fdx.lib.fdx_dwconv_pointwise_supported(32, 16, 1) == 1 and fdx.lib.fdx_dwconv_pointwise_supported(32, 16, 3) == 0
    assert fdx.lib.fdx_dwconv_pointwise_supported(192, 32, 1) == 1 and fdx.lib.fdx_dwconv_pointwise_supported(576, 96, 1) == 1
    assert fdx.lib.fdx_dwconv_pointwise_supported(576, 97, 1) == 0 and fdx.lib.fdx_dwconv_pointwise_supported(6, 8, 1) == 0


@pytest.mark.parametrize("case", [(2, 8, 8, 5, 2, 2, "valid"), (2, 9, 7, 4, 3, 2, "same"), (1, 9, 7, 3, 3, 2, "valid"),
                                  (2, 5, 5, 64, 2, 1, "same"), (1, 7, 10, 6, 3, 3, "same")])
@pytest.mark.parametrize("mode", ["max", "avg"])
def test_pool_vs_oracle(fdx, oracle, case, mode):
    n, h, w, c, k, s, padding = case
    say("pool", case, mode)
    x = rng_for("pool", case).standard_normal((n, h, w, c)).astype(np.float32)
    want = np.stack([oracle.pool2d(x[i], (k, k), (s, s), padding, mode) for i in range(n)])
    got = fdx.pool2d(x, (k, k), (s, s), padding, mode)
    assert rel(got, want) <= 1e-6


def test_pool_with_folded_zero_padding(fdx, oracle):
    say("pool folded zero pad")
    x = rng_for("poolz").standard_normal((2, 10, 10, 8)).astype(np.float32) - 2.0  # mostly negative: zeros must win
    for mode in ("max", "avg"):
        for padding in ("valid", "same"):
            padded = np.pad(x, ((0, 0), (1, 1), (1, 1), (0, 0)))
            want = np.stack([oracle.pool2d(padded[i], (3, 3), (2, 2), padding, mode) for i in range(2)])
            got = fdx.pool2d(x, (3, 3), (2, 2), padding, mode, zero_frame=(1, 1, 1, 1))
            assert rel(got, want) <= 1e-6


def test_global_pool_add_act_affine_pad(fdx, oracle):
    say("glue kernels")
    r = rng_for("glue")
    x = r.standard_normal((3, 7, 7, 100)).astype(np.float32)
    for mode in ("avg", "max"):
        want = np.stack([oracle.global_pool(x[i], mode) for i in range(3)])
        assert rel(fdx.global_pool(x, mode), want) <= 1e-6
    y = r.standard_normal(x.shape).astype(np.float32)
    assert np.array_equal(fdx.add(x, y), x + y)
    assert np.array_equal(fdx.add(x, y, fdx.relu_act()), np.maximum(x + y, 0))
    assert np.array_equal(fdx.add(x, y[0]), x + y[0])  # broadcast over the batch
    odd = r.standard_normal(1001).astype(np.float32)
    assert np.array_equal(fdx.add(odd, odd), odd + odd)
    assert rel(fdx.activation(x, fdx.gelu_act()), oracle.gelu(x)) <= 1e-6
    assert np.array_equal(fdx.activation(x, fdx.relu_act(6.0)), oracle.relu(x, 6.0, 0.0, 0.0))
    assert rel(fdx.activation(x, fdx.relu_act(4.0, 0.1, 1.0)), oracle.relu(x, 4.0, 0.1, 1.0)) <= 1e-6
    mean, beta = r.standard_normal(100).astype(np.float32), r.standard_normal(100).astype(np.float32)
    var, gamma = (0.5 + r.random(100)).astype(np.float32), (0.5 + r.random(100)).astype(np.float32)
    inv = (gamma / np.sqrt(var + np.float32(1e-3))).astype(np.float32)
    got = fdx.channel_affine(x, inv, (beta - mean * inv).astype(np.float32))
    assert rel(got, oracle.batchnorm(x, mean, var, gamma, beta, 1e-3)) <= 1e-5
    got = fdx.zero_pad2d(x, 1, 2, 3, 0)
    assert np.array_equal(got, np.pad(x, ((0, 0), (1, 2), (3, 0), (0, 0))))


@pytest.mark.parametrize("rows,depth", [(5, 33), (256, 512), (16, 768), (7, 1000), (3, 4097)])
def test_layernorm_vs_oracle(fdx, oracle, rows, depth):
    say("layernorm", rows, depth)
    r = rng_for("ln", rows, depth)
    x = (r.standard_normal((rows, depth)) * 3 + 1).astype(np.float32)
    g, b = r.standard_normal(depth).astype(np.float32), r.standard_normal(depth).astype(np.float32)
    assert rel(fdx.layernorm(x, g, b, 1e-3), oracle.layernorm(x, g, b, 1e-3)) <= TOL
    assert rel(fdx.layernorm(x, None, None, 1e-5), oracle.layernorm(x, None, None, 1e-5)) <= TOL


@pytest.mark.parametrize("rows,depth", [(4, 10), (64, 256), (5, 1000), (3, 50257), (9, 1)])
def test_softmax_vs_oracle(fdx, oracle, rows, depth):
    say("softmax", rows, depth)
    x = (rng_for("sm", rows, depth).standard_normal((rows, depth)) * 6).astype(np.float32)
    assert rel(fdx.softmax(x), oracle.softmax(x)) <= TOL
    big = x * 100  # saturating inputs keep finite outputs that sum to one
    got = fdx.softmax(big)
    assert np.isfinite(got).all() and np.abs(got.sum(-1) - 1).max() < 1e-4


def test_softmax_causal_prefix(fdx, oracle):
    say("softmax causal")
    t, s = 5, 8
    x = rng_for("smc").standard_normal((3 * t, s)).astype(np.float32)
    got = fdx.softmax(x, causal_period=t, causal_offset=s - t)
    for row in range(3 * t):
        vis = row % t + 1 + (s - t)
        assert rel(got[row, :vis], oracle.softmax(x[row, :vis])) <= TOL
        assert (got[row, vis:] == 0).all()


def test_embedding_and_argmax(fdx, oracle):
    say("embedding argmax")
    r = rng_for("emb")
    table = r.standard_normal((50, 24)).astype(np.float32)
    ids = np.array([0, 49, 3.7, 3, 17], np.float32)
    assert np.array_equal(fdx.embedding(ids, table), oracle.embedding(ids, table.reshape(-1), 50, 24))
    with pytest.raises(fdx.FdxError):
        fdx.embedding(np.array([50], np.float32), table)
    x = r.standard_normal((6, 50257)).astype(np.float32)
    x[0, 100] = x[0, 40000] = 50.0  # tie: the first maximum wins
    x[1, :] = -1.0
    idx, val = fdx.argmax(x)
    want = [oracle.argmax(x[i]) for i in range(6)]
    assert idx.tolist() == want and idx[0] == 100 and idx[1] == 0
    assert np.array_equal(val, x[np.arange(6), idx])


def numpy_attention(q, k, v, heads, dk, dv, causal):
    b, t, _ = q.shape
    s = k.shape[1]
    out = np.zeros((b, t, heads * dv))
    for bi in range(b):
        for h in range(heads):
            Q, K, V = q[bi, :, h * dk:(h + 1) * dk], k[bi, :, h * dk:(h + 1) * dk], v[bi, :, h * dv:(h + 1) * dv]
            S = Q.astype(np.float64) @ K.astype(np.float64).T / np.sqrt(dk)
            if causal:
                S = np.where(np.arange(s)[None, :] <= np.arange(t)[:, None] + (s - t), S, -np.inf)
            P = np.exp(S - S.max(-1, keepdims=True))
            P /= P.sum(-1, keepdims=True)
            out[bi, :, h * dv:(h + 1) * dv] = P @ V
    return out


@pytest.mark.parametrize("b,t,s,heads,dk,dv,causal", [(2, 5, 7, 3, 4, 5, False), (2, 16, 16, 2, 64, 64, True),
                                                      (1, 33, 33, 4, 16, 16, True), (2, 64, 64, 8, 64, 64, False),
                                                      (1, 3, 9, 2, 8, 8, True),
                                                      # depths the fused (flash-style) kernel takes: ragged tiles, key
                                                      # prefix longer than the queries, several query tiles, one query
                                                      (2, 256, 256, 4, 64, 64, False), (2, 130, 200, 3, 64, 64, True),
                                                      (1, 300, 300, 2, 64, 64, True), (2, 100, 300, 3, 32, 32, False),
                                                      (1, 129, 129, 2, 128, 128, True), (3, 1, 70, 2, 64, 64, False),
                                                      (2, 64, 65, 2, 32, 32, True)])
def test_mha_prefill(fdx, oracle, b, t, s, heads, dk, dv, causal):
    say("mha prefill", b, t, s, heads, dk, dv, causal)
    r = rng_for("mha", b, t, s, heads, dk, dv, causal)
    q = r.standard_normal((b, t, heads * dk)).astype(np.float32)
    k = r.standard_normal((b, s, heads * dk)).astype(np.float32)
    v = r.standard_normal((b, s, heads * dv)).astype(np.float32)
    got = fdx.mha_prefill(q, k, v, heads, dk, dv, causal)
    assert rel(got, numpy_attention(q, k, v, heads, dk, dv, causal)) <= TOL
    if not causal:  # the oracle's MultiHeadAttention with identity projections is this core
        eye_k = np.zeros((heads * dk, heads, dk), np.float32)
        eye_v = np.zeros((heads * dv, heads, dv), np.float32)
        for h in range(heads):
            eye_k[h * dk:(h + 1) * dk, h] = np.eye(dk)
            eye_v[h * dv:(h + 1) * dv, h] = np.eye(dv)
        if dk == dv:
            w = [eye_k.reshape(-1), eye_k.reshape(-1), eye_v.reshape(-1), np.eye(heads * dv, dtype=np.float32).reshape(-1)]
            want = oracle.mha(q[0], v[0], k[0], heads, dk, dv, w, False)
            assert rel(got[0], want) <= TOL


@pytest.mark.parametrize("b,heads,dk,dv,length,max_len", [(2, 3, 8, 8, 5, 9), (16, 12, 64, 64, 129, 256),
                                                          (3, 2, 64, 32, 256, 256), (1, 1, 6, 10, 1, 4)])
def test_mha_decode(fdx, b, heads, dk, dv, length, max_len):
    say("mha decode", b, heads, dk, dv, length, max_len)
    r = rng_for("dec", b, heads, dk, dv, length)
    q = r.standard_normal((b, heads * dk)).astype(np.float32)
    kc = r.standard_normal((b, max_len, heads * dk)).astype(np.float32)
    vc = r.standard_normal((b, max_len, heads * dv)).astype(np.float32)
    got = fdx.mha_decode(q, kc, vc, heads, dk, dv, length)
    want = numpy_attention(q[:, None], kc[:, :length], vc[:, :length], heads, dk, dv, False)[:, 0]
    assert rel(got, want) <= TOL


def test_launcher_argument_errors(fdx):
    say("argument errors")
    a = fdx.DevBuf(64)
    with pytest.raises(fdx.FdxError):
        fdx.check(fdx.lib.fdx_gemm_bias_act_f32(None, 4, None, 4, 1, 1, 4, fdx.ctypes.c_float(1), None, 0, None, None, None, 1, None))
    with pytest.raises(fdx.FdxError):
        fdx.check(fdx.lib.fdx_pool2d_nhwc_f32(fdx._dp(a), 1, 2, 2, 1, 2, 2, 1, 1, 0, 0, 0, 0, 0, 0, 1, 1, 7, fdx._dp(a)))
    with pytest.raises(fdx.FdxError):
        fdx.window_geometry(0, 4, 3, 3, 1, 1, "same")


def test_shader_clock_probe(fdx):
    """The measurement aid bench.py uses: a sampler on its own stream, bounded, one at a time."""
    say("clock probe")
    c = fdx.ctypes
    mean, lo, hi = c.c_double(), c.c_double(), c.c_double()
    with pytest.raises(fdx.FdxError):  # nothing started
        fdx.check(fdx.lib.fdx_clock_probe_stop(c.c_double(1.0), c.byref(mean), c.byref(lo), c.byref(hi)))
    with pytest.raises(fdx.FdxError):
        fdx.check(fdx.lib.fdx_clock_probe_start(1, 100))
    fdx.check(fdx.lib.fdx_clock_probe_start(40, 100))
    with pytest.raises(fdx.FdxError):  # one at a time
        fdx.check(fdx.lib.fdx_clock_probe_start(40, 100))
    x = fdx.DevBuf.from_host(np.ones((1 << 20,), np.float32))
    y = fdx.DevBuf(4 << 20)
    act = fdx.relu_act()
    for _ in range(20):  # some work beside it on the library stream
        fdx.check(fdx.lib.fdx_activation_f32(fdx._dp(x), c.c_size_t(1 << 20), c.byref(act), fdx._dp(y)))
    fdx.sync()
    fdx.check(fdx.lib.fdx_clock_probe_stop(c.c_double(3.5), c.byref(mean), c.byref(lo), c.byref(hi)))
    assert 0.3 < lo.value <= mean.value <= hi.value < 4.0, (lo.value, mean.value, hi.value)
    assert y.to_host((1 << 20,))[123] == 1.0


# (16, 3072, 768), (16, 4096, 1024), (9, 8192, 128): column groups in a multiple of 8, so the K ranges of a group (4, 4 and 8
# of them) meet inside their XCD's L2; (1, 2048, 48): three column groups, the K ranges meet through memory
DENSE_ROWS = [(16, 768, 2304), (16, 768, 768), (16, 3072, 768), (3, 64, 100), (16, 768, 50257), (5, 20, 33), (7, 1024, 40),
              (16, 100, 64), (1, 2048, 48), (16, 4096, 1024), (9, 8192, 128)]


@pytest.mark.parametrize("m,k,n", DENSE_ROWS)
def test_dense_rows_decode_shape(fdx, oracle, m, k, n):
    """The weight-streaming Dense for <= 16 rows (split along K for long K) against the oracle's Dense."""
    say("dense_rows", m, k, n)
    r = rng_for("dense_rows", m, k, n)
    x = r.standard_normal((m, k)).astype(np.float32)
    w = (r.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
    b = r.standard_normal(n).astype(np.float32)
    res = r.standard_normal((m, n)).astype(np.float32)
    want = oracle.gelu(oracle.dense(x, np.ascontiguousarray(w.T).reshape(-1), b, n) + res)
    dx, dw, db, dr = (fdx.DevBuf.from_host(a) for a in (x, w, b, res))
    out = fdx.DevBuf(4 * m * n)
    act = fdx.gelu_act()
    got = []
    for _ in range(3):  # repeated: the split-K tickets and flags must be back at zero after a launch
        fdx.check(fdx.lib.fdx_dense_rows_f32(fdx._dp(dx), m, k, fdx._dp(dw), fdx._dp(db), n, fdx._dp(dr), fdx.ctypes.byref(act),
                                             fdx._dp(out)))
        got.append(out.to_host((m, n)))
        assert rel(got[-1], want) <= TOL
    assert np.array_equal(got[0], got[1]) and np.array_equal(got[0], got[2])  # partial tiles are added in a fixed order


@pytest.mark.parametrize("m,k,n", [(16, 768, 2304), (3, 64, 100), (16, 768, 50257), (7, 1024, 40), (16, 100, 64)])
def test_layernorm_dense_rows_folded(fdx, oracle, m, k, n):
    """LayerNormalization + Dense in one launch through folded weights against oracle LN followed by oracle Dense,
    on rows with a mean far from zero (the folded form subtracts mean * rowsum after the product)."""
    say("layernorm_dense_rows", m, k, n)
    r = rng_for("ln_dense_rows", m, k, n)
    x = (r.standard_normal((m, k)) * 2 + 3.0).astype(np.float32)
    w = (r.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
    b = r.standard_normal(n).astype(np.float32)
    g, be = r.standard_normal(k).astype(np.float32), r.standard_normal(k).astype(np.float32)
    want = oracle.dense(oracle.layernorm(x, g, be, 1e-5), np.ascontiguousarray(w.T).reshape(-1), b, n)
    dx, dw, db, dg, dbe = (fdx.DevBuf.from_host(a) for a in (x, w, b, g, be))
    wf, ws, bf, out = fdx.DevBuf(4 * n * k), fdx.DevBuf(4 * n), fdx.DevBuf(4 * n), fdx.DevBuf(4 * m * n)
    fdx.check(fdx.lib.fdx_fold_layernorm_f32(fdx._dp(dg), fdx._dp(dbe), fdx._dp(dw), fdx._dp(db), n, k, fdx._dp(wf), fdx._dp(ws),
                                             fdx._dp(bf)))
    fdx.check(fdx.lib.fdx_layernorm_dense_rows_f32(fdx._dp(dx), m, k, fdx.ctypes.c_float(1e-5), fdx._dp(wf), fdx._dp(ws),
                                                   fdx._dp(bf), n, None, None, fdx._dp(out)))
    assert rel(out.to_host((m, n)), want) <= TOL
    # no gamma / beta / bias
    fdx.check(fdx.lib.fdx_fold_layernorm_f32(None, None, fdx._dp(dw), None, n, k, fdx._dp(wf), fdx._dp(ws), fdx._dp(bf)))
    fdx.check(fdx.lib.fdx_layernorm_dense_rows_f32(fdx._dp(dx), m, k, fdx.ctypes.c_float(1e-3), fdx._dp(wf), fdx._dp(ws),
                                                   fdx._dp(bf), n, None, None, fdx._dp(out)))
    want = oracle.dense(oracle.layernorm(x, None, None, 1e-3), np.ascontiguousarray(w.T).reshape(-1), None, n)
    assert rel(out.to_host((m, n)), want) <= TOL


SPLIT_CASES = [
    # n, h, w, cin, cout, kh, kw, strides, padding
    (2, 7, 7, 64, 64, 3, 3, (1, 1), "same"),     # K = 576: 3x3 taps cut inside a tap's channels
    (3, 14, 14, 48, 96, 3, 3, (1, 1), "same"),   # cin a multiple of 16 only: BK 16 configurations
    (2, 7, 7, 512, 128, 1, 1, (1, 1), "valid"),  # pointwise: plain GEMM path, K = 512
    (1, 9, 9, 32, 40, 5, 5, (2, 2), "same"),     # strided, ragged M and N
]


@pytest.mark.parametrize("tile", [210, 310, 211, 412, 213, 314, 215, 415])
@pytest.mark.parametrize("case", SPLIT_CASES)
def test_conv2d_split_k(fdx, oracle, case, tile):
    """The K range of every output tile cut into 2..4 units whose partial tiles the last arriving workgroup adds
    (forced: configuration + 100 * splits); twice in a row, so the tickets must have been reset; with a residual and
    ReLU in the epilogue, which only the adding workgroup may apply."""
    n, h, w, cin, cout, kh, kw, strides, padding = case
    say("conv2d split-K", case, "tile", tile)
    r = rng_for("conv-split", case)
    x = r.standard_normal((n, h, w, cin)).astype(np.float32)
    wj = (r.standard_normal((cout, kh, kw, cin)) / np.sqrt(kh * kw * cin)).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    wo = oracle.conv2d_prepare(wj, cout, kh, kw, cin)
    conv = np.stack([oracle.conv2d(x[i], wo, b, cout, kh, kw, strides, (1, 1), padding) for i in range(n)])
    res = r.standard_normal(conv.shape).astype(np.float32)
    want = oracle.relu(oracle.add(res, conv))
    fdx.lib.fdx_debug_force_tile(tile)
    try:
        first = fdx.conv2d(x, wj, b, strides, (1, 1), padding, residual=res, act=fdx.relu_act())
        second = fdx.conv2d(x, wj, b, strides, (1, 1), padding, residual=res, act=fdx.relu_act())
    finally:
        fdx.lib.fdx_debug_force_tile(-1)
    assert rel(first, want) <= TOL
    assert np.array_equal(first, second)  # partials are added in split order: the result does not depend on arrival order


@pytest.mark.parametrize("tile", [213, 415])
def test_gemm_split_k_many_tiles(fdx, oracle, tile):
    say("gemm split-K", tile)
    r = rng_for("gemm-split", tile)
    m, n, k = 1000, 384, 2048
    a = r.standard_normal((m, k)).astype(np.float32)
    w = (r.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)
    b = r.standard_normal(n).astype(np.float32)
    want = oracle.gelu(oracle.dense(a, w.reshape(-1), b, n))
    fdx.lib.fdx_debug_force_tile(tile)
    try:
        got = fdx.gemm(a, w.T, b, act=fdx.gelu_act())
    finally:
        fdx.lib.fdx_debug_force_tile(-1)
    assert rel(got, want) <= TOL


@pytest.mark.parametrize("strips", [2, 3, 5, 8])
@pytest.mark.parametrize("tile,cap", [(15, 0), (12, 24), (14, 10), (13, 0), (16, 0), (18, 0)])
def test_gemm_and_conv_tiles_numbered_in_column_strips(fdx, oracle, strips, tile, cap):
    """Whole-tile launches may number their output tiles strip by strip (so that an XCD's contiguous tile range needs
    only its strip's columns of the weights); the order must not change a single value.  Column-tile counts that the
    strip count does not divide, row counts that are no multiple of the tile, and a capped persistent grid (several
    tiles per workgroup) are covered; the unstriped run is the reference."""
    say("column strips", strips, "tile", tile, "cap", cap)
    r = rng_for("strips", strips, tile)
    m, n, k = 1000, 704, 256  # 11 column tiles of 64, 6 (5.5) of 128
    a = r.standard_normal((m, k)).astype(np.float32)
    w = (r.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
    b = r.standard_normal(n).astype(np.float32)
    res = r.standard_normal((m, n)).astype(np.float32)
    x = r.standard_normal((2, 18, 17, 64)).astype(np.float32)
    wj = (r.standard_normal((320, 3, 3, 64)) / 24.0).astype(np.float32)
    bj = r.standard_normal(320).astype(np.float32)
    fdx.lib.fdx_debug_force_tile(tile)
    fdx.lib.fdx_debug_persist_cap(cap)
    try:
        plain = fdx.gemm(a, w, b, residual=res, act=fdx.relu_act())
        plain_c = fdx.conv2d(x, wj, bj, (1, 1), (1, 1), "same", act=fdx.relu_act())
        fdx.check(fdx.lib.fdx_debug_force_strips(strips))
        got = fdx.gemm(a, w, b, residual=res, act=fdx.relu_act())
        got_c = fdx.conv2d(x, wj, bj, (1, 1), (1, 1), "same", act=fdx.relu_act())
    finally:
        fdx.lib.fdx_debug_force_strips(0)
        fdx.lib.fdx_debug_persist_cap(0)
        fdx.lib.fdx_debug_force_tile(-1)
    want = np.maximum(a.astype(np.float64) @ w.astype(np.float64).T + b + res, 0)
    assert rel(plain, want) <= TOL
    assert np.array_equal(got, plain)
    assert np.array_equal(got_c, plain_c)


@pytest.mark.parametrize("tile,cap", [(10215, 24), (10315, 24), (10413, 8), (10214, 16), (10612, 40), (10815, 9)])
def test_conv2d_hybrid_whole_tiles_plus_split_remainder(fdx, oracle, tile, cap):
    """Persistent grid capped to `cap` workgroups: the tiles that fill whole rounds run as whole tiles, the last partial
    round is cut into K ranges (configuration + 100 * splits + 10000); result equals the oracle and repeats bit for bit."""
    say("conv2d hybrid", tile, cap)
    n, h, w, cin, cout = 3, 20, 19, 64, 96
    r = rng_for("conv-hybrid", tile)
    x = r.standard_normal((n, h, w, cin)).astype(np.float32)
    wj = (r.standard_normal((cout, 3, 3, cin)) / np.sqrt(9 * cin)).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    wo = oracle.conv2d_prepare(wj, cout, 3, 3, cin)
    conv = np.stack([oracle.conv2d(x[i], wo, b, cout, 3, 3, (1, 1), (1, 1), "same") for i in range(n)])
    res = r.standard_normal(conv.shape).astype(np.float32)
    want = oracle.relu(oracle.add(res, conv))
    fdx.lib.fdx_debug_force_tile(tile)
    fdx.lib.fdx_debug_persist_cap(cap)
    try:
        first = fdx.conv2d(x, wj, b, (1, 1), (1, 1), "same", residual=res, act=fdx.relu_act())
        second = fdx.conv2d(x, wj, b, (1, 1), (1, 1), "same", residual=res, act=fdx.relu_act())
    finally:
        fdx.lib.fdx_debug_force_tile(-1)
        fdx.lib.fdx_debug_persist_cap(0)
    assert rel(first, want) <= TOL
    assert np.array_equal(first, second)


@pytest.mark.parametrize("tile,cap", [(20010, 0), (20011, 0), (20012, 0), (20013, 0), (20014, 0), (20015, 0),
                                      (20015, 9), (20012, 40), (20010, 8), (20011, 24), (20014, 133)])
def test_conv2d_stream_k(fdx, oracle, tile, cap):
    """Stream-K scheduling (20000 + configuration): the slabs of all tiles are dealt out in equal stretches, one per
    workgroup, so tiles are shared by two or more workgroups at arbitrary cut points; grid sizes from 8 workgroups (a
    stretch spans several tiles) to the resident count (several workgroups per tile). Result equals the oracle and
    repeats bit for bit."""
    say("conv2d stream-K", tile, cap)
    n, h, w, cin, cout = 3, 20, 19, 64, 96
    r = rng_for("conv-streamk", tile, cap)
    x = r.standard_normal((n, h, w, cin)).astype(np.float32)
    wj = (r.standard_normal((cout, 3, 3, cin)) / np.sqrt(9 * cin)).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    wo = oracle.conv2d_prepare(wj, cout, 3, 3, cin)
    conv = np.stack([oracle.conv2d(x[i], wo, b, cout, 3, 3, (1, 1), (1, 1), "same") for i in range(n)])
    res = r.standard_normal(conv.shape).astype(np.float32)
    want = oracle.relu(oracle.add(res, conv))
    fdx.lib.fdx_debug_force_tile(tile)
    fdx.lib.fdx_debug_persist_cap(cap)
    try:
        first = fdx.conv2d(x, wj, b, (1, 1), (1, 1), "same", residual=res, act=fdx.relu_act())
        second = fdx.conv2d(x, wj, b, (1, 1), (1, 1), "same", residual=res, act=fdx.relu_act())
    finally:
        fdx.lib.fdx_debug_force_tile(-1)
        fdx.lib.fdx_debug_persist_cap(0)
    assert rel(first, want) <= TOL
    assert np.array_equal(first, second)


@pytest.mark.parametrize("m,n,k,tile", [(1000, 256, 512, 20010), (4096, 128, 1024, 20011), (300, 64, 2048, 20015),
                                        (129, 132, 64, 20012)])
def test_gemm_stream_k(fdx, m, n, k, tile):
    say("gemm stream-K", m, n, k, tile)
    r = rng_for("gemm-streamk", m, n, k)
    a = r.standard_normal((m, k)).astype(np.float32)
    w = (r.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
    bias = r.standard_normal(n).astype(np.float32)
    want = a.astype(np.float64) @ w.astype(np.float64).T + bias
    fdx.lib.fdx_debug_force_tile(tile)
    try:
        got = fdx.gemm(a, w, bias)
        again = fdx.gemm(a, w, bias)
    finally:
        fdx.lib.fdx_debug_force_tile(-1)
    assert rel(got, want) <= TOL
    assert np.array_equal(got, again)


@pytest.mark.parametrize("case", [
    # n, h, w, cin, cout, k, padding, explicit zero frame (top/left = bottom/right)
    (2, 30, 30, 3, 64, 7, "valid", 3),   # ResNet stem: ZeroPadding2D(3) then 7x7 / 2 valid
    (2, 33, 29, 3, 64, 7, "same", 0),    # odd extents, TF same padding
    (3, 17, 18, 4, 64, 3, "same", 0),    # four channels, 3x3 / 2
    (1, 20, 20, 4, 128, 5, "valid", 1),
    (2, 16, 16, 3, 96, 8, "valid", 0),   # even kernel
])
def test_conv2d_space_to_depth_stem(fdx, oracle, case):
    """Stride-2 convolutions over 3 or 4 channels through the space-to-depth view against the oracle's Conv2D."""
    n, h, w, cin, cout, k, padding, frame = case
    say("conv2d s2d", case)
    r = rng_for("conv-s2d", case)
    x = r.standard_normal((n, h, w, cin)).astype(np.float32)
    wj = (r.standard_normal((cout, k, k, cin)) / np.sqrt(k * k * cin)).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    wo = oracle.conv2d_prepare(wj, cout, k, k, cin)
    xp = np.pad(x, ((0, 0), (frame, frame), (frame, frame), (0, 0)))
    want = oracle.relu(np.stack([oracle.conv2d(xp[i], wo, b, cout, k, k, (2, 2), (1, 1), padding) for i in range(n)]))
    got = fdx.conv2d_s2d(x, wj, b, padding, act=fdx.relu_act(), extra_pad=(frame, frame))
    assert rel(got, want) <= TOL
    # and the general path on the same operands agrees
    plain = fdx.conv2d(xp, wj, b, (2, 2), (1, 1), padding, act=fdx.relu_act())
    assert rel(got, plain) <= TOL
