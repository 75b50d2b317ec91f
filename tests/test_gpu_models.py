"""Whole-model parity: converted-JSON files written by the package's model writers, loaded through
fdx_model_create and run batched on the GPU, against the CPU oracle walking the same file sample by sample.
Tolerance: per output tensor max|gpu - ref| / max|ref| <= 1e-4 (fp32, summation order differs)."""
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


def with_taps(spec, names):
    """Adds intermediate layers as extra model outputs so that parity is checked before a saturating softmax."""
    cfg = spec["architecture"]["config"]
    cfg["output_layers"] = cfg["output_layers"] + [[n, 0, 0] for n in names]
    spec["output_shapes"] = spec["output_shapes"] + [None] * len(names)  # placeholders, fixed below
    return spec


def run_both(fdx, oracle, modelgen, spec, inputs, tol=TOL):
    js = modelgen.dumps(spec)
    ref = oracle.OracleModel(js)
    n = inputs[0].shape[0]
    want = [ref.predict([x[i] for x in inputs]) for i in range(n)]
    want = [np.stack([w[k] for w in want]) for k in range(len(want[0]))]
    model = fdx.Model(js)
    got = model.predict(inputs)
    errs = [rel(g, w) for g, w in zip(got, want)]
    say("  rel errors:", ["%.2e" % e for e in errs])
    assert max(errs) <= tol
    return got, want, model


def fix_tap_shapes(spec, oracle, modelgen, sample_inputs):
    tmp = dict(spec)
    tmp["output_shapes"] = [[1]] * len(spec["output_shapes"])
    ref = oracle.OracleModel(modelgen.dumps(tmp))
    outs = ref.predict(sample_inputs)
    spec["output_shapes"] = [list(o.shape) for o in outs]
    return spec


def test_small_cnn_256_samples(fdx, oracle, modelgen):
    say("small_cnn")
    spec = modelgen.small_cnn()
    x = np.random.default_rng(11).uniform(-1, 1, (256, 32, 32, 3)).astype(np.float32)
    got, want, model = run_both(fdx, oracle, modelgen, spec, [x])
    assert np.abs(got[0].sum(-1) - 1).max() < 1e-5
    # predict_class semantics: argmax with first-max-wins equals the oracle's
    assert [int(np.argmax(g)) for g in got[0]] == [oracle.argmax(w) for w in want[0]]
    # batch 1 equals row 0 of the batched run (samples are independent)
    one = model.predict([x[:1]])
    assert rel(one[0], got[0][:1]) <= 1e-6


def test_embedded_self_test_and_failure(fdx, oracle, modelgen):
    say("embedded tests")
    spec = modelgen.small_cnn()
    x = np.random.default_rng(12).uniform(-1, 1, (32, 32, 3)).astype(np.float32)
    ref = oracle.OracleModel(modelgen.dumps(spec))
    y = ref.predict([x])[0]
    spec["tests"] = [{"inputs": [x], "outputs": [y]}]
    fdx.Model(modelgen.dumps(spec), verify=True, verify_epsilon=1e-5)  # passes
    spec["tests"] = [{"inputs": [x], "outputs": [y + 0.01]}]
    with pytest.raises(fdx.FdxError, match="test failed"):
        fdx.Model(modelgen.dumps(spec), verify=True)
    fdx.Model(modelgen.dumps(spec), verify=False)  # verification is optional


def test_resnet_scaled_down(fdx, oracle, modelgen):
    say("resnet scaled")
    spec = modelgen.resnet50(seed=21, input_size=64, width=16, blocks=(2, 2, 2, 2), classes=20, random_bn=True)
    spec = with_taps(spec, ["avg_pool", "conv2_block1_out", "pool1_pool"])
    x = np.random.default_rng(13).uniform(0, 1, (3, 64, 64, 3)).astype(np.float32)
    spec = fix_tap_shapes(spec, oracle, modelgen, [x[0]])
    run_both(fdx, oracle, modelgen, spec, [x])


def test_resnet50_full_width_two_images(fdx, oracle, modelgen):
    say("resnet50 full")
    spec = modelgen.resnet50()
    spec = with_taps(spec, ["avg_pool"])
    x = np.random.default_rng(14).uniform(0, 1, (2, 224, 224, 3)).astype(np.float32)
    spec = fix_tap_shapes(spec, oracle, modelgen, [x[0]])
    got, want, model = run_both(fdx, oracle, modelgen, spec, [x])
    assert abs(model.last_flops() - 2 * modelgen.model_flops(spec)) / (2 * modelgen.model_flops(spec)) < 1e-9


def test_mobilenet_v2_truncated(fdx, oracle, modelgen):
    say("mobilenet")
    spec = modelgen.mobilenet_v2(seed=22, input_size=96, classes=30, random_bn=True, truncate=8)
    spec = with_taps(spec, ["global_average_pooling2d", "block_3_depthwise_relu"])
    x = np.random.default_rng(15).uniform(0, 1, (3, 96, 96, 3)).astype(np.float32)
    spec = fix_tap_shapes(spec, oracle, modelgen, [x[0]])
    run_both(fdx, oracle, modelgen, spec, [x])


@pytest.mark.parametrize("mode", [2, 1, 0])
def test_depthwise_pointwise_pairs_forced_either_way(fdx, oracle, modelgen, mode):
    """The depthwise 3x3 + 1x1 pairs of inverted-residual blocks (stride 1 and 2 with the folded ZeroPadding2D, folded
    BatchNormalization, ReLU6 in between, residual Add behind) and of SeparableConv2D, forced to run as one launch each
    (mode 1), as two (mode 0), and with the 1x1 expansion in front taken into the same launch where the block has one
    (mode 2): all must match the oracle.  (Left to itself a plan times the forms and keeps the fastest.)"""
    say("depthwise + pointwise pairs, forced fusion mode", mode)
    spec = modelgen.mobilenet_v2(seed=25, input_size=64, classes=20, random_bn=True, truncate=11)
    x = np.random.default_rng(18).uniform(0, 1, (5, 64, 64, 3)).astype(np.float32)
    b = modelgen.Builder("sep", 26)
    img = b.input((13, 11, 8), "img")
    s1 = b.separable_conv2d(img, 24, 3, "sep1", padding="same", activation="relu")
    s2 = b.separable_conv2d(s1, 10, 3, "sep2", strides=2, padding="valid", use_bias=False)
    sep = b.finish([s2])
    xs = np.random.default_rng(19).standard_normal((3, 13, 11, 8)).astype(np.float32)
    fdx.check(fdx.lib.fdx_debug_force_dw_fusion(mode))
    try:
        run_both(fdx, oracle, modelgen, spec, [x])
        run_both(fdx, oracle, modelgen, sep, [xs])
    finally:
        fdx.check(fdx.lib.fdx_debug_force_dw_fusion(-1))


def test_mobilenet_v2_full_size_fusion_invariance(fdx, oracle, modelgen):
    """At the real layer shapes (224x224, all 17 blocks, batch 8): one launch per depthwise + 1x1 pair, two launches per
    pair and the timed choice give the same features, and one image agrees with the oracle."""
    say("mobilenet_v2 full size, fused vs two launches")
    spec = modelgen.mobilenet_v2(seed=27, random_bn=True)
    spec = with_taps(spec, ["global_average_pooling2d"])
    x = np.random.default_rng(20).uniform(0, 1, (8, 224, 224, 3)).astype(np.float32)
    spec = fix_tap_shapes(spec, oracle, modelgen, [x[0]])
    js = modelgen.dumps(spec)
    outs = []
    try:
        for mode in (2, 1, 0, -1):
            fdx.check(fdx.lib.fdx_debug_force_dw_fusion(mode))
            outs.append(fdx.Model(js, verify=False).predict([x]))
    finally:
        fdx.check(fdx.lib.fdx_debug_force_dw_fusion(-1))
    # the forms add the same products in different orders (one launch keeps a block's sums in registers, separate 1x1
    # launches cut a long K into ranges on the small maps): a fifth of the bar against the oracle
    for other in outs[1:]:
        for a, b in zip(outs[0], other):
            assert rel(a, b) <= TOL / 5
    want = oracle.OracleModel(js).predict([x[0]])
    for g, w in zip(outs[0], want):
        assert rel(g[0], w) <= TOL


def test_encoder_small(fdx, oracle, modelgen):
    say("encoder")
    spec = modelgen.encoder(seed=23, layers=2, seq=24, d_model=64, heads=4, ffn=128, bias_std=0.1, random_affine=True)
    x = np.random.default_rng(16).standard_normal((3, 24, 64)).astype(np.float32)
    run_both(fdx, oracle, modelgen, spec, [x])


def test_gpt2_tiny_predict_is_unmasked(fdx, oracle, modelgen):
    say("gpt2 tiny predict")
    spec = modelgen.gpt2(seed=24, layers=2, d_model=32, heads=4, vocab=97, max_pos=32, bias_std=0.1, random_affine=True,
                         std=0.2)
    r = np.random.default_rng(17)
    ids = r.integers(0, 97, (2, 9)).astype(np.float32)
    pos = np.tile(np.arange(9, dtype=np.float32), (2, 1))
    run_both(fdx, oracle, modelgen, spec, [ids, pos])


@pytest.mark.parametrize("mode", [1, 0, -1])
def test_resnet_with_either_3x3_kernel(fdx, oracle, modelgen, mode):
    """The 3x3 stride-1 convolutions of a (narrow) ResNet50 through the Winograd kernel, through the direct kernel, and
    with the plan timing both: every form meets the oracle."""
    say("resnet 3x3 kernels, mode", mode)
    js = modelgen.dumps(modelgen.resnet50(seed=61, input_size=64, width=64, blocks=(2, 2, 1, 1), classes=10, random_bn=True))
    x = np.random.default_rng(62).uniform(0, 1, (3, 64, 64, 3)).astype(np.float32)
    want = [oracle.OracleModel(js).predict([x[i]])[0] for i in range(3)]
    try:
        fdx.check(fdx.lib.fdx_debug_force_winograd(mode))
        got = fdx.Model(js, verify=False).predict([x])[0]
    finally:
        fdx.check(fdx.lib.fdx_debug_force_winograd(-1))
    for i in range(3):
        assert rel(got[i], want[i]) <= TOL


def test_predict_from_device_pointers(fdx, modelgen):
    """fdx_model_predict_dev reads 16-byte aligned device inputs where they lie and copies misaligned ones first; both
    return what the host-pointer call returns, also when the same plan is used with another buffer afterwards, with the
    first buffer overwritten in between, and with host inputs again."""
    import ctypes
    say("predict_dev aligned / misaligned inputs")
    model = fdx.Model(modelgen.dumps(modelgen.small_cnn()))
    r = np.random.default_rng(77)
    xs = [r.uniform(-1, 1, (9, 32, 32, 3)).astype(np.float32) for _ in range(3)]
    want = [model.predict([x])[0] for x in xs]
    out = fdx.DevBuf(want[0].nbytes)
    fp = ctypes.POINTER(ctypes.c_float)

    def run(ptr_value):
        ip = (fp * 1)(ctypes.cast(ctypes.c_void_p(ptr_value), fp))
        op = (fp * 1)(fdx._dp(out))
        dims, ranks = model._dims([(32, 32, 3)])
        fdx.check(fdx.lib.fdx_model_predict_dev(model._h, 9, ip, dims, ranks, op, None, None))
        fdx.sync()
        return out.to_host(want[0].shape)

    a = fdx.DevBuf.from_host(xs[0])
    assert np.array_equal(run(a.ptr.value), want[0])
    b = fdx.DevBuf(xs[1].nbytes + 16)  # the same data four bytes off a 16-byte boundary
    fdx.check(fdx.lib.fdx_h2d(ctypes.c_void_p(b.ptr.value + 4), xs[1].ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(xs[1].nbytes)))
    assert np.array_equal(run(b.ptr.value + 4), want[1])
    fdx.check(fdx.lib.fdx_h2d(a.ptr, xs[2].ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(xs[2].nbytes)))
    assert np.array_equal(run(a.ptr.value), want[2])
    assert np.array_equal(model.predict([xs[0]])[0], want[0])
    assert np.array_equal(run(b.ptr.value + 4), want[1])


@pytest.mark.parametrize("batch", [16, 13, 8])
def test_large_host_inputs_are_staged_in_pieces(fdx, modelgen, batch):
    """Host inputs of several MB travel through the library's pinned buffers in pieces of whole samples, and a network
    that starts with a convolution runs it piece by piece behind the copy (include/fdeep/model.hpp:28-42: samples are
    independent).  The result must be what the device-pointer call returns on the same data, for one contiguous block,
    for one pointer per sample, for a batch that does not divide into equal pieces, and on a second call."""
    say("staged host inputs, batch", batch)
    spec = modelgen.resnet50(input_size=160, width=16, blocks=(1, 1, 1, 1), classes=10, random_bn=True)
    model = fdx.Model(modelgen.dumps(spec))
    r = np.random.default_rng(90 + batch)
    x = r.uniform(0, 1, (batch, 160, 160, 3)).astype(np.float32)  # 4.9 MB at batch 16, 2.4 MB at batch 8 (the plain copy)
    d_x = fdx.DevBuf.from_host(x)
    d_out = fdx.DevBuf(4 * batch * 10)
    model.predict_dev(batch, [d_x], [(160, 160, 3)], [d_out])
    fdx.sync()
    want = d_out.to_host((batch, 10))
    for _ in range(2):
        got = model.predict([x])[0]
        assert rel(got, want) <= 3e-6, np.abs(got - want).max()
    scattered = [[np.array(x[b])] for b in range(batch)]  # one allocation per sample
    got = model.predict_samples(scattered)[0]
    assert rel(got, want) <= 3e-6
    # a network whose first layer is not a convolution of its own launch: pieces are copied, nothing runs behind them
    b2 = modelgen.Builder("two_in", 5)
    u = b2.input((256, 256, 4), "u")
    v = b2.input((256, 256, 4), "v")
    y = b2.add([u, v], "sum")
    y = b2.conv2d(y, 8, 3, "c", padding="same", activation="relu")
    m2 = fdx.Model(modelgen.dumps(b2.finish([b2.gap(y, "gap")])))
    a, c = (r.standard_normal((batch, 256, 256, 4)).astype(np.float32) for _ in range(2))
    d_a, d_c, d_o = fdx.DevBuf.from_host(a), fdx.DevBuf.from_host(c), fdx.DevBuf(4 * batch * 8)
    m2.predict_dev(batch, [d_a, d_c], [(256, 256, 4)] * 2, [d_o])
    fdx.sync()
    assert rel(m2.predict([a, c])[0], d_o.to_host((batch, 8))) <= 3e-6
    assert rel(m2.predict_samples([[a[b], c[b]] for b in range(batch)])[0], d_o.to_host((batch, 8))) <= 3e-6


def test_large_host_inputs_from_several_threads(fdx, modelgen):
    """predict is callable from many host threads (FAQ.md:103-114); with inputs large enough for the pinned pieces the
    threads take turns at the library's staging buffers.  Three threads, two models, three calls each: every result
    equals the serial one."""
    import threading
    say("staged host inputs from three threads")
    spec = modelgen.resnet50(input_size=160, width=16, blocks=(1, 1, 1, 1), classes=10, random_bn=True)
    models = [fdx.Model(modelgen.dumps(spec)), fdx.Model(modelgen.dumps(spec))]
    r = np.random.default_rng(95)
    xs = [r.uniform(0, 1, (16 + 4 * i, 160, 160, 3)).astype(np.float32) for i in range(3)]
    want = [models[i % 2].predict([xs[i]])[0] for i in range(3)]
    got = [[None] * 3 for _ in range(3)]
    errors = []

    def work(i):
        try:
            for k in range(3):
                got[i][k] = models[i % 2].predict([xs[i]])[0]
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(3)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(3):
        for k in range(3):
            assert np.array_equal(got[i][k], want[i]), (i, k)


def test_input_shape_errors(fdx, modelgen):
    say("shape errors")
    model = fdx.Model(modelgen.dumps(modelgen.small_cnn()))
    with pytest.raises(fdx.FdxError, match="Invalid inputs shape"):
        model.predict([np.zeros((1, 32, 32, 4), np.float32)])
    with pytest.raises(fdx.FdxError, match="Invalid inputs shape"):
        model.predict([np.zeros((1, 32 * 32 * 3), np.float32)])  # same volume, wrong rank
    with pytest.raises(fdx.FdxError):
        fdx.Model(b'{"image_data_format": "channels_first"}')
    bad = modelgen.small_cnn()
    bad["architecture"]["config"]["layers"][1]["class_name"] = "Conv9D"
    with pytest.raises(fdx.FdxError, match="unknown layer type: Conv9D"):
        fdx.Model(modelgen.dumps(bad))


def test_variable_input_size_cycles_through_more_shapes_than_cached_plans(fdx, oracle, modelgen):
    """A fully convolutional model with variable height and width (input_shapes [null, null, 3]): every (batch, shape)
    pair gets its own launch plan; a few recent ones are kept, so going round more shapes than that re-plans, and
    coming back to a kept one reuses its buffers. Every call is checked against the oracle."""
    say("variable-size fully convolutional model")
    b = modelgen.Builder("fcn", 33)
    x = b.input((16, 16, 3), "img")
    y = b.conv2d(x, 8, 3, "c1", padding="same", activation="relu", bias_std=0.1)
    y = b.pool(y, "p1", 2, 2)
    y = b.conv2d(y, 16, 3, "c2", strides=2, padding="same", activation="relu", bias_std=0.1)
    y = b.conv2d_transpose(y, 8, 3, "up", strides=2, padding="same", activation="relu")
    y = b.conv2d(y, 4, 1, "head", bias_std=0.1)
    spec = b.finish([y])
    spec["input_shapes"] = [[None, None, 3]]
    spec["output_shapes"] = [[None, None, 4]]
    for layer in spec["architecture"]["config"]["layers"]:
        if layer["class_name"] == "InputLayer":
            layer["config"]["batch_shape"] = [None, None, None, 3]
    js = modelgen.dumps(spec)
    ref = oracle.OracleModel(js)
    model = fdx.Model(js)
    r = np.random.default_rng(34)
    sizes = [(16, 16), (12, 20), (9, 7), (24, 8), (31, 5), (10, 10)]
    inputs = {s: r.standard_normal((2 + i % 2,) + s + (3,)).astype(np.float32) for i, s in enumerate(sizes)}
    for s in sizes + sizes[::-1] + [sizes[0], sizes[0]]:
        xi = inputs[s]
        want = np.stack([ref.predict([xi[i]])[0] for i in range(xi.shape[0])])
        got = model.predict([xi])[0]
        assert rel(got, want) <= TOL, s
    with pytest.raises(fdx.FdxError, match="Invalid inputs shape"):
        model.predict([np.zeros((1, 8, 8, 4), np.float32)])


@pytest.mark.parametrize("cin,cout", [(24, 144), (40, 96), (72, 64), (8, 64)])
def test_pointwise_convolution_on_channel_counts_between_slabs(fdx, oracle, modelgen, cin, cout):
    """1x1 convolutions whose channel count is a multiple of 4 but not of 16 read each pixel as a 16-float-aligned row
    that laps into the next pixel, against filter rows padded with zero taps; the last pixel of the last image has
    nothing behind it. With BatchNormalization folded in, ReLU6 and a residual Add behind the convolution."""
    say("pointwise conv", cin, cout)
    b = modelgen.Builder("pw_%d_%d" % (cin, cout), 50 + cin)
    x = b.input((9, 7, cin), "img")
    skip = b.conv2d(x, cout, 3, "skip", padding="same", bias_std=0.1)
    y = b.conv2d(x, cout, 1, "pw", use_bias=False)
    y = b.batchnorm(y, "pw_bn", random_stats=True)
    y = b.relu(y, "pw_relu", max_value=6.0)
    z = b.conv2d(y, cout, 1, "pw2", bias_std=0.2) if cout % 16 else b.conv2d(x, cout, 1, "pw2", bias_std=0.2)
    out = b.add([z, skip], "sum")
    spec = b.finish([out, y])
    xs = np.random.default_rng(51).standard_normal((5, 9, 7, cin)).astype(np.float32)
    run_both(fdx, oracle, modelgen, spec, [xs])


@pytest.mark.parametrize("stride,size,c_in,c_mid,c_out", [(1, (9, 7), 64, 32, 128), (2, (15, 13), 64, 48, 256), (2, (8, 8), 128, 64, 64),
                                                           ((2, 1), (11, 6), 32, 16, 96)])
@pytest.mark.parametrize("one_launch", [1, 0])
def test_block_with_a_convolution_on_its_shortcut(fdx, oracle, modelgen, stride, size, c_in, c_mid, c_out, one_launch):
    """Add(BatchNormalization(Conv2D 1x1(a)), BatchNormalization(Conv2D 1x1 / stride(b))) + ReLU: the two convolutions run
    as one GEMM over the channels of both inputs (the strided one reads every stride-th pixel of its map), or one after
    the other on the joint filter when the one-launch kernel is switched off.  Odd map sizes, a non-square stride, and a
    second block behind the first so that the sum is read again."""
    say("shortcut convolution", stride, size, c_in, c_mid, c_out, "one launch" if one_launch else "two launches")
    b = modelgen.Builder("sc_%s_%d_%d" % (str(stride).replace(" ", ""), c_in, c_out), 61 + c_in + c_out)
    x = b.input(size + (c_in,), "img")
    y = b.conv2d(x, c_mid, 1, "c1", strides=stride, use_bias=False)
    y = b.batchnorm(y, "c1_bn", random_stats=True)
    y = b.relu(y, "c1_relu")
    z = b.conv2d(y, c_out, 1, "c3", bias_std=0.2)
    z = b.batchnorm(z, "c3_bn", random_stats=True)
    sc = b.conv2d(x, c_out, 1, "sc", strides=stride, bias_std=0.1)
    sc = b.batchnorm(sc, "sc_bn", random_stats=True)
    out = b.add([sc, z], "sum")
    out = b.relu(out, "sum_relu")
    y2 = b.conv2d(out, c_mid, 1, "d1", activation="relu", bias_std=0.1)
    z2 = b.conv2d(y2, c_out, 1, "d3", bias_std=0.1)
    out2 = b.add([out, z2], "sum2")
    spec = b.finish([out2, out])
    xs = np.random.default_rng(62).standard_normal((5,) + size + (c_in,)).astype(np.float32)
    fdx.check(fdx.lib.fdx_debug_dual_conv(one_launch))
    try:
        run_both(fdx, oracle, modelgen, spec, [xs])
    finally:
        fdx.check(fdx.lib.fdx_debug_dual_conv(1))


@pytest.mark.parametrize("c_in,c_mid,c_out,stride", [(64, 64, 256, 1), (64, 64, 128, 2), (32, 128, 256, 1), (128, 128, 512, 2)])
@pytest.mark.parametrize("mode", [1, 0])
def test_block_tail_and_next_block_head_as_one_launch(fdx, oracle, modelgen, c_in, c_mid, c_out, stride, mode):
    """Three bottleneck blocks of 1x1 convolutions: the last convolution of a block (with its shortcut convolution, or its
    Add, and the ReLU in the epilogue) and the first convolution of the next block run as one launch, the second taking the
    first's result from LDS -- forced on (at sizes the library's rule would leave alone) and off; every block's sum is a
    model output, so both results of each launch are compared.  Pixel counts that are no multiple of the 64-row block."""
    say("chained 1x1 convolutions", c_in, c_mid, c_out, stride, "one launch" if mode else "two launches")
    b = modelgen.Builder("chain_%d_%d_%d_%d" % (c_in, c_mid, c_out, stride), 71 + c_in + c_out)
    x = b.input((11, 9, c_in), "img")
    sums = []
    for blk in range(3):
        first = blk == 0
        y = b.conv2d(x, c_mid, 1, "b%d_c1" % blk, strides=stride if first else 1, use_bias=False)
        y = b.batchnorm(y, "b%d_c1_bn" % blk, random_stats=True)
        y = b.relu(y, "b%d_c1_relu" % blk)
        z = b.conv2d(y, c_out, 1, "b%d_c3" % blk, bias_std=0.2)
        z = b.batchnorm(z, "b%d_c3_bn" % blk, random_stats=True)
        if first:
            sc = b.conv2d(x, c_out, 1, "b0_sc", strides=stride, bias_std=0.1)
            sc = b.batchnorm(sc, "b0_sc_bn", random_stats=True)
        else:
            sc = x
        x = b.add([sc, z], "b%d_sum" % blk)
        x = b.relu(x, "b%d_out" % blk)
        sums.append(x)
    tail = b.conv2d(x, 64, 1, "tail", activation="relu", bias_std=0.1)
    spec = b.finish([tail] + sums)
    xs = np.random.default_rng(72).standard_normal((5, 11, 9, c_in)).astype(np.float32)
    fdx.check(fdx.lib.fdx_debug_force_chain(mode))
    try:
        run_both(fdx, oracle, modelgen, spec, [xs])
    finally:
        fdx.check(fdx.lib.fdx_debug_force_chain(-1))


@pytest.mark.parametrize("center,scale,offset", [(True, True, 0.0), (False, True, 0.0), (True, False, 3.0), (True, True, 40.0)])
def test_layernorm_inside_the_readers_gemms(fdx, oracle, modelgen, center, scale, offset):
    """A LayerNormalization over the last axis whose readers are Dense layers and a self-attention layer is computed inside
    those layers' GEMMs (row statistics gathered in the K loop, gamma / beta folded into the filters): against the oracle,
    and against the same model with the LayerNormalization as a launch of its own.  With and without gamma / beta, with
    rows whose mean is far from zero (40 standard deviations: the sums behind the statistics are taken relative to a
    value of the row), two Dense readers of one LayerNormalization, a residual Add in the reader's epilogue, and a
    LayerNormalization that also feeds a plain Add (not folded)."""
    say("layernorm inside the gemm", center, scale, offset)
    b = modelgen.Builder("lnf_%d%d_%d" % (center, scale, int(offset)), 81 + int(offset))
    x = b.input((24, 64), "tokens")
    n1 = b.layernorm_axes(x, "ln1", [-1], eps=1e-5, center=center, scale=scale)
    att = b.mha(n1, n1, "att", heads=4, key_dim=16, bias_std=0.1)
    x1 = b.add([x, att], "res1")
    n2 = b.layernorm_axes(x1, "ln2", [-1], eps=1e-3, center=center, scale=scale)
    f1 = b.dense(n2, 128, "fc1", activation="gelu", bias_std=0.1)
    g1 = b.dense(n2, 64, "gate", bias_std=0.1)          # a second reader of ln2
    f2 = b.dense(f1, 64, "fc2", bias_std=0.1)
    x2 = b.add([x1, f2], "res2")
    x3 = b.add([x2, g1], "res3")
    n3 = b.layernorm_axes(x3, "ln3", [-1], eps=1e-5, center=center, scale=scale)
    f3 = b.dense(n3, 96, "head", bias_std=0.1)
    mixed = b.add([n3, x3], "not_folded")                # ln3 has a reader that is no GEMM: it keeps its own launch
    spec = b.finish([f3, x3, mixed])
    xs = (np.random.default_rng(82).standard_normal((5, 24, 64)) + offset).astype(np.float32)
    fdx.check(fdx.lib.fdx_debug_force_ln_fold(1))
    try:
        got, want, model = run_both(fdx, oracle, modelgen, spec, [xs])
        fdx.check(fdx.lib.fdx_profile_enable(1))
        fdx.check(fdx.lib.fdx_profile_reset())
        model.predict([xs])
        fdx.sync()
        families, i = set(), 0
        while True:
            name = fdx.ctypes.create_string_buffer(128)
            n, ms, fl, by = fdx.ctypes.c_uint64(), fdx.ctypes.c_double(), fdx.ctypes.c_double(), fdx.ctypes.c_double()
            if fdx.lib.fdx_profile_get(i, name, 128, fdx.ctypes.byref(n), fdx.ctypes.byref(ms), fdx.ctypes.byref(fl), fdx.ctypes.byref(by)) != 0:
                break
            families.add(name.value.decode())
            i += 1
        fdx.check(fdx.lib.fdx_profile_enable(0))
        fdx.check(fdx.lib.fdx_debug_force_ln_fold(0))
        plain = fdx.Model(modelgen.dumps(spec), verify=False).predict([xs])
    finally:
        fdx.check(fdx.lib.fdx_profile_enable(0))
        fdx.check(fdx.lib.fdx_debug_force_ln_fold(-1))
    assert "gemm_ln_f32" in families, families  # the folded form really ran
    for a, c in zip(got, plain):
        assert rel(a, c) <= TOL / 5


def test_shortcut_convolution_on_variable_input_sizes(fdx, oracle, modelgen):
    """The joined shortcut convolution (stride 2) under variable height and width: odd and even sizes, each with a plan of
    its own; the strided rows of the second input follow the size of the call."""
    say("shortcut convolution, variable sizes")
    b = modelgen.Builder("sc_var", 91)
    x = b.input((12, 12, 32), "img")
    y = b.conv2d(x, 32, 1, "c1", strides=2, activation="relu", bias_std=0.1)
    z = b.conv2d(y, 64, 1, "c3", bias_std=0.1)
    sc = b.conv2d(x, 64, 1, "sc", strides=2, bias_std=0.1)
    out = b.relu(b.add([sc, z], "sum"), "out")
    spec = b.finish([out])
    spec["input_shapes"] = [[None, None, 32]]
    spec["output_shapes"] = [[None, None, 64]]
    for layer in spec["architecture"]["config"]["layers"]:
        if layer["class_name"] == "InputLayer":
            layer["config"]["batch_shape"] = [None, None, None, 32]
    js = modelgen.dumps(spec)
    ref = oracle.OracleModel(js)
    model = fdx.Model(js)
    r = np.random.default_rng(92)
    for i, size in enumerate([(12, 12), (7, 9), (15, 4), (1, 1), (8, 13)]):
        xi = r.standard_normal((2 + i % 3,) + size + (32,)).astype(np.float32)
        want = np.stack([ref.predict([xi[k]])[0] for k in range(xi.shape[0])])
        got = model.predict([xi])[0]
        assert got.shape == want.shape and rel(got, want) <= TOL, size
