"""Parity at the shapes the benchmark runs, where the kernels taken differ from the small-model tests: the
GPT-2-small-shaped decode session (d 768, 12 heads x 64, FFN 3072, vocabulary 50257, batch 16, prompt 128), the
transformer encoder at 6 x (d 512, 8 heads, FFN 2048), sequence 256, batch 32, and ResNet50 / MobileNetV2 at batch
64 / 128 with the per-shape tuner live and with its table exported, imported and frozen.

Tolerance: per output tensor max|gpu - ref| / max|ref| <= 1e-4 against the oracle; greedy ids identical wherever the
oracle's top-2 logit margin exceeds 1e-3; GPU-against-GPU comparisons of independently batched samples <= 3e-5."""
import threading

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


def margin(row):
    top = np.sort(row)[-2:]
    return top[1] - top[0]


@pytest.fixture(scope="module")
def gpt2_small_two_blocks(fdx, modelgen):
    """GPT-2-small layer shapes with two blocks (the twelve blocks repeat the same launches; two keep the oracle, which
    recomputes every prefix, at seconds per sequence)."""
    js = modelgen.dumps(modelgen.gpt2(seed=41, layers=2, max_pos=256, bias_std=0.1, random_affine=True))
    return js, fdx.Model(js, verify=False)


def test_gpt2_small_shape_session_against_oracle(fdx, oracle, gpt2_small_two_blocks):
    """Batch 16, prompt 128: prefill logits and 8 decode steps on forced continuation tokens for two of the sequences
    against the oracle's causal prediction of the whole 136-token sequence (row t of that prediction is what the
    session must return after t + 1 tokens)."""
    say("GPT-2-small-shape session vs oracle")
    js, model = gpt2_small_two_blocks
    ref = oracle.OracleModel(js)
    B, P, N, V = 16, 128, 8, 50257
    r = np.random.default_rng(42)
    prompts = r.integers(0, V, (B, P))
    forced = r.integers(0, V, (N, B))
    checked = (0, 11)
    want = {}
    for b in checked:
        ids = np.concatenate([prompts[b], forced[:, b]]).astype(np.float32)
        want[b] = ref.predict([ids, np.arange(P + N, dtype=np.float32)], causal=True)[0]
    sess = fdx.Session(model, B, 256)
    logits, nxt = sess.prefill(prompts)
    worst = 0.0
    for b in checked:
        worst = max(worst, rel(logits[b], want[b][P - 1]))
        if margin(want[b][P - 1]) > 1e-3:
            assert nxt[b] == oracle.argmax(want[b][P - 1])
    for i in range(N):
        logits, nxt = sess.decode_step(forced[i])
        for b in checked:
            row = want[b][P + i]
            worst = max(worst, rel(logits[b], row))
            assert rel(logits[b], row) <= TOL, (i, b)
            if margin(row) > 1e-3:
                assert nxt[b] == oracle.argmax(row), (i, b)
    say("  worst relative error over prefill + %d steps: %.2e" % (N, worst))
    assert worst <= TOL
    assert sess.length() == P + N


def test_gpt2_small_shape_greedy_loop_equals_single_steps(fdx, gpt2_small_two_blocks):
    """128 greedy tokens after a 128-token prompt at batch 16 (the benchmark's session): the captured-step loop
    returns the tokens and last logits of 128 single steps."""
    say("GPT-2-small-shape greedy loop vs single steps")
    js, model = gpt2_small_two_blocks
    B, P, N, V = 16, 128, 128, 50257
    prompts = np.random.default_rng(43).integers(0, V, (B, P))
    sess = fdx.Session(model, B, 256)
    _, first = sess.prefill(prompts)
    tokens, last_logits = sess.decode_greedy(first, N)
    assert sess.length() == P + N
    sess2 = fdx.Session(model, B, 256)
    _, cur = sess2.prefill(prompts)
    assert np.array_equal(cur, first)
    for i in range(N):
        logits, nxt = sess2.decode_step(cur)
        assert np.array_equal(nxt, tokens[i]), i
        cur = nxt
    assert rel(logits, last_logits) <= 1e-6
    # a second loop on a reset session repeats the first bit for bit
    sess.reset()
    _, first_b = sess.prefill(prompts)
    tokens_b, logits_b = sess.decode_greedy(first_b, N)
    assert np.array_equal(tokens_b, tokens) and np.array_equal(logits_b, last_logits)


@pytest.fixture(scope="module")
def gpt2_small_full(fdx, modelgen):
    """The decoder as benchmarked: twelve blocks, vocabulary 50257, 1024 positions; biases and LayerNorm affines drawn at
    random so that a dropped bias or affine shows."""
    js = modelgen.dumps(modelgen.gpt2(seed=47, bias_std=0.1, random_affine=True))
    return js, fdx.Model(js, verify=False)


def test_gpt2_small_full_depth_session_against_cached_oracle(fdx, oracle, gpt2_small_full):
    """Twelve blocks, batch 16, prompt 128: the prefill logits and 8 decode steps on forced continuation tokens for two
    of the sequences against the oracle's KV-cached decoder fed the same 136 tokens one by one (its row t is what the
    session must return after t + 1 tokens; multi_head_attention_layer.hpp:74-110 on query = last row, value = prefix).
    Ids are compared wherever the oracle's top-2 margin exceeds 1e-3 (tensor.hpp:281-302: first maximum wins)."""
    say("GPT-2-small, 12 blocks, session vs the oracle's cached decoder")
    js, model = gpt2_small_full
    ref = oracle.OracleModel(js)
    B, P, N, V = 16, 128, 8, 50257
    r = np.random.default_rng(48)
    prompts = r.integers(0, V, (B, P))
    forced = r.integers(0, V, (N, B))
    checked = (3, 14)
    want = {}

    def run_oracle(b):
        dec = oracle.CachedDecoder(ref)
        rows = {}
        for t, tok in enumerate(np.concatenate([prompts[b], forced[:, b]])):
            row = dec.step(int(tok))
            if t >= P - 1:
                rows[t] = row.copy()
        want[b] = rows

    threads = [threading.Thread(target=run_oracle, args=(b,)) for b in checked]
    for t in threads:
        t.start()
    sess = fdx.Session(model, B, 256)
    logits, nxt = sess.prefill(prompts)
    got = [(logits.copy(), nxt.copy())]
    for i in range(N):
        logits, nxt = sess.decode_step(forced[i])
        got.append((logits.copy(), nxt.copy()))
    assert sess.length() == P + N
    for t in threads:
        t.join()
    worst, fired, skipped = 0.0, 0, 0
    for i, (logits, nxt) in enumerate(got):
        for b in checked:
            row = want[b][P - 1 + i]
            e = rel(logits[b], row)
            worst = max(worst, e)
            assert e <= TOL, (i, b, e)
            if margin(row) > 1e-3:
                fired += 1
                assert nxt[b] == oracle.argmax(row), (i, b)
            else:
                skipped += 1
    say("  worst relative error over prefill + %d steps: %.2e; id comparisons fired %d, skipped for margin %d"
        % (N, worst, fired, skipped))
    assert fired >= len(got)


def test_gpt2_small_full_depth_greedy_loop_equals_single_steps(fdx, gpt2_small_full):
    """Twelve blocks: 128 greedy tokens after a 128-token prompt at batch 16 through the step loop equal 128 single
    steps, and a second loop on the reset session repeats the first bit for bit."""
    say("GPT-2-small, 12 blocks, greedy loop vs single steps")
    js, model = gpt2_small_full
    B, P, N, V = 16, 128, 128, 50257
    prompts = np.random.default_rng(49).integers(0, V, (B, P))
    sess = fdx.Session(model, B, 256)
    _, first = sess.prefill(prompts)
    tokens, last_logits = sess.decode_greedy(first, N)
    assert sess.length() == P + N
    sess2 = fdx.Session(model, B, 256)
    _, cur = sess2.prefill(prompts)
    assert np.array_equal(cur, first)
    for i in range(N):
        logits, nxt = sess2.decode_step(cur)
        assert np.array_equal(nxt, tokens[i]), i
        cur = nxt
    assert rel(logits, last_logits) <= 1e-6
    sess.reset()
    _, first_b = sess.prefill(prompts)
    tokens_b, logits_b = sess.decode_greedy(first_b, N)
    assert np.array_equal(tokens_b, tokens) and np.array_equal(logits_b, last_logits)


def test_encoder_at_benchmark_shape(fdx, oracle, modelgen):
    """The full encoder configuration (fused attention kernel on 64-wide heads, stacked Q/K/V projection, both residual
    Adds in projection epilogues) at batch 32: two samples against the oracle, the others against batch-1 runs."""
    say("encoder 6 x (d512, 8 heads, ffn 2048), seq 256, batch 32")
    js = modelgen.dumps(modelgen.encoder(seed=44, bias_std=0.1, random_affine=True))
    x = np.random.default_rng(45).standard_normal((32, 256, 512)).astype(np.float32)
    model = fdx.Model(js, verify=False)
    got = model.predict([x])[0]
    ref = oracle.OracleModel(js)
    for i in (0, 31):
        want = ref.predict([x[i]])[0]
        e = rel(got[i], want)
        say("  sample %d rel err %.2e" % (i, e))
        assert e <= TOL
    for i in range(1, 31):
        one = model.predict([x[i:i + 1]])[0]
        assert rel(one[0], got[i]) <= 1e-5, i


def _features(modelgen, oracle, spec, tap, sample):
    cfg = spec["architecture"]["config"]
    cfg["output_layers"] = cfg["output_layers"] + [[tap, 0, 0]]
    tmp = dict(spec)
    tmp["output_shapes"] = [[1]] * 2
    spec["output_shapes"] = [list(o.shape) for o in oracle.OracleModel(modelgen.dumps(tmp)).predict([sample])]
    return modelgen.dumps(spec)


@pytest.mark.parametrize("name,batch,small", [("resnet50", 64, 2), ("mobilenet_v2", 128, 8)])
def test_cnn_batch_invariance_and_frozen_tuner(fdx, oracle, modelgen, name, batch, small, tmp_path):
    """At the benchmark batch the tuner picks other kernel variants (split-K, stream-K, fused depthwise pairs) than at
    the small batches the oracle comparisons use.  Samples are independent (include/fdeep/model.hpp:28-42): rows of the
    large batch must equal the same images run at the small batch, one image must meet the oracle, and with the table
    exported, imported and frozen two fresh loads return bit-identical results."""
    say(name, "batch", batch, "vs batch", small)
    spec = getattr(modelgen, name)(seed=46, random_bn=True)
    tap = "avg_pool" if name == "resnet50" else "global_average_pooling2d"
    x = np.random.default_rng(47).uniform(0, 1, (batch, 224, 224, 3)).astype(np.float32)
    js = _features(modelgen, oracle, spec, tap, x[0])
    fdx.tuner_timing(True)  # timing runs are opt-in; the default (closed rules) is what every other test runs on
    model = fdx.Model(js, verify=False)
    first = model.predict([x])
    # With every choice of the plan made, a host input runs the first layers piece by piece behind its copy; the pieces'
    # own shapes are timed on this second pass, after which the process is warmed up for good.
    big = model.predict([x])
    for f, g in zip(first, big):
        assert rel(f, g) <= 3e-5
    picks = [0, batch - 1] + list(range(1, small - 1))
    little = model.predict([x[picks]])
    for g, l in zip(big, little):
        assert rel(g[picks], l) <= 3e-5  # the two batches may run different kernel forms, which sum in different orders
    want = oracle.OracleModel(js).predict([x[batch - 1]])
    for g, w in zip(big, want):
        assert rel(g[batch - 1], w) <= TOL
    # freeze: what this process has tuned becomes the table of "another deployment"
    table = fdx.tuner_export()
    assert len(table.splitlines()) >= 10
    try:
        fdx.tuner_import(table)
        fdx.tuner_freeze(True)
        a = fdx.Model(js, verify=False).predict([x])
        b = fdx.Model(js, verify=False).predict([x])
        for u, v in zip(a, b):
            assert np.array_equal(u, v)
        for u, g in zip(a, big):
            assert np.array_equal(u, g)  # the same table picks the same kernels as the run that made it
        # the deployment itself: a process that has tuned nothing imports the table, freezes it and predicts
        (tmp_path / "table.txt").write_text(table)
        (tmp_path / "model.json").write_bytes(js if isinstance(js, bytes) else js.encode())
        np.save(tmp_path / "x.npy", x)
        import os, subprocess, sys
        root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
        say("  fresh process with the imported table")
        run = subprocess.run([sys.executable, "-c", FRESH_PROCESS_MODEL, root, str(tmp_path)], capture_output=True, text=True, timeout=110)
        assert run.returncode == 0 and run.stdout.strip().endswith("ok"), (run.returncode, run.stdout[-400:], run.stderr[-800:])
        for i, u in enumerate(a):
            assert np.array_equal(u, np.load(tmp_path / ("out%d.npy" % i)))
        # a shape the table has not seen takes the closed rule, and still meets the oracle
        c = fdx.Model(js, verify=False).predict([x[:3]])
        for u, g in zip(c, big):
            assert rel(u, g[:3]) <= 3e-5
    finally:
        fdx.tuner_freeze(False)
        fdx.tuner_timing(False)


@pytest.mark.parametrize("name,batch", [("resnet50", 64), ("mobilenet_v2", 128)])
def test_cnn_closed_rules_and_first_call_latency(fdx, oracle, modelgen, name, batch):
    """The default: nothing is timed, every kernel choice follows the closed rules.  One image of the benchmark batch
    meets the oracle, a second load returns the same bits, and the first predict of the shape (plan building, workspace
    allocation, first launches) costs at most 50 ms more than the tenth."""
    import time
    say(name, "batch", batch, "closed rules, first call against tenth")
    spec = getattr(modelgen, name)(seed=50, random_bn=True)
    tap = "avg_pool" if name == "resnet50" else "global_average_pooling2d"
    x = np.random.default_rng(51).uniform(0, 1, (batch, 224, 224, 3)).astype(np.float32)
    js = _features(modelgen, oracle, spec, tap, x[0])
    model = fdx.Model(js, verify=False)
    d_x = fdx.DevBuf.from_host(x)
    shapes = [(224, 224, 3)]
    d_outs = [fdx.DevBuf(4 * batch * int(np.prod(sh))) for sh in model.infer_shapes(shapes)]
    times = []
    for i in range(10):
        fdx.sync()
        t0 = time.perf_counter()
        model.predict_dev(batch, [d_x], shapes, d_outs)
        fdx.sync()
        times.append((time.perf_counter() - t0) * 1e3)
    say("  first call %.1f ms, tenth %.1f ms" % (times[0], times[9]))
    assert times[0] - times[9] <= 50.0, times
    got = model.predict([x])
    want = oracle.OracleModel(js).predict([x[5]])
    for g, w in zip(got, want):
        assert rel(g[5], w) <= TOL
    again = fdx.Model(js, verify=False).predict([x])
    for g, a in zip(got, again):
        assert np.array_equal(g, a)


def test_predict_from_several_host_threads(fdx, modelgen):
    """model.predict is const and callable from many threads at once (FAQ.md:103-114, include/fdeep/model.hpp:28-42):
    four host threads on one model and on two models concurrently return what the serial calls return."""
    say("predict from four host threads")
    cnn = fdx.Model(modelgen.dumps(modelgen.small_cnn()))
    enc = fdx.Model(modelgen.dumps(modelgen.encoder(seed=48, layers=2, seq=32, d_model=128, heads=2, ffn=256, bias_std=0.1)))
    r = np.random.default_rng(49)
    xs = [r.uniform(-1, 1, (5 + i, 32, 32, 3)).astype(np.float32) for i in range(4)]
    es = [r.standard_normal((2 + i, 32, 128)).astype(np.float32) for i in range(4)]
    serial_c = [cnn.predict([x])[0] for x in xs]
    serial_e = [enc.predict([e])[0] for e in es]
    results, errors = {}, []

    def work(t):
        try:
            for it in range(25):
                i = (t + it) % 4
                if t % 2 == 0 or it % 3 == 0:
                    out = cnn.predict([xs[i]])[0]
                    ok = np.array_equal(out, serial_c[i])
                else:
                    out = enc.predict([es[i]])[0]
                    ok = np.array_equal(out, serial_e[i])
                if not ok:
                    errors.append((t, it, i))
            results[t] = True
        except Exception as exc:  # noqa: BLE001 - reported below
            errors.append((t, repr(exc)))

    threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not errors, errors[:5]
    assert len(results) == 4


FRESH_PROCESS_MODEL = r"""
import importlib, os, sys, numpy as np
sys.path.insert(0, sys.argv[1])
d = sys.argv[2]
fdx = importlib.import_module("frugally-deep_amd")
fdx.tuner_import(open(os.path.join(d, "table.txt")).read())
fdx.tuner_freeze(True)
model = fdx.Model(os.path.join(d, "model.json"), verify=False)
for i, o in enumerate(model.predict([np.load(os.path.join(d, "x.npy"))])):
    np.save(os.path.join(d, "out%d.npy" % i), o)
print("ok", flush=True)
"""


FRESH_PROCESS_IMPORT = r"""
import importlib, sys, numpy as np
sys.path.insert(0, sys.argv[1])
fdx = importlib.import_module("frugally-deep_amd")
# conv M N K Cin kh kw sy sx batch res choice: every tile of a 2048 x 256 x 512 GEMM cut into two K ranges (64 x 64 x 32
# tile), the same as only the last round (hybrid), and as stream-K
m, n, k = 2048, 256, 512
r = np.random.default_rng(5)
a = r.standard_normal((m, k)).astype(np.float32)
w = (r.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
b = r.standard_normal(n).astype(np.float32)
want = a.astype(np.float64) @ w.astype(np.float64).T + b
for choice in (215, 10215, 20015):
    fdx.tuner_import("0 %d %d %d 0 0 0 0 0 1 0 %d\n" % (m, n, k, choice))
    fdx.tuner_freeze(True)
    got = fdx.gemm(a, w, b)
    err = float(np.abs(got - want).max() / np.abs(want).max())
    print("choice", choice, "err", err, flush=True)
    assert err < 1e-5, err
print("ok", flush=True)
"""


def test_imported_split_choice_in_a_fresh_process(fdx):
    """A deployment imports its tuner table before anything has run: the split variants' workspace, which the timing
    runs of a tuning process allocate on the way, has to be there for the first launch all the same."""
    import os, subprocess, sys
    say("imported table, fresh process")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", FRESH_PROCESS_IMPORT, root], capture_output=True, text=True, timeout=110)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), (out.returncode, out.stdout[-400:], out.stderr[-800:])
