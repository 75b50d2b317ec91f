"""KV-cache decode sessions against the oracle's causal definition (row t = the reference's
MultiHeadAttention(query = x[t:t+1], value = x[0:t+1])).  Logits: max|gpu - ref| / max|ref| <= 1e-4;
greedy token ids must be identical wherever the oracle's top-2 logit margin exceeds 1e-3."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-4


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    assert a.shape == b.shape
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)


def say(*a):
    print(*a, flush=True)


def oracle_logits(ref, ids):
    """ids [t] -> logits [t, vocab] under causal attention."""
    pos = np.arange(len(ids), dtype=np.float32)
    return ref.predict([np.asarray(ids, np.float32), pos], causal=True)[0]


def margin(row):
    top = np.sort(row)[-2:]
    return top[1] - top[0]


@pytest.mark.parametrize("cfg", [dict(layers=2, d_model=32, heads=4, vocab=97, max_pos=40),
                                 dict(layers=3, d_model=64, heads=2, vocab=211, max_pos=40)])
def test_prefill_then_decode_matches_oracle(fdx, oracle, modelgen, cfg):
    say("session tiny", cfg)
    spec = modelgen.gpt2(seed=31, bias_std=0.1, random_affine=True, std=0.2, **cfg)
    js = modelgen.dumps(spec)
    ref = oracle.OracleModel(js)
    model = fdx.Model(js)
    B, P, N = 3, 7, 6
    r = np.random.default_rng(32)
    prompts = r.integers(0, cfg["vocab"], (B, P))
    sess = fdx.Session(model, B, 32)
    logits, nxt = sess.prefill(prompts)
    seqs = [list(prompts[b]) for b in range(B)]
    for b in range(B):
        want = oracle_logits(ref, seqs[b])[-1]
        assert rel(logits[b], want) <= TOL
        if margin(want) > 1e-3:
            assert nxt[b] == oracle.argmax(want)
    assert sess.length() == P
    # teacher-forced decode steps: feed the oracle's greedy token so both sides see the same history
    for step in range(N):
        feed = []
        for b in range(B):
            feed.append(oracle.argmax(oracle_logits(ref, seqs[b])[-1]))
            seqs[b].append(feed[-1])
        logits, nxt = sess.decode_step(np.array(feed))
        for b in range(B):
            want = oracle_logits(ref, seqs[b])[-1]
            assert rel(logits[b], want) <= TOL, (step, b)
            if margin(want) > 1e-3:
                assert nxt[b] == oracle.argmax(want)
    assert sess.length() == P + N
    # chunked prefill (a second multi-token call on a non-empty cache) equals one long prefill
    sess.reset()
    sess.prefill(prompts[:, :4])
    logits2, _ = sess.prefill(prompts[:, 4:])
    sess.reset()
    logits1, _ = sess.prefill(prompts)
    assert rel(logits2, logits1) <= 1e-5


def test_greedy_loop_equals_stepwise_and_full_recompute(fdx, oracle, modelgen):
    say("session greedy")
    cfg = dict(layers=2, d_model=48, heads=3, vocab=151, max_pos=64)
    js = modelgen.dumps(modelgen.gpt2(seed=33, bias_std=0.1, random_affine=True, std=0.2, **cfg))
    model = fdx.Model(js)
    B, P, N = 4, 9, 12
    prompts = np.random.default_rng(34).integers(0, cfg["vocab"], (B, P))
    sess = fdx.Session(model, B, 64)
    _, first = sess.prefill(prompts)
    tokens, last_logits = sess.decode_greedy(first, N)
    # step-by-step session gives the same tokens
    sess2 = fdx.Session(model, B, 64)
    _, nxt = sess2.prefill(prompts)
    assert np.array_equal(nxt, first)
    cur = first
    for i in range(N):
        logits, nxt = sess2.decode_step(cur)
        assert np.array_equal(nxt, tokens[i])
        cur = nxt
    assert rel(logits, last_logits) <= 1e-6
    # prefix identity on the GPU itself: prefilling the whole generated sequence reproduces the last logits
    full = np.concatenate([prompts, first[:, None], tokens[:-1].T], axis=1)
    sess3 = fdx.Session(model, B, 64)
    logits3, nxt3 = sess3.prefill(full)
    assert rel(logits3, last_logits) <= 1e-5
    # and the oracle agrees on one sequence
    ref = oracle.OracleModel(js)
    want = oracle_logits(ref, full[0])[-1]
    assert rel(last_logits[0], want) <= TOL


def test_session_rejects_non_decoder_models_and_overflow(fdx, modelgen):
    say("session errors")
    cnn = fdx.Model(modelgen.dumps(modelgen.small_cnn()))
    with pytest.raises(fdx.FdxError):
        fdx.Session(cnn, 1, 8)
    js = modelgen.dumps(modelgen.gpt2(seed=35, layers=1, d_model=16, heads=2, vocab=19, max_pos=16))
    sess = fdx.Session(fdx.Model(js), 2, 4)
    sess.prefill(np.zeros((2, 3)))
    sess.decode_step(np.zeros(2))
    with pytest.raises(fdx.FdxError, match="exceeds max_len"):
        sess.decode_step(np.zeros(2))


def test_session_rejects_layers_that_mix_positions(fdx, modelgen):
    """A cached decode step works on one position at a time: LayerNormalization over anything but the depth axis and
    Flatten / Reshape layers (which regroup the (T, depth) sample) are refused when the session is created, instead of
    being computed over one position's depth."""
    say("session: position-mixing layers")
    import copy
    base = modelgen.gpt2(seed=40, layers=1, d_model=16, heads=2, vocab=19, max_pos=16)
    for axis in ([1], [1, 2], [-2]):
        spec = copy.deepcopy(base)
        for layer in spec["architecture"]["config"]["layers"]:
            if layer["name"] == "h0_ln2":
                layer["config"]["axis"] = axis
        with pytest.raises(fdx.FdxError, match="axis other than the last"):
            fdx.Session(fdx.Model(modelgen.dumps(spec), verify=False), 2, 8)
    for cls, cfg in (("Reshape", {"target_shape": [-1, 16]}), ("Flatten", {})):
        b = modelgen.Builder("mix", 41)
        ids, pos = b.input((None,), "ids"), b.input((None,), "positions")
        x = b.add([b.embedding(ids, 19, 16, "wte"), b.embedding(pos, 16, 16, "wpe")], "embed_add")
        h = b.layernorm(x, "ln1", 1e-5)
        h = b.mha(h, h, "attn", 2, 8)
        x = b.add([x, h], "add1")
        x = b._add(cls, "regroup", cfg, [x], x.shape)
        x = b.dense(x, 19, "lm_head")
        model = fdx.Model(modelgen.dumps(b.finish([x])), verify=False)
        with pytest.raises(fdx.FdxError, match="reshapes across positions"):
            fdx.Session(model, 2, 8)
    fdx.Session(fdx.Model(modelgen.dumps(base), verify=False), 2, 8)  # the unmodified decoder is accepted


def test_vocabulary_sized_head_leaves_its_own_argmax(fdx, modelgen):
    """With tens of thousands of logits per row the logits launch strides over the column groups and leaves
    per-workgroup maxima, from which the greedy ids are picked without another pass over the logits: the ids must be
    the first maximum of the logits the same step returns, for batch sizes that fill and do not fill the 16 rows,
    and the captured loop must produce the same tokens as single steps."""
    say("session with a vocabulary-sized head")
    cfg = dict(layers=1, d_model=64, heads=1, vocab=40009, max_pos=32)
    js = modelgen.dumps(modelgen.gpt2(seed=36, bias_std=0.1, random_affine=True, std=0.2, **cfg))
    model = fdx.Model(js)
    for B in (16, 5):
        prompts = np.random.default_rng(37 + B).integers(0, cfg["vocab"], (B, 6))
        sess = fdx.Session(model, B, 32)
        logits, first = sess.prefill(prompts)
        assert np.array_equal(first, np.argmax(logits, -1).astype(first.dtype))
        tokens, last_logits = sess.decode_greedy(first, 7)
        sess2 = fdx.Session(model, B, 32)
        _, cur = sess2.prefill(prompts)
        for i in range(7):
            logits, nxt = sess2.decode_step(cur)
            assert np.array_equal(nxt, np.argmax(logits, -1).astype(nxt.dtype)), (B, i)
            assert np.array_equal(nxt, tokens[i]), (B, i)
            cur = nxt
        assert rel(logits, last_logits) <= 1e-6


def test_attention_with_output_projection_in_one_launch(fdx, oracle, modelgen, monkeypatch):
    """With 64-wide heads the decode step runs attention and the layer's output projection (bias, residual Add) as one
    launch whose per-head partial rows are added in head order by the last workgroup to arrive, when FDX_DECODE_FUSE_PROJ=1
    is set while the session is created (two launches measure slightly faster and are the default).  Both forms against each other, step by step and in the
    captured loop, for a batch that fills the 16 rows and one that does not, and the fused form against the oracle."""
    say("decode attention + output projection, one launch vs two")
    cfg = dict(layers=3, d_model=192, heads=3, vocab=211, max_pos=64)
    js = modelgen.dumps(modelgen.gpt2(seed=38, bias_std=0.1, random_affine=True, std=0.2, **cfg))
    model = fdx.Model(js)
    ref = oracle.OracleModel(js)
    for B in (16, 5):
        P, N = 7, 20
        prompts = np.random.default_rng(39 + B).integers(0, cfg["vocab"], (B, P))
        two = fdx.Session(model, B, 64)
        monkeypatch.setenv("FDX_DECODE_FUSE_PROJ", "1")
        one = fdx.Session(model, B, 64)
        monkeypatch.delenv("FDX_DECODE_FUSE_PROJ")
        _, first = two.prefill(prompts)
        _, first1 = one.prefill(prompts)
        assert np.array_equal(first, first1)
        want_tokens, want_logits = two.decode_greedy(first, N)
        tokens, logits = one.decode_greedy(first1, N)
        assert np.array_equal(tokens, want_tokens)
        assert rel(logits, want_logits) <= 1e-5
        # single steps, twice over the same positions after a reset (the tickets must be back at zero)
        for _ in range(2):
            one.reset()
            two.reset()
            _, cur = one.prefill(prompts)
            two.prefill(prompts)
            for i in range(6):
                la, na = two.decode_step(cur)
                lb, nb = one.decode_step(cur)
                assert np.array_equal(na, nb) and np.array_equal(nb, want_tokens[i])
                assert rel(lb, la) <= 1e-5
                cur = nb
        seq = np.concatenate([prompts[0], first[:1], want_tokens[:5, 0]]).astype(np.float32)
        want = oracle_logits(ref, seq)[-1]
        assert rel(lb[0], want) <= TOL


def test_embedding_folded_into_its_readers_gives_the_same_tokens(fdx, modelgen):
    """The opt-in form of the decode step in which the first projection GEMM and the first residual operand form the
    token + position rows themselves (one launch fewer): same sums in the same order, so logits and tokens are
    bit-identical to the default step."""
    print("decode step with the embedding folded into its readers", flush=True)
    js = modelgen.dumps(modelgen.gpt2(seed=61, layers=2, d_model=768, heads=12, vocab=50257, max_pos=128, bias_std=0.1,
                                      random_affine=True))
    model = fdx.Model(js, verify=False)
    B, P, N = 16, 24, 12
    prompts = np.random.default_rng(62).integers(0, 50257, (B, P))
    outs = []
    for mode in (0, 1):
        fdx.check(fdx.lib.fdx_debug_decode_embed_fold(mode))
        try:
            sess = fdx.Session(model, B, 64)
        finally:
            fdx.check(fdx.lib.fdx_debug_decode_embed_fold(-1))
        _, first = sess.prefill(prompts)
        tokens, logits = sess.decode_greedy(first, N)
        step_logits, step_next = sess.decode_step(tokens[-1])
        outs.append((tokens, logits, step_logits, step_next))
        sess.close()
    for a, b in zip(outs[0], outs[1]):
        assert np.array_equal(a, b)


def test_greedy_loop_with_the_embedding_in_the_previous_steps_last_launch(fdx, modelgen):
    """Inside a greedy loop over a vocabulary-sized head the token + position embedding of a step rides in the last launch
    of the step before (the loop's first embedding runs ahead of the replays).  The loop, called twice with a single
    step in between, must give the tokens of single steps; a loop that would run past the position table keeps the
    stand-alone embedding launch."""
    say("greedy loop, embedding merged into the arg-max launch")
    cfg = dict(layers=2, d_model=64, heads=2, vocab=40009, max_pos=24)
    js = modelgen.dumps(modelgen.gpt2(seed=63, bias_std=0.1, random_affine=True, std=0.2, **cfg))
    model = fdx.Model(js)
    B = 6
    prompts = np.random.default_rng(64).integers(0, cfg["vocab"], (B, 5))
    loop = fdx.Session(model, B, 32)
    _, first = loop.prefill(prompts)
    part1, _ = loop.decode_greedy(first, 6)            # positions 5 .. 10
    _, mid = loop.decode_step(part1[-1])               # a single step between two loops (position 11)
    part2, last_logits = loop.decode_greedy(mid, 7)    # positions 12 .. 18
    single = fdx.Session(model, B, 32)
    _, cur = single.prefill(prompts)
    want = []
    for i in range(6 + 1 + 7):
        logits, cur_next = single.decode_step(cur)
        want.append(cur_next)
        cur = cur_next
    got = list(part1) + [mid] + list(part2)
    for i, (g, w) in enumerate(zip(got, want)):
        assert np.array_equal(g, w), i
    assert rel(logits, last_logits) <= 1e-6
    # positions 19 .. 23 exist, 24 does not: a loop of 6 from here runs past the table and takes the stand-alone embedding
    # launches, like the single steps (a position without a row contributes zeros in both)
    part3, _ = loop.decode_greedy(part2[-1], 6)
    for i in range(6):
        _, cur = single.decode_step(cur)
        assert np.array_equal(part3[i], cur), i
