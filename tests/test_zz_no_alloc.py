"""The Dense entry point that allocates nothing (its split-K scratch is a fixed device array inside the library)
against fdx_dense_rows_f32, which allocates its workspace on first use: same kernels, same split, so the results must be
bit-identical.  Two calls in a row, the second on a smaller input, then the limits."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _run(fdx, fn, x, w, b, res, act):
    m, k = x.shape
    n = w.shape[0]
    dx, dw, db, dr = (fdx.DevBuf.from_host(a) for a in (x, w, b, res))
    out = fdx.DevBuf.from_host(np.full((m, n), np.nan, np.float32))
    fdx.check(fn(fdx._dp(dx), m, k, fdx._dp(dw), fdx._dp(db), n, fdx._dp(dr), fdx.ctypes.byref(act), fdx._dp(out)))
    return out.to_host((m, n))


def test_no_alloc_dense_rows_equals_the_allocating_entry_point(fdx, oracle):
    fdx.check(fdx.lib.fdx_init(0))
    r = np.random.default_rng(71)
    act = fdx.gelu_act()
    # (16, 3072, 768): 48 column groups x 4 K ranges through the scratch array; then smaller: (5, 2048, 320), 20 x 2;
    # then one that needs no scratch at all
    for m, k, n in [(16, 3072, 768), (5, 2048, 320), (3, 64, 100)]:
        print("no-alloc dense_rows", m, k, n, flush=True)
        x = r.standard_normal((m, k)).astype(np.float32)
        w = (r.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
        b = r.standard_normal(n).astype(np.float32)
        res = r.standard_normal((m, n)).astype(np.float32)
        want = _run(fdx, fdx.lib.fdx_dense_rows_f32, x, w, b, res, act)
        got = _run(fdx, fdx.lib.fdx_dense_rows_noalloc_f32, x, w, b, res, act)
        assert np.array_equal(got, want), (m, k, n, np.abs(got - want).max())
        ref = oracle.gelu(oracle.dense(x, np.ascontiguousarray(w.T).reshape(-1), b, n) + res)
        assert np.abs(got - ref).max() / np.abs(ref).max() <= 1e-4


def test_no_alloc_dense_rows_rejects_sizes_beyond_its_scratch(fdx):
    fdx.check(fdx.lib.fdx_init(0))
    buf = fdx.DevBuf(64)
    for m, k, n, text in [(17, 64, 64, "1 to 16 rows"), (4, 64, 70000, "output columns"), (4, 40000, 64, "input columns"),
                          (4, 8192, 65536, "exceed the fixed scratch")]:
        st = fdx.lib.fdx_dense_rows_noalloc_f32(fdx._dp(buf), m, k, fdx._dp(buf), None, n, None, None, fdx._dp(buf))
        assert st != 0
        assert text in fdx.lib.fdx_last_error().decode(), (m, k, n, fdx.lib.fdx_last_error())
