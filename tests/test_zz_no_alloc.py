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


FRESH_PROCESS = r"""
import ctypes, importlib, sys
import numpy as np
sys.path.insert(0, sys.argv[1])
fdx = importlib.import_module("frugally-deep_amd")
fdx.check(fdx.lib.fdx_init(0))
r = np.random.default_rng(72)
m, k, n = 16, 3072, 768   # 48 column groups x 4 K ranges: the shape that needs the scratch
x = r.standard_normal((m, k)).astype(np.float32)
w = (r.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
b = r.standard_normal(n).astype(np.float32)
res = r.standard_normal((m, n)).astype(np.float32)
dx, dw, db, dr = (fdx.DevBuf.from_host(a) for a in (x, w, b, res))
out = fdx.DevBuf.from_host(np.full((m, n), np.nan, np.float32))
act = fdx.gelu_act()
# one small call of the same entry point first (a shape that needs no scratch): the runtime loads the library's GPU code
# on the first launch, which takes device memory once per process whichever kernel comes first
tiny = fdx.DevBuf.from_host(np.zeros((3, 100), np.float32))
fdx.check(fdx.lib.fdx_dense_rows_noalloc_f32(fdx._dp(dx), 3, 64, fdx._dp(dw), None, 100, None, None, fdx._dp(tiny)))
fdx.sync()
free0, free1, total = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
fdx.check(fdx.lib.fdx_dev_mem_info(ctypes.byref(free0), ctypes.byref(total)))
# the first compute call of this process: nothing has allocated a workspace on its behalf
fdx.check(fdx.lib.fdx_dense_rows_noalloc_f32(fdx._dp(dx), m, k, fdx._dp(dw), fdx._dp(db), n, fdx._dp(dr), ctypes.byref(act), fdx._dp(out)))
fdx.sync()
fdx.check(fdx.lib.fdx_dev_mem_info(ctypes.byref(free1), ctypes.byref(total)))
print("free before", free0.value, "after", free1.value, flush=True)
assert free1.value == free0.value, (free0.value, free1.value)
got = out.to_host((m, n))
want = x.astype(np.float64) @ w.astype(np.float64).T + b + res
want = 0.5 * want * (1.0 + np.vectorize(__import__("math").erf)(want / np.sqrt(2.0)))
err = float(np.abs(got - want).max() / np.abs(want).max())
print("err", err, flush=True)
assert err < 1e-5, err
# and the allocating entry point, called afterwards, returns the same bits
out2 = fdx.DevBuf.from_host(np.full((m, n), np.nan, np.float32))
fdx.check(fdx.lib.fdx_dense_rows_f32(fdx._dp(dx), m, k, fdx._dp(dw), fdx._dp(db), n, fdx._dp(dr), ctypes.byref(act), fdx._dp(out2)))
assert np.array_equal(out2.to_host((m, n)), got)
print("ok", flush=True)
"""


def test_no_alloc_dense_rows_first_in_a_fresh_process_leaves_device_memory_alone(fdx):
    """The property the entry point exists for: called as the first compute call of a process (no allocating entry point
    has run, so no workspace exists that it could lean on), the free device memory is the same before and after."""
    import os, subprocess, sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", FRESH_PROCESS, root], capture_output=True, text=True, timeout=300)
    print(out.stdout, out.stderr[-2000:], flush=True)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok")


def test_no_alloc_dense_rows_rejects_sizes_beyond_its_scratch(fdx):
    fdx.check(fdx.lib.fdx_init(0))
    buf = fdx.DevBuf(64)
    for m, k, n, text in [(17, 64, 64, "1 to 16 rows"), (4, 64, 70000, "output columns"), (4, 40000, 64, "input columns"),
                          (4, 8192, 65536, "exceed the fixed scratch")]:
        st = fdx.lib.fdx_dense_rows_noalloc_f32(fdx._dp(buf), m, k, fdx._dp(buf), None, n, None, None, fdx._dp(buf))
        assert st != 0
        assert text in fdx.lib.fdx_last_error().decode(), (m, k, n, fdx.lib.fdx_last_error())
    # an activation no epilogue carries: refused as by every launcher with an epilogue
    tanh = fdx.named_act("tanh")
    st = fdx.lib.fdx_dense_rows_noalloc_f32(fdx._dp(buf), 4, 64, fdx._dp(buf), None, 64, None, fdx.ctypes.byref(tanh), fdx._dp(buf))
    assert st == 4  # FDX_ERR_UNSUPPORTED
