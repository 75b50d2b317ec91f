"""Benchmark of the forward hot path on one MI355X.  Prints ONE JSON line.

Primary figure (BASELINE.json metric, configs[1]): ResNet50-architecture CNN, fp32, batch 64, 224x224x3,
random-init He-normal weights, synthetic uniform[0,1] inputs already resident in HBM.  One step = one batched
predict (fdx_model_predict_dev) of 64 images; `value` = images / second.

Second half of the metric, reported under "gpt2_decode": GPT-2-small-shaped decoder (12 layers, d 768, 12 heads,
vocab 50257, untied head), batch 16, prompt 128 random ids, then 128 greedy tokens with the key/value cache;
tokens / second over the decode loop and the fraction of the HBM roofline for the bytes a step must stream.
"""
import argparse
import concurrent.futures
import ctypes
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "oracle")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_FP32_MFMA_TFLOPS = 157.3  # MI355X dense fp32 matrix peak
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
# HBM bytes per launch of each workload's dominant kernel, measured with rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs
# of this file and scaled by a plain copy of known size (a process cannot read these counters for itself; the
# summaries under profiles/ give the commands and the raw readings).  Valid for the default configurations only.
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = {"igemm + wino, ResNet50 b64": 163.5e6, "skinny_gemm, GPT-2 decode b16": 11.3e6}


def under_profiler():
    """True when a ROCm profiler drives this process (rocprofv3 preloads its tool library and sets ROCPROF* variables)."""
    pre = os.environ.get("LD_PRELOAD", "")
    return "rocprofiler" in pre or "rocprof" in pre or any(k.startswith(("ROCPROF", "ROCPROFILER")) for k in os.environ)


def log_address_map(stage):
    """Under a profiler: keeps a copy of /proc/self/maps per stage, so that a fault address from a runtime or profiler
    thread (none of the library's own: it starts no threads) can be attributed to a mapping afterwards."""
    if not under_profiler():
        return
    try:
        out_dir = os.path.join(ROOT, "gpurun_out")
        os.makedirs(out_dir, exist_ok=True)
        with open("/proc/self/maps") as src, open(os.path.join(out_dir, "bench_maps_%d_%s.txt" % (os.getpid(), stage)), "w") as dst:
            dst.write(src.read())
    except OSError:
        pass


def load_package():
    import __graft_entry__ as entry
    entry._ensure_built()
    return importlib.import_module("frugally-deep_amd"), importlib.import_module("frugally-deep_amd.modelgen")


def profile_families(fdx):
    fams = {}
    i = 0
    while True:
        name = ctypes.create_string_buffer(128)
        launches, ms, flops, nbytes = ctypes.c_uint64(), ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
        if fdx.lib.fdx_profile_get(i, name, 128, ctypes.byref(launches), ctypes.byref(ms), ctypes.byref(flops),
                                   ctypes.byref(nbytes)) != 0:
            break
        executed = ctypes.c_double()
        fdx.check(fdx.lib.fdx_profile_get_executed(i, ctypes.byref(executed)))
        fams[name.value.decode()] = dict(launches=launches.value, ms=ms.value, flops=flops.value, bytes=nbytes.value,
                                         executed=executed.value)
        i += 1
    return fams


def host_cores():
    """Host threads the CPU baseline uses: the cores this process may run on, at most the 16 a one-GPU box grants."""
    try:
        n = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        n = os.cpu_count() or 1
    return max(1, min(n, 16))


def cpu_model_name():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


CPU_BUILD = None
CPU_KIND_NOTE = "restated reference CPU path (no Eigen): the oracle's plain-C port of the reference algorithm, kind 'port'"


def cpu_baseline_resnet(js, x, cores, warmup=3, passes=5):
    """The oracle (a port of the reference CPU path) timed with one prediction per core in parallel threads, 3 warm-up
    and 5 timed passes as the reference's own harness does (test/applications_performance.cpp:59-77)."""
    import fdeep_oracle
    global CPU_BUILD
    CPU_BUILD = fdeep_oracle.use_native_build()
    ref = fdeep_oracle.OracleModel(js)
    samples = [x[i % x.shape[0]] for i in range(cores)]
    with concurrent.futures.ThreadPoolExecutor(cores) as pool:
        for _ in range(warmup):
            list(pool.map(lambda s: ref.predict([s]), samples))
        t0 = time.perf_counter()
        for _ in range(passes):
            list(pool.map(lambda s: ref.predict([s]), samples))
        dt = time.perf_counter() - t0
    return cores * passes / dt


def cpu_baseline_decode(js, cores, prompt=4, warmup=3, timed=5):
    """KV-cached greedy decoding on the CPU oracle, one sequence per core in parallel threads: a short prompt and 3
    warm-up steps per sequence, then 5 timed steps each (a step streams every weight of the model once per sequence,
    whatever the context length, so the short context hardly changes its cost)."""
    import fdeep_oracle
    global CPU_BUILD
    CPU_BUILD = fdeep_oracle.use_native_build()
    ref = fdeep_oracle.OracleModel(js)
    rng = np.random.default_rng(7)
    decoders = [fdeep_oracle.CachedDecoder(ref) for _ in range(cores)]
    state = [int(t) for t in rng.integers(0, 50257, cores)]

    def run(i, steps):
        tok = state[i]
        for _ in range(steps):
            tok = fdeep_oracle.argmax(decoders[i].step(tok))
        state[i] = tok

    with concurrent.futures.ThreadPoolExecutor(cores) as pool:
        list(pool.map(lambda i: run(i, prompt + warmup), range(cores)))
        t0 = time.perf_counter()
        list(pool.map(lambda i: run(i, timed), range(cores)))
        dt = time.perf_counter() - t0
    return cores * timed / dt


def shader_clock_during(fdx, run_step, steps, ms_per_step):
    """Shader clock (GHz) while `steps` forward passes run: the library's probe samples the cycle counter against the
    constant-rate wall counter every 100 us on a stream of its own.  Outside the timed region."""
    period_us = 100
    window_ms = steps * ms_per_step
    samples = int(min(65536, max(8, window_ms * 1e3 / period_us * 1.05 + 4)))
    fdx.sync()
    fdx.check(fdx.lib.fdx_clock_probe_start(samples, period_us))
    for _ in range(steps):
        run_step()
    fdx.sync()
    mean, lo, hi = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
    fdx.check(fdx.lib.fdx_clock_probe_stop(ctypes.c_double(window_ms), ctypes.byref(mean), ctypes.byref(lo), ctypes.byref(hi)))
    # the same probe with nothing else running
    fdx.check(fdx.lib.fdx_clock_probe_start(64, period_us))
    imean, ilo, ihi = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
    fdx.check(fdx.lib.fdx_clock_probe_stop(ctypes.c_double(6.0), ctypes.byref(imean), ctypes.byref(ilo), ctypes.byref(ihi)))
    return {"mean_ghz": round(mean.value, 3), "min_ghz": round(lo.value, 3), "max_ghz": round(hi.value, 3),
            "idle_ghz": round(imean.value, 3),
            "what": "shader cycle counter against the 100 MHz wall counter, one sample per 100 us over %d forward passes "
                    "run after the timed region (min / max: single periods); idle = the same probe with nothing else running. "
                    "The published peak the roofline uses assumes 2.4 GHz" % steps}


def bench_resnet(fdx, modelgen, args):
    batch = args.batch
    spec = modelgen.resnet50()
    flops_per_image = modelgen.model_flops(spec)
    js = modelgen.dumps(spec)
    t0 = time.perf_counter()
    model = fdx.Model(js, verify=False)
    load_s = time.perf_counter() - t0

    x = np.random.default_rng(1234).uniform(0, 1, (batch, 224, 224, 3)).astype(np.float32)
    d_in = fdx.DevBuf.from_host(x)
    d_out = fdx.DevBuf(4 * batch * 1000)
    shapes = [(224, 224, 3)]

    fdx.sync()
    t0 = time.perf_counter()
    model.predict_dev(batch, [d_in], shapes, [d_out])
    fdx.sync()
    first_call_ms = (time.perf_counter() - t0) * 1e3
    for _ in range(args.warmup):
        model.predict_dev(batch, [d_in], shapes, [d_out])
    fdx.sync()
    ms = ctypes.c_float()
    t0 = time.perf_counter()
    fdx.check(fdx.lib.fdx_timer_start())
    for _ in range(args.steps):
        model.predict_dev(batch, [d_in], shapes, [d_out])
    fdx.check(fdx.lib.fdx_timer_stop(ctypes.byref(ms)))
    fdx.sync()
    wall_s = time.perf_counter() - t0
    seconds = max(ms.value / 1e3, 1e-9)
    img_s = batch * args.steps / seconds
    probs = d_out.to_host((batch, 1000))
    assert np.isfinite(probs).all() and np.abs(probs.sum(-1) - 1).max() < 1e-3

    # per-kernel pass: HIP events around every launch on the library stream (same work, outside the timed region)
    prof_steps = max(2, args.steps // 4)
    fdx.check(fdx.lib.fdx_profile_enable(1))
    fdx.check(fdx.lib.fdx_profile_reset())
    for _ in range(prof_steps):
        model.predict_dev(batch, [d_in], shapes, [d_out])
    fdx.sync()
    fams = profile_families(fdx)
    fdx.check(fdx.lib.fdx_profile_enable(0))
    mfma = {k: v for k, v in fams.items() if v["flops"] > 0}
    mf_flops = sum(v["flops"] for v in mfma.values())
    mf_ms = sum(v["ms"] for v in mfma.values())
    mf_launches = sum(v["launches"] for v in mfma.values())
    achieved = mf_flops / (mf_ms / 1e3) / 1e12 if mf_ms > 0 else 0.0
    # what the matrix cores really issued: the Winograd launches carry 16 products per 2x2 output tile where the direct
    # sum has 36, so their algorithmic figure can exceed the peak; this one cannot
    executed = sum(v["executed"] for v in mfma.values()) / (mf_ms / 1e3) / 1e12 if mf_ms > 0 else 0.0
    total_ms = sum(v["ms"] for v in fams.values())

    result = {
        "metric": "ResNet50-shape img/s (fp32,b%d)" % args.batch,
        "value": round(img_s, 2),
        "unit": "img/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(seconds * 1e3 / args.steps, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "ResNet50-architecture CNN, random-init He-normal fp32, 224x224x3 uniform[0,1], batch %d" % batch,
                   "batch": batch, "gflop_per_image": round(flops_per_image / 1e9, 4)},
        "model_roofline_frac": round(img_s * flops_per_image / (PEAK_FP32_MFMA_TFLOPS * 1e12), 4),
        "roofline": {
            "bound": "mfma",
            "kernel": "igemm_fast_kernel (implicit-GEMM Conv2D / GEMM, fp32 MFMA, all tile instantiations) + wino_kernel (3x3 stride-1 "
                      "convolutions, Winograd F(2x2,3x3) on fp32 MFMA); flops are the algorithmic direct-sum count of every launch",
            "achieved": round(achieved, 3),
            "peak": PEAK_FP32_MFMA_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
            "executed_achieved": round(executed, 3),
            "executed_frac": round(executed / PEAK_FP32_MFMA_TFLOPS, 4),
            "executed_note": "multiply-adds the kernels issue (Winograd launches: 16 per 2x2 output tile and channel pair instead of "
                             "36) / time / peak: the hardware utilisation, where frac is the algorithmic direct-sum rate",
            "family_tflops": {k: {"algorithmic": round(v["flops"] / (v["ms"] / 1e3) / 1e12, 2),
                                  "executed": round(v["executed"] / (v["ms"] / 1e3) / 1e12, 2)} for k, v in sorted(mfma.items()) if v["ms"] > 0},
            "flops_per_launch": round(mf_flops / max(mf_launches, 1), 1),
            "avg_launch_ms": round(mf_ms / max(mf_launches, 1), 5),
            "share_of_step_time": round(mf_ms / total_ms, 4) if total_ms else None,
            "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH["igemm + wino, ResNet50 b64"] if batch == 64 else None,
        },
        "kernel_ms_per_step": {k: round(v["ms"] / prof_steps, 4) for k, v in sorted(fams.items())},
        "wall_ms_per_step": round(wall_s * 1e3 / args.steps, 4),
        "load_seconds": round(load_s, 2),
        "first_call_ms": round(first_call_ms, 1),
        "kernel_choice": "timed per shape on first sight (--tune)" if args.tune else "closed rules, nothing timed (the library's default)",
    }
    if not args.no_clock_probe:
        result["shader_clock"] = shader_clock_during(fdx, lambda: model.predict_dev(batch, [d_in], shapes, [d_out]), args.steps,
                                                     seconds * 1e3 / args.steps)
    # what a model.predict caller with host tensors sees: the same batch through fdx_model_predict, host-to-device copy
    # of the 38.5 MB input and device-to-host copy of the outputs included (pageable host memory on the caller's side)
    for _ in range(3):
        model.predict([x])
    reps = max(5, args.steps // 2)
    t0 = time.perf_counter()
    for _ in range(reps):
        model.predict([x])
    e2e_s = (time.perf_counter() - t0) / reps
    result["end_to_end"] = {"value": round(batch / e2e_s, 1), "unit": "img/s", "ms_per_step": round(e2e_s * 1e3, 3),
                            "what": "fdx_model_predict on host pointers (pageable numpy memory), batch %d: input H2D + forward + output "
                                    "D2H, wall clock; the input travels in four pieces through pinned buffers and the first layers run "
                                    "piece by piece behind the copy" % batch}
    if not args.no_cpu_baseline:
        cores = host_cores()
        cpu = cpu_baseline_resnet(js, x, cores)
        result["cpu_baseline"] = {"value": round(cpu, 3), "unit": "img/s", "cores": cores, "kind": "port",
                                  "what": CPU_KIND_NOTE, "build": CPU_BUILD, "cpu": cpu_model_name(),
                                  "sample": "%d ResNet50 predictions per pass (one per core, in parallel threads), "
                                            "3 warm-up + 5 timed passes of the CPU oracle" % cores}
    model.close()
    return result


def bench_secondary(fdx, modelgen, name, spec, batch, inputs, steps, warmup, clock_probe=True):
    """Secondary configurations (MobileNetV2 b128, transformer encoder b32): samples / second of one batched predict
    with inputs resident, and per kernel family the HIP-event time with its own roofline (TFLOP/s against the fp32
    MFMA peak for the GEMM families, algorithmic GB/s against HBM for the memory-bound ones)."""
    js = modelgen.dumps(spec)
    model = fdx.Model(js, verify=False)
    shapes = [tuple(x.shape[1:]) for x in inputs]
    d_in = [fdx.DevBuf.from_host(x) for x in inputs]
    out_shapes = model.infer_shapes(shapes)
    d_out = [fdx.DevBuf(4 * batch * int(np.prod(s))) for s in out_shapes]
    for _ in range(warmup):
        model.predict_dev(batch, d_in, shapes, d_out)
    fdx.sync()
    ms = ctypes.c_float()
    fdx.check(fdx.lib.fdx_timer_start())
    for _ in range(steps):
        model.predict_dev(batch, d_in, shapes, d_out)
    fdx.check(fdx.lib.fdx_timer_stop(ctypes.byref(ms)))
    flops = model.last_flops()
    y = d_out[0].to_host((batch,) + tuple(out_shapes[0]))
    assert np.isfinite(y).all()
    fdx.check(fdx.lib.fdx_profile_enable(1))
    fdx.check(fdx.lib.fdx_profile_reset())
    prof_steps = 3
    for _ in range(prof_steps):
        model.predict_dev(batch, d_in, shapes, d_out)
    fdx.sync()
    fams = profile_families(fdx)
    fdx.check(fdx.lib.fdx_profile_enable(0))
    per_family = {}
    for k, v in sorted(fams.items()):
        e = {"ms_per_step": round(v["ms"] / prof_steps, 4), "launches_per_step": v["launches"] // prof_steps}
        if v["flops"] > 0:
            tf = v["flops"] / (v["ms"] / 1e3) / 1e12
            e.update(TFLOP_s=round(tf, 2), mfma_frac=round(tf / PEAK_FP32_MFMA_TFLOPS, 4))
        elif v["bytes"] > 0:
            gb = v["bytes"] / (v["ms"] / 1e3) / 1e9
            e.update(GB_s=round(gb, 1), hbm_frac=round(gb / PEAK_HBM_GBS, 4))
        per_family[k] = e
    sec = ms.value / 1e3 / steps
    res = {"workload": name, "batch": batch, "value": round(batch / sec, 1), "unit": "samples/s", "ms_per_step": round(sec * 1e3, 4),
           "gflop_per_sample": round(flops / batch / 1e9, 4),
           "model_mfma_frac": round(flops / sec / (PEAK_FP32_MFMA_TFLOPS * 1e12), 4), "kernels": per_family}
    if clock_probe:
        res["shader_clock"] = shader_clock_during(fdx, lambda: model.predict_dev(batch, d_in, shapes, d_out), steps, sec * 1e3)
        res["shader_clock"].pop("what")
    model.close()
    for b in d_in + d_out:
        b.free()
    return res


def gpt2_step_bytes(L, batch=16, layers=12, d=768, ffn=3072, vocab=50257):
    """Bytes one decode step must stream at context length L (keys visible incl. the new token)."""
    w_layers = layers * (4 * d * d + 4 * d + 2 * d * ffn + ffn + d + 4 * d) * 4
    w_head = (d * vocab + vocab) * 4
    kv = layers * 2 * L * d * 4 * batch
    logits = batch * vocab * 4
    return w_layers + w_head + kv + logits


def bench_gpt2(fdx, modelgen, args):
    batch, prompt, new = 16, 128, 128
    spec = modelgen.gpt2()
    js = modelgen.dumps(spec)
    del spec
    log_address_map("gpt2_generated")
    t0 = time.perf_counter()
    model = fdx.Model(js, verify=False)
    load_s = time.perf_counter() - t0
    cpu = None
    if not args.no_cpu_baseline:
        cores = host_cores()
        cpu = {"value": round(cpu_baseline_decode(js, cores), 2), "unit": "tok/s", "cores": cores, "kind": "port",
               "what": CPU_KIND_NOTE, "build": CPU_BUILD, "cpu": cpu_model_name(),
               "sample": "%d sequences (one per core, in parallel threads) on the CPU oracle's KV-cached decoder: 4 prompt + 3 "
                         "warm-up steps, then 5 timed greedy steps each" % cores}
    del js
    ids = np.random.default_rng(99).integers(0, 50257, (batch, prompt)).astype(np.float32)
    sess = fdx.Session(model, batch, prompt + new)
    d_ids = fdx.DevBuf.from_host(ids)
    d_first, d_tok, d_log = fdx.DevBuf(4 * batch), fdx.DevBuf(4 * new * batch), fdx.DevBuf(4 * batch * 50257)
    ms = ctypes.c_float()
    best = None
    for rep in range(1 + max(1, args.decode_reps)):  # first repetition is the warm-up
        sess.reset()
        fdx.check(fdx.lib.fdx_timer_start())
        fdx.check(fdx.lib.fdx_session_prefill(sess._h, fdx._dp(d_ids), prompt, None, fdx._dp(d_first)))
        fdx.check(fdx.lib.fdx_timer_stop(ctypes.byref(ms)))
        prefill_ms = ms.value
        fdx.check(fdx.lib.fdx_timer_start())
        fdx.check(fdx.lib.fdx_session_decode_greedy(sess._h, fdx._dp(d_first), new, fdx._dp(d_tok), fdx._dp(d_log)))
        fdx.check(fdx.lib.fdx_timer_stop(ctypes.byref(ms)))
        if rep > 0 and (best is None or ms.value < best[0]):
            best = (ms.value, prefill_ms)
    decode_ms, prefill_ms = best
    tokens = d_tok.to_host((new, batch))
    assert np.isfinite(tokens).all() and tokens.min() >= 0 and tokens.max() < 50257
    total_bytes = sum(gpt2_step_bytes(prompt + 1 + i) for i in range(new))
    achieved = total_bytes / (decode_ms / 1e3) / 1e9
    out = {
        "metric": "GPT-2-small-shape KV-cache greedy decode tok/s (fp32, batch 16, prompt 128 + 128 new)",
        "value": round(batch * new / (decode_ms / 1e3), 1),
        "unit": "tok/s",
        "ms_per_step": round(decode_ms / new, 4),
        "prefill_ms": round(prefill_ms, 3),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4), "bytes_per_step_mean": round(total_bytes / new),
                     "kernel": "skinny_gemm_kernel (Dense for 16 rows, weights streamed once; 48 of the step's 63 launches plus the LM head's striding variant)",
                     "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH["skinny_gemm, GPT-2 decode b16"],
                     "traffic_note": "isolated-kernel run (--workload gpt2_kernels, the step's five Dense shapes against rings of "
                                     "weight copies), not a counter run of the decode loop itself"},
        "load_seconds": round(load_s, 2),
    }
    if not args.no_clock_probe:  # one more generation with the probe beside it
        sess.reset()
        fdx.check(fdx.lib.fdx_session_prefill(sess._h, fdx._dp(d_ids), prompt, None, fdx._dp(d_first)))
        fdx.sync()
        fdx.check(fdx.lib.fdx_clock_probe_start(int(min(65536, decode_ms * 10 * 1.05 + 4)), 100))
        fdx.check(fdx.lib.fdx_session_decode_greedy(sess._h, fdx._dp(d_first), new, fdx._dp(d_tok), fdx._dp(d_log)))
        fdx.sync()
        mean, lo, hi = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
        fdx.check(fdx.lib.fdx_clock_probe_stop(ctypes.c_double(decode_ms), ctypes.byref(mean), ctypes.byref(lo), ctypes.byref(hi)))
        out["shader_clock"] = {"mean_ghz": round(mean.value, 3), "min_ghz": round(lo.value, 3), "max_ghz": round(hi.value, 3)}
    if cpu:
        out["cpu_baseline"] = cpu
    sess.close()
    model.close()
    return out


def bench_gpt2_kernels(fdx, args):
    """The decode step's dominant kernel (the weight-streaming Dense for 16 rows) alone, at the five GEMM shapes of
    a GPT-2-small block, each against a ring of weight copies larger than the caches so every launch streams
    from HBM.  Used for per-kernel roofline figures and counter runs; not part of the headline metric."""
    m, reps = 16, max(4, args.steps)
    shapes = [("qkv (LayerNorm folded)", 768, 2304, True, False), ("attention output + residual", 768, 768, False, True),
              ("mlp fc (LayerNorm folded, gelu)", 768, 3072, True, False), ("mlp proj + residual", 3072, 768, False, True),
              ("lm head (LayerNorm folded)", 768, 50257, True, False)]
    rng = np.random.default_rng(5)
    out = []
    ms = ctypes.c_float()
    for name, k, n, ln, res in shapes:
        copies = max(1, int(args.ring_mb * 1e6 // (4 * k * n)))
        w = fdx.DevBuf(4 * k * n * copies)
        host = (rng.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
        for c in range(copies):
            fdx.check(fdx.lib.fdx_h2d(ctypes.c_void_p(w.ptr.value + 4 * k * n * c), host.ctypes.data_as(ctypes.c_void_p),
                                      ctypes.c_size_t(host.nbytes)))
        x = fdx.DevBuf.from_host(rng.standard_normal((m, k)).astype(np.float32))
        bias = fdx.DevBuf.from_host(rng.standard_normal(n).astype(np.float32))
        rsum = fdx.DevBuf.from_host(host.sum(1).astype(np.float32))
        r = fdx.DevBuf.from_host(rng.standard_normal((m, n)).astype(np.float32)) if res else None
        y = fdx.DevBuf(4 * m * n)
        f32p = ctypes.POINTER(ctypes.c_float)

        def launch(c):
            wp = ctypes.cast(ctypes.c_void_p(w.ptr.value + 4 * k * n * c), f32p)
            if ln:
                fdx.check(fdx.lib.fdx_layernorm_dense_rows_f32(fdx._dp(x), m, k, ctypes.c_float(1e-5), wp, fdx._dp(rsum),
                                                               fdx._dp(bias), n, None, None, fdx._dp(y)))
            else:
                fdx.check(fdx.lib.fdx_dense_rows_f32(fdx._dp(x), m, k, wp, fdx._dp(bias), n, fdx._dp(r), None, fdx._dp(y)))

        for c in range(copies):
            launch(c)
        fdx.sync()
        fdx.check(fdx.lib.fdx_timer_start())
        for i in range(reps * copies):
            launch(i % copies)
        fdx.check(fdx.lib.fdx_timer_stop(ctypes.byref(ms)))
        us = ms.value * 1e3 / (reps * copies)
        nbytes = 4.0 * (k * n + n + m * k + m * n * (2 if res else 1))
        out.append({"shape": name, "rows": m, "k": k, "n": n, "us_per_launch_back_to_back": round(us, 2),
                    "algorithmic_bytes": int(nbytes), "GB_per_s": round(nbytes / us / 1e3, 1),
                    "hbm_frac": round(nbytes / us / 1e3 / PEAK_HBM_GBS, 4)})
        for b in (w, x, bias, rsum, y) + ((r,) if r else ()):
            b.free()
    return {"metric": "decode Dense kernel, 16 rows, weights streamed from HBM", "unit": "us per launch",
            "n_gpus": 1, "kernels": out}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=10,
                    help="untimed passes before the timed ones (the shader clock needs about 30 ms of load to settle after an idle period)")
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--decode-reps", type=int, default=2)
    ap.add_argument("--workload", choices=["all", "resnet50", "gpt2", "gpt2_kernels", "mobilenet_v2", "encoder"], default="all")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-clock-probe", action="store_true", help="skip the shader-clock pass after the timed region")
    ap.add_argument("--tuner-import", default=None, help="per-shape tuner table to load and freeze before anything runs "
                                                         "(fdx_tuner_import + fdx_tuner_freeze: nothing is timed, every run picks the same kernels)")
    ap.add_argument("--tune", action="store_true", help="let the first sight of every shape time its candidate kernels "
                                                        "(fdx_tuner_timing(1)); the default runs on the closed rules, as a "
                                                        "caller who sets nothing does")
    ap.add_argument("--tuner-export", default=None, help="write the per-shape tuner table of this run to this file at the end")
    ap.add_argument("--ring-mb", type=float, default=600.0,
                    help="gpt2_kernels: total size of the ring of weight copies a kernel cycles through (larger than the "
                         "caches by default, so every launch streams from HBM)")
    ap.add_argument("--calibrate-copy-mib", type=int, default=0,
                    help="also launch one plain device copy (act_kernel, no activation) of this many MiB, whose known "
                         "traffic scales the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (samples are independent; more GPUs would each take a "
                 "slice of the batch with their own copy of the weights) -- use --gpus 1")
    log_address_map("start")
    fdx, modelgen = load_package()
    log_address_map("library_loaded")
    if args.tuner_import:
        fdx.tuner_import(open(args.tuner_import).read())
        fdx.tuner_freeze(True)
    if args.tune:
        fdx.tuner_timing(True)
    if args.calibrate_copy_mib > 0:
        n = args.calibrate_copy_mib * (1 << 20) // 4
        src, dst = fdx.DevBuf(4 * n), fdx.DevBuf(4 * n)
        fdx.check(fdx.lib.fdx_activation_f32(fdx._dp(src), ctypes.c_size_t(n), None, fdx._dp(dst)))
        fdx.sync()
        src.free()
        dst.free()
    result = {}
    if args.workload in ("all", "resnet50"):
        result = bench_resnet(fdx, modelgen, args)
    if args.workload == "gpt2_kernels":
        result = bench_gpt2_kernels(fdx, args)
    if args.workload in ("all", "gpt2"):
        g = bench_gpt2(fdx, modelgen, args)
        if result:
            result["gpt2_decode"] = g
        else:
            result = g
    rng = np.random.default_rng(77)
    secondary = {}
    if args.workload in ("all", "mobilenet_v2"):
        x = rng.uniform(0, 1, (128, 224, 224, 3)).astype(np.float32)
        secondary["mobilenet_v2"] = bench_secondary(fdx, modelgen, "MobileNetV2 alpha 1.0 architecture, 224x224x3, batch 128",
                                                    modelgen.mobilenet_v2(), 128, [x], max(3, args.steps), max(3, 3 * args.warmup),
                                                    not args.no_clock_probe)
    if args.workload in ("all", "encoder"):
        x = rng.standard_normal((32, 256, 512)).astype(np.float32)
        secondary["encoder"] = bench_secondary(fdx, modelgen, "6-layer pre-LN transformer encoder, seq 256, d 512, 8 heads, "
                                               "ffn 2048 (erf-GELU), batch 32", modelgen.encoder(), 32, [x],
                                               max(3, args.steps), max(3, 3 * args.warmup // 2), not args.no_clock_probe)
    if secondary:
        if result:
            result["secondary"] = secondary
        else:
            result = {"metric": "secondary configurations", "n_gpus": 1, "secondary": secondary}
    if args.tuner_export:
        with open(args.tuner_export, "w") as f:
            f.write(fdx.tuner_export())
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
