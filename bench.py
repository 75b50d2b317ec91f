"""Benchmark of the forward hot path on one MI355X.

Primary line (BASELINE.json metric, configs[1]): ResNet50-architecture CNN, fp32, batch 64, 224x224x3,
random-init He-normal weights, synthetic uniform[0,1] inputs already resident in HBM.  One step = one
batched predict (fdx_model_predict_dev) of 64 images.  Prints ONE JSON line.
"""
import argparse
import concurrent.futures
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


def load_package():
    import __graft_entry__ as entry
    entry._ensure_built()
    return importlib.import_module("frugally-deep_amd"), importlib.import_module("frugally-deep_amd.modelgen")


def profile_families(fdx):
    import ctypes
    fams = {}
    i = 0
    while True:
        name = ctypes.create_string_buffer(128)
        launches, ms, flops, nbytes = ctypes.c_uint64(), ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
        if fdx.lib.fdx_profile_get(i, name, 128, ctypes.byref(launches), ctypes.byref(ms), ctypes.byref(flops),
                                   ctypes.byref(nbytes)) != 0:
            break
        fams[name.value.decode()] = dict(launches=launches.value, ms=ms.value, flops=flops.value, bytes=nbytes.value)
        i += 1
    return fams


def cpu_baseline_resnet(js, x, cores, passes=2):
    """The oracle (a port of the reference CPU path) timed with one prediction per core in parallel."""
    import fdeep_oracle
    ref = fdeep_oracle.OracleModel(js)
    samples = [x[i % x.shape[0]] for i in range(cores)]
    with concurrent.futures.ThreadPoolExecutor(cores) as pool:
        list(pool.map(lambda s: ref.predict([s]), samples))  # warm-up pass
        t0 = time.perf_counter()
        for _ in range(passes):
            list(pool.map(lambda s: ref.predict([s]), samples))
        dt = time.perf_counter() - t0
    return cores * passes / dt


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (samples are independent; more GPUs would each take a "
                 "slice of the batch with their own copy of the weights) -- use --gpus 1")

    fdx, modelgen = load_package()
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

    for _ in range(args.warmup):
        model.predict_dev(batch, [d_in], shapes, [d_out])
    fdx.sync()
    import ctypes
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
    fdx.check(fdx.lib.fdx_profile_enable(1))
    fdx.check(fdx.lib.fdx_profile_reset())
    for _ in range(max(2, args.steps // 4)):
        model.predict_dev(batch, [d_in], shapes, [d_out])
    fdx.sync()
    fams = profile_families(fdx)
    fdx.check(fdx.lib.fdx_profile_enable(0))
    mfma = {k: v for k, v in fams.items() if v["flops"] > 0}
    mf_flops = sum(v["flops"] for v in mfma.values())
    mf_ms = sum(v["ms"] for v in mfma.values())
    mf_launches = sum(v["launches"] for v in mfma.values())
    achieved = mf_flops / (mf_ms / 1e3) / 1e12 if mf_ms > 0 else 0.0
    total_ms = sum(v["ms"] for v in fams.values())

    result = {
        "metric": "ResNet50-shape img/s (fp32,b64)",
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
            "kernel": "igemm_kernel (implicit-GEMM Conv2D / GEMM, fp32 MFMA, all tile instantiations)",
            "achieved": round(achieved, 3),
            "peak": PEAK_FP32_MFMA_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
            "flops_per_launch": round(mf_flops / max(mf_launches, 1), 1),
            "avg_launch_ms": round(mf_ms / max(mf_launches, 1), 5),
            "share_of_step_time": round(mf_ms / total_ms, 4) if total_ms else None,
            "traffic": None,
        },
        "kernel_ms_per_step": {k: round(v["ms"] / max(2, args.steps // 4), 4) for k, v in sorted(fams.items())},
        "wall_ms_per_step": round(wall_s * 1e3 / args.steps, 4),
        "load_seconds": round(load_s, 2),
    }
    if not args.no_cpu_baseline:
        cores = min(os.cpu_count() or 1, 16)
        cpu = cpu_baseline_resnet(js, x, cores)
        result["cpu_baseline"] = {"value": round(cpu, 3), "unit": "img/s", "cores": cores, "kind": "port",
                                  "sample": "%d ResNet50 predictions per pass (one per core, in parallel threads), "
                                            "1 warm-up + 2 timed passes of the CPU oracle" % cores}
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
