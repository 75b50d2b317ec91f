"""The C++ facade (include/fdeep/fdeep.hpp) compiled with g++ against libfdx.so.  On the CPU box the
program must compile and link; on the GPU box it runs the reference-style load / predict_multi checks."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "frugally-deep_amd")
EXE = os.path.join(ROOT, "tests", "cpp", "facade_test.bin")


def compile_facade():
    src = os.path.join(ROOT, "tests", "cpp", "facade_test.cpp")
    if os.path.exists(EXE) and os.path.getmtime(EXE) >= max(os.path.getmtime(src), os.path.getmtime(
            os.path.join(ROOT, "include", "fdeep", "fdeep.hpp")), os.path.getmtime(os.path.join(PKG, "libfdx.so"))):
        return
    subprocess.check_call(["g++", "-std=c++14", "-O1", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"), src,
                           "-L", PKG, "-lfdx", "-Wl,-rpath," + PKG, "-Wl,-rpath,/opt/rocm/lib", "-pthread", "-o", EXE])


def test_value_types_follow_the_reference(fdx):
    """tensor / tensor_shape / tensor_shape_variable / tensor_pos members and reshape_tensor_vectors of the facade
    (host code only: the program touches no GPU)."""
    src = os.path.join(ROOT, "tests", "cpp", "value_types_test.cpp")
    exe = os.path.join(ROOT, "tests", "cpp", "value_types_test.bin")
    subprocess.check_call(["g++", "-std=c++14", "-O1", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"), src,
                           "-L", PKG, "-lfdx", "-Wl,-rpath," + PKG, "-Wl,-rpath,/opt/rocm/lib", "-pthread", "-o", exe])
    out = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    print(out.stdout, out.stderr, flush=True)
    assert out.returncode == 0 and "value_types_test ok" in out.stdout


def test_facade_compiles_and_links(fdx):
    compile_facade()
    assert os.path.exists(EXE)


@pytest.mark.gpu
def test_facade_runs_reference_style_checks(fdx, oracle, modelgen, tmp_path):
    print("cpp facade", flush=True)
    if not os.path.exists(EXE):
        compile_facade()
    spec = modelgen.small_cnn()
    ref = oracle.OracleModel(modelgen.dumps(spec))
    x = np.random.default_rng(41).uniform(-1, 1, (32, 32, 3)).astype(np.float32)
    spec["tests"] = [{"inputs": [x], "outputs": [ref.predict([x])[0]]}]
    path = tmp_path / "small_cnn.json"
    path.write_bytes(modelgen.dumps(spec))
    # the program's own non-constant input, classified by the oracle
    idx = np.arange(32 * 32 * 3, dtype=np.float32)
    probe = np.sin(np.float32(0.37) * idx).astype(np.float32).reshape(32, 32, 3)
    want = oracle.argmax(ref.predict([probe])[0])
    # a model with a layer class only a custom creator knows: Dense -> ScaleShift (2x + offset[c]) -> Dense
    b = modelgen.Builder("with_custom", 77)
    t_in = b.input((5, 8), "x")
    h = b.dense(t_in, 6, "fc1", activation="relu", bias_std=0.2)
    b.params["scale_shift"] = {"offset": np.arange(6, dtype=np.float32) / 4}
    c = b._add("ScaleShift", "scale_shift", {"name": "scale_shift"}, [h], h.shape)
    cspec = b.finish([b.dense(c, 3, "fc2", bias_std=0.2)])
    xc = np.random.default_rng(42).standard_normal((5, 8)).astype(np.float32)
    p = cspec["trainable_params"]
    hid = oracle.relu(oracle.dense(xc, p["fc1"]["weights"].reshape(-1), p["fc1"]["bias"], 6))
    hid = (2.0 * hid + p["scale_shift"]["offset"]).astype(np.float32)
    cspec["tests"] = [{"inputs": [xc], "outputs": [oracle.dense(hid, p["fc2"]["weights"].reshape(-1), p["fc2"]["bias"], 3)]}]
    cpath = tmp_path / "with_custom.json"
    cpath.write_bytes(modelgen.dumps(cspec))
    out = subprocess.run([EXE, str(path), str(want), str(cpath)], capture_output=True, text=True, timeout=120)
    print(out.stdout, out.stderr, flush=True)
    assert out.returncode == 0 and "facade_test ok" in out.stdout
