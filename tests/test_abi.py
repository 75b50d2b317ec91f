"""The C-ABI library loads without a GPU and exports every entry point include/fdx.h and include/fdx_debug.h declare."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(headers=("fdx.h", "fdx_debug.h")):
    text = "".join(open(os.path.join(ROOT, "include", h)).read() for h in headers)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    # function declarations only: "fdx_status (*callback)(...)" members and typedefs are not exported symbols
    return sorted(set(re.findall(r"\b(fdx_[a-z0-9_]+)\s*\((?!\*)", text)))


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for must in ("fdx_conv2d_nhwc_f32", "fdx_dwconv2d_nhwc_f32", "fdx_gemm_bias_act_f32", "fdx_mha_prefill_f32",
                 "fdx_mha_decode_f32", "fdx_layernorm_f32", "fdx_softmax_f32", "fdx_pool2d_nhwc_f32", "fdx_eltwise_add_f32",
                 "fdx_embedding_f32", "fdx_argmax_f32", "fdx_model_create", "fdx_model_predict", "fdx_session_create",
                 "fdx_session_decode_step", "fdx_last_error"):
        assert must in names
    # the boundary header holds no measurement aids or test hooks: those live in fdx_debug.h
    boundary = declared_symbols(("fdx.h",))
    assert not [n for n in boundary if n.startswith(("fdx_debug_", "fdx_profile_", "fdx_timer_", "fdx_clock_probe_"))]


def test_library_exports_every_declared_symbol(fdx):
    missing = [n for n in declared_symbols() if not hasattr(fdx.lib, n)]
    assert not missing, missing


def test_host_only_entry_points_work_without_a_gpu(fdx, oracle):
    # window geometry is host arithmetic: it must agree with the oracle everywhere
    for n in range(1, 12):
        for k in range(1, 6):
            for s in range(1, 4):
                for padding in ("same", "valid", "causal"):
                    if padding == "valid" and n < k:
                        continue
                    assert fdx.window_geometry(n, n + 2, k, k, s, s, padding) == oracle.window_geometry(n, n + 2, k, k, s, s, padding)
    with pytest.raises(fdx.FdxError):
        fdx.window_geometry(4, 4, 3, 3, 0, 1, "same")


def test_loader_rejects_bad_files_without_touching_the_gpu_path(fdx):
    # argument validation happens before any device work
    h = ctypes.c_void_p()
    assert fdx.lib.fdx_model_create(None, 0, 0, ctypes.c_float(0), ctypes.byref(h)) != 0
    assert b"null" in fdx.lib.fdx_last_error()


def test_modelgen_flops_and_format(modelgen, oracle):
    spec = modelgen.resnet50()
    assert modelgen.model_flops(spec) == 7_715_946_496  # 3.858 GMAC per 224x224 image, x2
    small = modelgen.small_cnn()
    js = modelgen.dumps(small)
    import json
    back = json.loads(js)
    assert back["image_data_format"] == "channels_last" and back["input_shapes"] == [[32, 32, 3]]
    w = oracle.decode_floats(back["trainable_params"]["conv1"]["weights"])
    assert np.array_equal(w, small["trainable_params"]["conv1"]["weights"].reshape(-1))
    assert all(len(c) <= 1024 for c in back["trainable_params"]["fc"]["weights"])
    # vectorised chunk writer == plain one
    arr = np.arange(1000, dtype=np.float32)
    assert json.loads(modelgen._encode_floats_json(arr)) == modelgen.encode_floats(arr)
    for n in (0, 1, 191, 192, 193, 384):
        a = np.arange(n, dtype=np.float32)
        assert json.loads(modelgen._encode_floats_json(a)) == modelgen.encode_floats(a)


def test_model_check_runs_without_a_gpu(fdx, modelgen):
    """fdx_model_check is the loader's host half: a good file passes and a defective one comes back with the loader's own
    message, on a machine with no GPU."""
    fdx.model_check(modelgen.dumps(modelgen.small_cnn()))
    fdx.model_check(modelgen.dumps(modelgen.gpt2(layers=1, d_model=16, heads=2, vocab=50, max_pos=16)))
    with pytest.raises(fdx.FdxError, match="channels_last"):
        fdx.model_check(b'{"image_data_format": "channels_first"}')
    with pytest.raises(fdx.FdxError):
        fdx.model_check(b'{"image_data_format": "channels_last", "architecture": {')
