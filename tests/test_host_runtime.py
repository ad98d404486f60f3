"""CPU-only tests of the host logic behind the C ABI: the library loads and
exports every declared symbol, per-node shape/precision inference and graph
verification give the statuses and values the compiled reference gave
(tests/golden/host_golden.json), the parameter blob round-trips."""
import ctypes
import json
import os
import re
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import cases  # noqa: E402
import make_golden  # noqa: E402

import cvm_runtime_amd
from cvm_runtime_amd import graphgen, runtime, synth

ROOT = os.path.dirname(HERE)
GOLD = json.load(open(os.path.join(HERE, "golden", "host_golden.json")))


def test_library_exports_every_declared_symbol():
    lib = cvm_runtime_amd.lib()
    declared = set()
    for h in ("cvm_hip_ops.h", "cvm_c_api.h", "cvm_hip_ext.h"):
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        declared |= set(re.findall(r"\b(cvmhip_\w+|CVMAPI\w+|CVMHIP\w+)\s*\(", text))
    assert len(declared) > 60
    missing = [s for s in sorted(declared) if not hasattr(lib, s)]
    assert not missing, missing


def test_op_registry_lists_every_reference_cpu_operator():
    names = runtime.list_ops()
    ref_cpu_ops = ["relu", "dense", "conv2d", "max_pool2d", "cvm_precision", "abs", "concatenate", "repeat", "negative",
                   "tile", "expand_dims", "squeeze", "transpose", "strided_slice", "slice_like", "take", "cvm_lut",
                   "upsampling", "get_valid_counts", "non_max_suppression", "where", "elemwise_add", "elemwise_sub",
                   "clip", "flatten", "reshape", "cvm_clip", "cvm_right_shift", "cvm_left_shift", "broadcast_add",
                   "broadcast_sub", "broadcast_mul", "broadcast_max", "broadcast_div", "broadcast_greater", "sum", "max"]
    for op in ref_cpu_ops:
        assert "cvm.runtime.hip." + op in names


@pytest.mark.parametrize("index", range(len(cases.INFER_CASES)))
def test_node_inference_matches_reference(index):
    op, attrs, shapes, precs = cases.INFER_CASES[index]
    want = GOLD["infer"][index]
    rc, oshapes, oprecs, msg = runtime.infer_node(op, attrs, shapes, precs)
    assert rc == want["status"], (op, attrs, msg)
    if rc == 0:
        assert [list(s) for s in oshapes] == want["shapes"]
        assert oprecs == want["precs"]


def test_graph_file_verification_statuses_match_reference(capfd):
    for name, js in make_golden.malformed_graphs().items():
        v = ctypes.c_ulonglong()
        rc = cvm_runtime_amd.lib().CVMAPIGetGasFromGraphFile(ctypes.c_char_p(js.encode()), ctypes.byref(v))
        assert rc == GOLD["malformed"][name], name
    capfd.readouterr()


@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg3", "cfg4", "cfg5"])
def test_gas_of_generated_models_matches_reference(name, capfd):
    g, heads = make_golden.small_models()[name]
    js, _ = g.build(heads)
    assert runtime.CVMAPIGetGasFromGraphFile(js) == GOLD["models"][name]["query"]["CVMAPIGetGasFromModel"]
    capfd.readouterr()


def test_param_blob_round_trip_and_layout():
    a = synth.tensor("blob", "a", (3, 4), -127, 127).astype(np.int8)
    b = synth.tensor("blob", "b", (5,), -70000, 70000)
    blob = graphgen.save_params([("alpha", a), ("beta", b)])
    assert blob[:8] == (0xF7E58D4F05049CB7).to_bytes(8, "little")
    back = graphgen.load_params(blob)
    assert np.array_equal(back["alpha"], a) and np.array_equal(back["beta"], b)


def test_null_arguments_are_runtime_errors(capfd):
    lib = cvm_runtime_amd.lib()
    assert lib.CVMAPIInference(None, None, 0, None) == 2
    assert lib.CVMAPIGetInputLength(None, None) == 2
    net = ctypes.c_void_p()
    assert lib.CVMAPILoadModel(b"{}", 2, b"x", 1, ctypes.byref(net), 7, 0) == 2     # unknown device type
    assert lib.CVMAPILoadModel(b"{}", 2, b"x", 1, ctypes.byref(net), 0, 0) == 2     # CPU backend not in this library
    capfd.readouterr()


def test_without_a_gpu_loading_a_model_fails_loudly(capfd):
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    g, heads = graphgen.conv_op_graph(1, 16, 12, 12, 8)
    js, pb = g.build(heads)
    with pytest.raises(runtime.CVMError):
        runtime.HipModel(js, pb)
    capfd.readouterr()
