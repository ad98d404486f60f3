"""TEST INFRASTRUCTURE ONLY: executes a CVM graph node by node on the CPU oracle,
and (where it was built) through the compiled reference's own C API."""
import ctypes
import json
import os

import numpy as np

import oracle


def run_graph(graph_json, params, data, return_all=False):
    """params: dict name -> int32 ndarray; data: int32 ndarray for node `data`.
    Mirrors CvmRuntime::Run (src/runtime/graph_runtime.cc:61-68) with SetInput's
    clamp of `data` to its precision (graph_runtime.cc:378-386)."""
    g = json.loads(graph_json)
    nodes = g["nodes"]
    row = g["node_row_ptr"]
    precs = g["attrs"]["precision"][1]
    op_attrs = g["attrs"]["op_attrs"][1]
    vals = [None] * row[-1]
    for nid, n in enumerate(nodes):
        if n["op"] == "null":
            if n["name"] == "data":
                r = (1 << (precs[row[nid]] - 1)) - 1
                vals[row[nid]] = np.clip(np.asarray(data, np.int32), -r, r).astype(np.int32)
            else:
                vals[row[nid]] = np.asarray(params[n["name"]], np.int32)
            continue
        func = n["attrs"]["func_name"]
        ins = [vals[row[e[0]] + e[1]] for e in n["inputs"]]
        outs = oracle.run_op(func, json.loads(op_attrs[nid]), ins)
        for i, o in enumerate(outs):
            vals[row[nid] + i] = o
    heads = [vals[row[e[0]] + e[1]] for e in g["heads"]]
    return (heads, vals) if return_all else heads


_REFLIB = None


def ref_lib():
    """The compiled reference runtime (only where oracle/_ref was built)."""
    global _REFLIB
    if _REFLIB is None:
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_ref", "libcvm_runtime_ref.so")
        _REFLIB = ctypes.CDLL(path)
    return _REFLIB


def ref_inference(graph_json, param_bytes, input_bytes, device_type=0, fill=0):
    """CVMAPILoadModel + CVMAPIInference of the compiled reference (device 0 = CPU, 2 = FORMAL).
    The output buffer is filled with byte `fill` before the call.  Returns (status, output bytes or None)."""
    L = ref_lib()
    if isinstance(graph_json, str):
        graph_json = graph_json.encode()
    net = ctypes.c_void_p()
    rc = L.CVMAPILoadModel(ctypes.c_char_p(graph_json), len(graph_json), ctypes.c_char_p(param_bytes),
                           len(param_bytes), ctypes.byref(net), device_type, 0)
    if rc != 0:
        return rc, None
    try:
        n = ctypes.c_ulonglong()
        L.CVMAPIGetOutputLength(net, ctypes.byref(n))
        out = ctypes.create_string_buffer(bytes([fill]) * n.value, n.value)
        rc = L.CVMAPIInference(net, ctypes.c_char_p(input_bytes), len(input_bytes), out)
        return rc, (out.raw if rc == 0 else None)
    finally:
        L.CVMAPIFreeModel(net)


def ref_query(graph_json, param_bytes, device_type=0):
    """Sizes and gas reported by the compiled reference for a model."""
    L = ref_lib()
    if isinstance(graph_json, str):
        graph_json = graph_json.encode()
    net = ctypes.c_void_p()
    rc = L.CVMAPILoadModel(ctypes.c_char_p(graph_json), len(graph_json), ctypes.c_char_p(param_bytes),
                           len(param_bytes), ctypes.byref(net), device_type, 0)
    if rc != 0:
        return rc, None
    out = {}
    v = ctypes.c_ulonglong()
    for fn in ("CVMAPIGetInputLength", "CVMAPIGetOutputLength", "CVMAPIGetInputTypeSize", "CVMAPIGetOutputTypeSize",
               "CVMAPIGetStorageSize", "CVMAPIGetGasFromModel"):
        getattr(L, fn)(net, ctypes.byref(v))
        out[fn] = v.value
    L.CVMAPIFreeModel(net)
    return 0, out
