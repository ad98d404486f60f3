"""ctypes binding of the model-level C ABI (include/cvm_c_api.h).

Function names and argument meaning follow the reference's own ctypes shim
(python/cvm/_ctypes/runtime.py:12-159), so code written against it runs on
this backend by swapping the import.  `HipModel` adds the staged calls of
include/cvm_hip_ext.h used for measurement.
"""
import ctypes
import json

from . import lib

SUCCEED, ERROR_LOGIC, ERROR_RUNTIME = 0, 1, 2
DEVICE_HIP = 3


class CVMError(RuntimeError):
    def __init__(self, status, what):
        super().__init__("%s failed with status %d (%s)" % (
            what, status, {1: "ERROR_LOGIC", 2: "ERROR_RUNTIME"}.get(status, "?")))
        self.status = status


def _ck(status, what):
    if status != SUCCEED:
        raise CVMError(status, what)


def CVMAPILoadModel(json_str, param_bytes, device_type=DEVICE_HIP, device_id=0):
    if isinstance(json_str, str):
        json_str = json_str.encode()
    net = ctypes.c_void_p()
    _ck(lib().CVMAPILoadModel(ctypes.c_char_p(json_str), ctypes.c_int(len(json_str)),
                              ctypes.c_char_p(param_bytes), ctypes.c_int(len(param_bytes)),
                              ctypes.byref(net), ctypes.c_int(device_type), ctypes.c_int(device_id)),
        "CVMAPILoadModel")
    return net


def CVMAPIFreeModel(net):
    _ck(lib().CVMAPIFreeModel(net), "CVMAPIFreeModel")


def _size(fn, net):
    v = ctypes.c_ulonglong()
    _ck(getattr(lib(), fn)(net, ctypes.byref(v)), fn)
    return v.value


def CVMAPIGetInputLength(net):
    return _size("CVMAPIGetInputLength", net)


def CVMAPIGetOutputLength(net):
    return _size("CVMAPIGetOutputLength", net)


def CVMAPIGetInputTypeSize(net):
    return _size("CVMAPIGetInputTypeSize", net)


def CVMAPIGetOutputTypeSize(net):
    return _size("CVMAPIGetOutputTypeSize", net)


def CVMAPIGetStorageSize(net):
    return _size("CVMAPIGetStorageSize", net)


def CVMAPIGetGasFromModel(net):
    return _size("CVMAPIGetGasFromModel", net)


def CVMAPIGetGasFromGraphFile(json_str):
    if isinstance(json_str, str):
        json_str = json_str.encode()
    v = ctypes.c_ulonglong()
    _ck(lib().CVMAPIGetGasFromGraphFile(ctypes.c_char_p(json_str), ctypes.byref(v)), "CVMAPIGetGasFromGraphFile")
    return v.value


def CVMAPIGetVersion(net):
    buf = ctypes.create_string_buffer(64)
    _ck(lib().CVMAPIGetVersion(net, buf), "CVMAPIGetVersion")
    return buf.value.decode()


def CVMAPIGetPreprocessMethod(net):
    buf = ctypes.create_string_buffer(64)
    _ck(lib().CVMAPIGetPreprocessMethod(net, buf), "CVMAPIGetPreprocessMethod")
    return buf.value.decode()


def CVMAPIInference(net, input_data):
    out = ctypes.create_string_buffer(CVMAPIGetOutputLength(net))
    _ck(lib().CVMAPIInference(net, ctypes.c_char_p(input_data), ctypes.c_int(len(input_data)), out), "CVMAPIInference")
    return out.raw


class HipModel:
    """A loaded model plus the staged / timed calls of the backend's extension ABI."""

    def __init__(self, json_str, param_bytes, device_type=DEVICE_HIP, device_id=0):
        self.net = CVMAPILoadModel(json_str, param_bytes, device_type, device_id)
        self.input_length = CVMAPIGetInputLength(self.net)
        self.output_length = CVMAPIGetOutputLength(self.net)

    def close(self):
        if self.net is not None:
            CVMAPIFreeModel(self.net)
            self.net = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def inference(self, input_data):
        return CVMAPIInference(self.net, input_data)

    def set_input(self, input_data):
        _ck(lib().CVMHIPSetInput(self.net, ctypes.c_char_p(input_data), ctypes.c_int(len(input_data))), "CVMHIPSetInput")

    def run(self):
        _ck(lib().CVMHIPRun(self.net), "CVMHIPRun")

    def get_output(self):
        out = ctypes.create_string_buffer(self.output_length)
        _ck(lib().CVMHIPGetOutput(self.net, out), "CVMHIPGetOutput")
        return out.raw

    def time_run(self, iterations):
        """Device milliseconds for `iterations` runs on the input already staged."""
        ms = ctypes.c_float()
        _ck(lib().CVMHIPTimeRun(self.net, ctypes.c_int(iterations), ctypes.byref(ms)), "CVMHIPTimeRun")
        return ms.value

    def launch_counts(self):
        """(kernel launches per run, layer-sequence launches among them, convolutions inside those)"""
        a, b, c = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        _ck(lib().CVMHIPLaunchCounts(self.net, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)), "CVMHIPLaunchCounts")
        return a.value, b.value, c.value

    def sequence_configs(self):
        """Tile-kernel configuration of every convolution inside the model's layer-sequence launches."""
        n = ctypes.c_int()
        _ck(lib().CVMHIPSequenceConfigs(self.net, None, ctypes.c_int(0), ctypes.byref(n)), "CVMHIPSequenceConfigs")
        buf = (ctypes.c_int * max(n.value, 1))()
        _ck(lib().CVMHIPSequenceConfigs(self.net, buf, ctypes.c_int(n.value), ctypes.byref(n)), "CVMHIPSequenceConfigs")
        return list(buf[:n.value])

    def profile_ops(self):
        buf = ctypes.create_string_buffer(1 << 16)
        _ck(lib().CVMHIPProfileOps(self.net, buf, ctypes.c_int(len(buf))), "CVMHIPProfileOps")
        return json.loads(buf.value.decode())


def infer_node(op, attrs, in_shapes, in_precs):
    """Shape and precision inference for one node on the host (no GPU needed).
    Returns (status, out_shapes, out_precs, message)."""
    n = len(in_shapes)
    shp = (ctypes.c_longlong * (6 * max(n, 1)))()
    nd = (ctypes.c_int * max(n, 1))()
    pr = (ctypes.c_int * max(n, 1))(*in_precs)
    for i, s in enumerate(in_shapes):
        nd[i] = len(s)
        for d, v in enumerate(s):
            shp[6 * i + d] = v
    oshp = (ctypes.c_longlong * 24)()
    ond = (ctypes.c_int * 4)()
    opr = (ctypes.c_int * 4)()
    nout = ctypes.c_int()
    err = ctypes.create_string_buffer(4096)
    rc = lib().CVMHIPInferNode(op.encode(), json.dumps(attrs).encode(), n, shp, nd, pr, ctypes.byref(nout),
                               oshp, ond, opr, err, 4096)
    shapes = [tuple(oshp[6 * i + d] for d in range(ond[i])) for i in range(nout.value)] if rc == 0 else []
    precs = [opr[i] for i in range(nout.value)] if rc == 0 else []
    return rc, shapes, precs, err.value.decode(errors="replace")


def list_ops():
    buf = ctypes.create_string_buffer(1 << 14)
    _ck(lib().CVMHIPListOps(buf, len(buf)), "CVMHIPListOps")
    return buf.value.decode().split()


def run_op(op, attrs, inputs, out_init=0, execute=True):
    """One registered operator on host arrays (CVMHIPRunOp): what the reference's
    tests/test_op.cc does per case.  Outputs start filled with `out_init`.
    Returns (status, failed_stage, outputs, message); with execute=False only
    attribute parsing and shape inference run (no GPU) and outputs are empty
    arrays of the inferred shapes."""
    import numpy as np
    L = lib()
    ins = [np.ascontiguousarray(v, dtype=np.int32) for v in inputs]
    n = len(ins)
    shp = (ctypes.c_longlong * (6 * max(n, 1)))()
    nd = (ctypes.c_int * max(n, 1))()
    ptrs = (ctypes.POINTER(ctypes.c_int) * max(n, 1))()
    for i, v in enumerate(ins):
        nd[i] = v.ndim
        for d, s in enumerate(v.shape):
            shp[6 * i + d] = s
        ptrs[i] = v.ctypes.data_as(ctypes.POINTER(ctypes.c_int))
    max_out = 4
    oshp = (ctypes.c_longlong * (6 * max_out))()
    ond = (ctypes.c_int * max_out)()
    nout = ctypes.c_int()
    stage = ctypes.c_int(-1)
    err = ctypes.create_string_buffer(4096)
    aj = json.dumps(attrs).encode()
    rc = L.CVMHIPRunOp(op.encode(), aj, n, shp, nd, ptrs, max_out, ctypes.byref(nout), oshp, ond, None, None,
                       ctypes.byref(stage), err, 4096)
    if rc != 0:
        return rc, stage.value, [], err.value.decode(errors="replace")
    shapes = [tuple(oshp[6 * i + d] for d in range(ond[i])) for i in range(nout.value)]
    outs = [np.full(s, out_init, np.int32) for s in shapes]
    if not execute:
        return 0, -1, outs, ""
    optrs = (ctypes.POINTER(ctypes.c_int) * max_out)()
    cap = (ctypes.c_longlong * max_out)()
    for i, o in enumerate(outs):
        optrs[i] = o.ctypes.data_as(ctypes.POINTER(ctypes.c_int))
        cap[i] = o.size
    rc = L.CVMHIPRunOp(op.encode(), aj, n, shp, nd, ptrs, max_out, ctypes.byref(nout), oshp, ond, optrs, cap,
                       ctypes.byref(stage), err, 4096)
    return rc, (stage.value if rc else -1), outs, err.value.decode(errors="replace")
