"""The operator plug-in for the reference's own graph runtime (cvm-runtime_amd/integration/hip_device.cc) EXECUTED: every
packed function is looked up in the reference's registry as "cvm.runtime.hip.<op>" and called with the reference's
argument convention (inputs, outputs, NodeAttrs; ext_space from HIPOpExtraSpace) on tensors allocated through the
registered "device_api.hip", for every operator case directory of tests/golden/op_cases (values written by the compiled
reference).  A wrong argument index or attribute field in a wrapper fails here.

The driver (oracle/hip_plugin_driver.cc, test infrastructure) is built by oracle/Makefile where the reference tree is
present, into oracle/_ref/libhip_plugin_driver.so, which links the compiled reference runtime and the product library;
the test is skipped where that object is absent."""
import ctypes
import json
import os

import numpy as np
import pytest

import __graft_entry__

__graft_entry__.load_package()
from cvm_runtime_amd import op_cases  # noqa: E402

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "oracle", "_ref", "libhip_plugin_driver.so")
TREE = os.path.join(ROOT, "tests", "golden", "op_cases")
CASES = [(op, p) for op, p in op_cases.list_cases(TREE)]


class PluginTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.POINTER(ctypes.c_int32)), ("ndim", ctypes.c_int32), ("shape", ctypes.c_int64 * 6)]


def _call(lib, op, attrs, ins, outs, copy_inputs_back=False):
    arrs = [np.ascontiguousarray(a, np.int32) for a in ins] + [np.ascontiguousarray(a, np.int32) for a in outs]
    t = (PluginTensor * len(arrs))()
    for i, a in enumerate(arrs):
        t[i].data = a.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
        t[i].ndim = a.ndim
        for d, s in enumerate(a.shape):
            t[i].shape[d] = s
    err = ctypes.create_string_buffer(2048)
    rc = lib.hip_plugin_op_call(op.encode(), json.dumps(attrs).encode(), len(ins), len(outs), t, 1 if copy_inputs_back else 0,
                                err, len(err))
    return rc, err.value.decode(errors="replace"), arrs[:len(ins)], arrs[len(ins):]


@pytest.fixture(scope="module")
def driver(dev):
    if not os.path.exists(DRIVER):
        pytest.skip("oracle/_ref/libhip_plugin_driver.so not built (needs the reference tree: make -C oracle plugin)")
    return ctypes.CDLL(DRIVER, mode=ctypes.RTLD_GLOBAL)


def test_every_operator_case_through_the_reference_registry(driver):
    ran, bad, ops = 0, [], set()
    for op, path in CASES:
        c = op_cases.read_case(path)
        if c["err"]:
            continue   # rejected by shape inference: there is nothing to execute
        outs0 = [np.zeros(o.shape, np.int32) for o in c["outs"]]
        rc, msg, _, outs = _call(driver, op, c["attrs"], c["ins"], outs0)
        ran += 1
        ops.add(op)
        if rc != 0:
            bad.append((op, os.path.basename(path), "status %d: %s" % (rc, msg[:200])))
            continue
        for i, (o, want) in enumerate(zip(outs, c["outs"])):
            if not np.array_equal(o, want):
                diff = np.flatnonzero(o.ravel() != want.ravel())
                bad.append((op, os.path.basename(path), "output %d: %d of %d values differ, first at %d: got %d, expected %d" % (
                    i, diff.size, want.size, diff[0], o.ravel()[diff[0]], want.ravel()[diff[0]])))
    assert not bad, bad
    assert ran >= 100 and len(ops) >= 30, (ran, sorted(ops))


def test_non_max_suppression_also_rewrites_its_input_like_the_reference(driver):
    """nms.cc:93-103 overwrites the rows past top_k in the INPUT with -1; the plug-in must leave the same bytes there."""
    import oracle
    rng = np.random.default_rng(5)
    n = 40
    x = np.zeros((1, n, 6), np.int32)
    x[0, :, 0] = rng.integers(0, 3, n)
    x[0, :, 1] = rng.permutation(n) + 10
    x[0, :, 2:4] = rng.integers(0, 200, (n, 2))
    x[0, :, 4:6] = x[0, :, 2:4] + rng.integers(1, 120, (n, 2))
    vc = np.array([n], np.int32)
    attrs = {"iou_threshold": "40", "force_suppress": "False", "top_k": "12", "max_output_size": "-1", "coord_start": "2",
             "score_index": "1", "id_index": "0", "return_indices": "False", "invalid_to_bottom": "True"}
    want_y, want_x = oracle.non_max_suppression(x, vc, 40, False, 12, max_output_size=-1, y_init=np.zeros_like(x))
    rc, msg, ins, outs = _call(driver, "non_max_suppression", attrs, [x.copy(), vc], [np.zeros_like(x)], copy_inputs_back=True)
    assert rc == 0, msg
    assert np.array_equal(outs[0], want_y)
    assert np.array_equal(ins[0], want_x)


def test_errors_keep_the_reference_classes(driver):
    """A wrapper that the library refuses with an argument error surfaces as the reference's logic error (status 1):
    conv2d without the scratch its FOpExtraSpace must provide cannot happen through the driver, so an operator that
    does not exist stands for the runtime class (status 2)."""
    rc, msg, _, _ = _call(driver, "relu", {}, [np.arange(8, dtype=np.int32) - 4], [np.zeros(8, np.int32)])
    assert rc == 0, msg
    err = ctypes.create_string_buffer(256)
    t = (PluginTensor * 1)()
    rc = driver.hip_plugin_op_call(b"no_such_operator", b"{}", 0, 0, t, 0, err, len(err))
    assert rc != 0
