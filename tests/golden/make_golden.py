"""Writes the golden fixtures from the COMPILED REFERENCE runtime (oracle/_ref,
built from /root/reference by oracle/Makefile with -O3 -fsigned-char
-std=c++11 -fopenmp).  The reference ships no fixtures of its own (its tests
read /data/... on the authors' machines), so the expected values are produced
here once and committed as data:

  ops_golden.npz     outputs of cvm.runtime.cpu.<op> for tests/golden/cases.py
  host_golden.json   FInferShape/FInferPrecision results, C-API sizes and gas,
                     output digests of the shrunk model graphs, status codes
                     of malformed models

    python tests/golden/make_golden.py      (only where oracle/_ref exists)
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)
import __graft_entry__  # noqa: E402

__graft_entry__.load_package()
import oracle  # noqa: E402
import oracle.graph as og  # noqa: E402
from cvm_runtime_amd import graphgen, synth  # noqa: E402
import cases  # noqa: E402


def small_models():
    return {
        "cfg1": graphgen.conv_op_graph(1, 16, 12, 12, 8),
        "cfg2": graphgen.resnet20_cifar(2),
        "cfg3": graphgen.resnet50(1, width=16, blocks=(1, 1, 1, 1), size=64, classes=10, config_id="tiny50"),
        "cfg4": graphgen.vgg16(1, size=32, width=8, fc=64, classes=10, config_id="tiny-vgg"),
        "cfg5": graphgen.ssd_mobilenet(size=64, alpha=0.25, config_id="tiny-ssd", neg_ids=True),
    }


def malformed_graphs():
    g, heads = graphgen.conv_op_graph(1, 16, 12, 12, 8)
    js, pb = g.build(heads)
    base = json.loads(js)
    out = {"valid": js}

    def variant(name, fn):
        d = json.loads(js)
        fn(d)
        out[name] = json.dumps(d)
    variant("bad_version", lambda d: d.__setitem__("version", "cvm_9"))
    variant("unknown_key", lambda d: d.__setitem__("extra", 1))
    variant("no_heads", lambda d: d.pop("heads"))
    variant("wrong_shape", lambda d: d["attrs"]["shape"][1].__setitem__(len(d["attrs"]["shape"][1]) - 1, [1, 8, 12, 13]))
    variant("bad_dltype", lambda d: d["attrs"]["dltype"][1].__setitem__(0, "float32"))
    variant("precision_unset", lambda d: d["attrs"]["precision"][1].__setitem__(0, -1))
    variant("wide_input", lambda d: d["attrs"]["precision"][1].__setitem__(0, 9))
    variant("storage_clash", lambda d: d["attrs"]["storage_id"][1].__setitem__(3, d["attrs"]["storage_id"][1][0]))
    variant("unknown_op", lambda d: d["nodes"][3]["attrs"].__setitem__("func_name", "softmax"))
    variant("bad_attr", lambda d: d["attrs"]["op_attrs"][1].__setitem__(3, json.dumps({"channels": "8", "kernel_size": "[3, 3]", "nope": "1"})))
    variant("zero_dim", lambda d: d["attrs"]["shape"][1].__setitem__(0, [1, 16, 0, 12]))
    variant("node_op_kind", lambda d: d["nodes"][3].__setitem__("op", "tvm_op"))
    variant("row_ptr", lambda d: d["node_row_ptr"].__setitem__(2, 7))
    variant("device_index", lambda d: d["attrs"].__setitem__("device_index", ["list_int", [0] * len(d["attrs"]["shape"][1])]))
    out["not_json"] = "{ this is not json"
    del base
    return out


def main():
    assert oracle.have_ref(), "build oracle/_ref first (make -C oracle ref)"
    arrays = {}
    for i, (op, attrs, _) in enumerate(cases.OP_CASES):
        ins = cases.make_inputs(i)
        shapes = [o.shape for o in oracle.run_op(op, attrs, ins)]   # shapes only; values come from the reference
        init = 9 if op == "where" else 7
        outs = [np.full(s, init, np.int32) for s in shapes]
        # cvm.runtime.cpu.cvm_left_shift always throws before computing anything
        # (src/runtime/cpu/ops/elemwise.cc:183 converts a handle argument to
        # std::string); its arithmetic is pinned on the FORMAL registration.
        dev = "formal" if op == "cvm_left_shift" else "cpu"
        rc, msg = oracle.ref_run_op(op, attrs, ins, outs, dev)
        assert rc == 0, (op, msg)
        for j, o in enumerate(outs):
            arrays["op%d_out%d" % (i, j)] = o
    for i in range(len(cases.NMS_CASES)):
        x, vc, attrs = cases.nms_inputs(i)
        rx, y = x.copy(), np.full_like(x, 5)
        rc, msg = oracle.ref_run_op("non_max_suppression", attrs, [rx, vc], [y])
        assert rc == 0, msg
        arrays["nms%d_y" % i] = y
        arrays["nms%d_x_after" % i] = rx
    np.savez_compressed(os.path.join(HERE, "ops_golden.npz"), **arrays)

    host = {"infer": [], "models": {}, "malformed": {}}
    for op, attrs, shapes, precs in cases.INFER_CASES:
        rc, oshapes, oprecs, _ = oracle.ref_infer(op, attrs, shapes, precs)
        host["infer"].append({"status": rc, "shapes": [list(s) for s in oshapes] if rc == 0 else [],
                              "precs": oprecs if rc == 0 else []})
    for name, (g, heads) in small_models().items():
        js, pb = g.build(heads)
        rc, q = og.ref_query(js, pb)
        assert rc == 0
        x = synth.tensor("golden-" + name, "data", g.shape((0, 0)), -127, 127)
        rc, out = og.ref_inference(js, pb, x.astype(np.int8).tobytes())
        assert rc == 0
        host["models"][name] = {"query": q, "output_sha256": hashlib.sha256(out).hexdigest(), "output_head": list(out[:32])}
    L = og.ref_lib()
    import ctypes
    for name, js in malformed_graphs().items():
        v = ctypes.c_ulonglong()
        host["malformed"][name] = L.CVMAPIGetGasFromGraphFile(ctypes.c_char_p(js.encode()), ctypes.byref(v))
    with open(os.path.join(HERE, "host_golden.json"), "w") as f:
        json.dump(host, f, indent=1)
    print("wrote", len(arrays), "arrays,", len(host["infer"]), "infer cases")


if __name__ == "__main__":
    main()
