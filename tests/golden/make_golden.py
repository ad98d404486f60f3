"""Writes the golden fixtures from the COMPILED REFERENCE runtime (oracle/_ref,
built from /root/reference by oracle/Makefile with -O3 -fsigned-char
-std=c++11 -fopenmp).  The reference ships no fixtures of its own (its tests
read /data/... on the authors' machines), so the expected values are produced
here once and committed as data:

  ops_golden.npz     outputs of cvm.runtime.cpu.<op> for tests/golden/cases.py
  host_golden.json   FInferShape/FInferPrecision results, C-API sizes and gas,
                     output digests of the shrunk model graphs, output bytes and
                     status of the post-processing models (argmax, detection,
                     several heads, graph version cvm_1.1.0), status codes of
                     malformed models

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


def _two_heads(cid, narrow, second_stride=1):
    """data -> conv -> two convolution heads, each transposed and reshaped to (1, rows, channels)."""
    g = graphgen.GraphBuilder(cid)
    x = g.var("data", (1, 3, 8, 8), 8)
    f = g.conv_relu_q(x, 8, 3, 1, 1)
    heads = []
    for oc, stride in ((4, 1), (2, second_stride)):
        c, fan_in = g.conv(f, oc, 3, stride, 1)
        if narrow:
            c = g.rshift(c, graphgen.shift_for(fan_in))
        n, ch, h, w = g.shape(c)
        heads.append(g.reshape(g.transpose(c, (0, 2, 3, 1)), (1, h * w, ch)))
    return g, heads


def postprocess_models():
    """Models that exercise CVMModel::SaveTensor / GetOutputLength (src/core/model.cc:181-331) beyond the plain
    copy: name -> (builder, heads, postprocess, version).  Graph version cvm_1.1.0 recomputes arg_nodes and
    node_row_ptr instead of verifying them (graph_runtime.cc:218-250); the keys stay in the JSON, because the
    compiled reference reads node_row_ptr before that point and crashes on a graph without it."""
    out = {}
    g, h = _two_heads("post-det32", narrow=False)
    out["detection_int32"] = (g, h, "detection", "cvm_1.0.0")          # rows of both heads side by side, int32
    g, h = _two_heads("post-two8", narrow=True)
    out["two_heads_int8"] = (g, h, None, "cvm_1.0.0")                  # outputs.size() > 1 without the tag, int8
    g, h = _two_heads("post-det8", narrow=True)
    out["detection_narrow_heads"] = (g, h, "detection", "cvm_1.0.0")   # the tag forces 4-byte outputs
    g, h = _two_heads("post-rows", narrow=False, second_stride=2)
    out["detection_rows_differ"] = (g, h, "detection", "cvm_1.0.0")    # 64 rows against 16: cannot concat
    g, h = graphgen.resnet20_cifar(4)
    out["argmax_batch4"] = (g, h, "argmax", "cvm_1.0.0")
    g, h = graphgen.conv_op_graph(1, 16, 12, 12, 8)
    out["version_1_1_0"] = (g, h, None, "cvm_1.1.0")
    return out


def stale_bookkeeping(js):
    """The same graph with an arg_nodes list that names only the first variable and a dltype that is not
    int32: version cvm_1.0.0 verifies both and rejects the graph, cvm_1.1.0 recomputes the one and never
    reads the other (graph_runtime.cc:218-250)."""
    d = json.loads(js)
    d["arg_nodes"] = d["arg_nodes"][:1]
    d["attrs"]["dltype"][1][0] = "float32"
    return json.dumps(d)


def build_postprocess_model(name):
    g, heads, post, version = postprocess_models()[name]
    js, pb = g.build(heads, postprocess=post, version=version)
    if version == "cvm_1.1.0":
        js = stale_bookkeeping(js)
    x = synth.tensor("golden-" + name, "data", g.shape((0, 0)), -127, 127)
    return js, pb, x


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
    # what cvm_1.1.0 tolerates (see stale_bookkeeping) is an error at cvm_1.0.0
    out["stale_bookkeeping_1_0_0"] = stale_bookkeeping(js)
    out["stale_bookkeeping_1_1_0"] = stale_bookkeeping(js).replace("cvm_1.0.0", "cvm_1.1.0")
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
    host["postprocess"] = {}
    for name in postprocess_models():
        js, pb, x = build_postprocess_model(name)
        rc, q = og.ref_query(js, pb)
        assert rc == 0, name
        # the output buffer starts as 0x5A bytes, so bytes the reference leaves unwritten show as 90
        rc, out = og.ref_inference(js, pb, x.astype(np.int8).tobytes(), fill=0x5A)
        host["postprocess"][name] = {"query": q, "status": rc, "output_hex": out.hex() if rc == 0 else ""}
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
