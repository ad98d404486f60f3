"""Writes tests/golden/op_cases/: operator case directories in the layout that
the reference's operator test replays (tests/test_op.cc:479-660; its own tree,
/data/ops_generator, made by python/mrt/ops_generator.py, is not part of the
reference).  Inputs are the seeded tensors of tests/golden/cases.py; expected
outputs, output shapes and the rejections announced in err.txt all come from
the COMPILED REFERENCE runtime (oracle/_ref: FInferShape and
cvm.runtime.cpu.<op>), never from this repository's own code.

    python tests/golden/make_op_cases.py      (only where oracle/_ref exists)
"""
import os
import shutil
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)
import __graft_entry__  # noqa: E402

__graft_entry__.load_package()
import oracle  # noqa: E402
from cvm_runtime_amd import op_cases  # noqa: E402
import cases  # noqa: E402

# shapes that the reference's FInferShape must reject (attributes themselves are well-formed: the
# reference's loop only survives failures of shape inference, not of attribute parsing)
REJECTED = [
    ("conv2d", {"channels": "6", "kernel_size": "[3, 3]", "use_bias": "False"}, [(1, 8, 9, 9), (6, 4, 3, 3)]),
    ("conv2d", {"channels": "6", "kernel_size": "[9, 9]", "use_bias": "False"}, [(1, 8, 5, 5), (6, 8, 9, 9)]),
    ("conv2d", {"channels": "6", "kernel_size": "[3, 3]", "use_bias": "True"}, [(1, 8, 9, 9), (6, 8, 3, 3), (5,)]),
    ("dense", {"units": "4", "use_bias": "False"}, [(2, 9), (4, 8)]),
    ("dense", {"units": "4", "use_bias": "True"}, [(2, 9), (4, 9), (3,)]),
    ("elemwise_add", {}, [(2, 3), (3, 2)]),
    ("broadcast_add", {}, [(2, 3), (4, 2)]),
    ("broadcast_mul", {}, [(5,), (3,)]),
    ("concatenate", {"axis": "1"}, [(3, 1, 4), (3, 2, 5)]),
    ("concatenate", {"axis": "3"}, [(3, 1, 4), (3, 2, 4)]),
    ("max_pool2d", {"pool_size": "[2, 2]", "padding": "(2, 2)"}, [(1, 3, 9, 11)]),
    ("max_pool2d", {"pool_size": "[12, 12]"}, [(1, 3, 9, 11)]),
    ("transpose", {"axes": "(0, 0, 1)"}, [(3, 4, 5)]),
    ("transpose", {"axes": "(0, 1)"}, [(3, 4, 5)]),
    ("reshape", {"shape": "(7, -1)"}, [(3, 4, 5)]),
    ("take", {"axis": "4"}, [(3, 4), (2,)]),
    ("slice_like", {"axis": "(0,)"}, [(3, 4), (5, 4)]),
    ("sum", {"axis": "(3,)"}, [(3, 4)]),
    ("expand_dims", {"axis": "4"}, [(3, 4)]),
    ("squeeze", {"axis": "(0,)"}, [(3, 1, 4)]),
    ("get_valid_counts", {"score_threshold": "0"}, [(3, 4)]),
    ("non_max_suppression", {"iou_threshold": "0"}, [(1, 8, 6), (1,)]),
    ("non_max_suppression", {"iou_threshold": "50"}, [(2, 8, 6), (3,)]),
    ("cvm_lut", {"in_dim": "60"}, [(4, 3), (50,)]),
    ("upsampling", {"scale": "0"}, [(1, 2, 3, 3)]),
    ("repeat", {"repeats": "0"}, [(2, 3)]),
    ("tile", {"reps": "(0, 2)"}, [(2, 3)]),
    ("strided_slice", {"begin": "(0,)", "end": "(2,)", "stride": "(0,)"}, [(3, 4)]),
]


def main():
    assert oracle.have_ref(), "build oracle/_ref first (make -C oracle ref)"
    root = os.path.join(HERE, "op_cases")
    shutil.rmtree(root, ignore_errors=True)
    count = {}

    def case_dir(op):
        count[op] = count.get(op, 0) + 1
        return os.path.join(root, op, "%02d" % (count[op] - 1))

    for i, (op, attrs, _) in enumerate(cases.OP_CASES):
        ins = cases.make_inputs(i)
        rc, shapes, _, msg = oracle.ref_infer(op, attrs, [v.shape for v in ins])
        assert rc == 0, (op, attrs, msg)
        outs = [np.zeros(s, np.int32) for s in shapes]
        # cvm.runtime.cpu.cvm_left_shift throws before computing anything (src/runtime/cpu/ops/elemwise.cc:183);
        # its arithmetic comes from the FORMAL registration
        rc, msg = oracle.ref_run_op(op, attrs, [v.copy() for v in ins], outs, "formal" if op == "cvm_left_shift" else "cpu")
        assert rc == 0, (op, attrs, msg)
        op_cases.write_case(case_dir(op), attrs, ins, outs)
    for i in range(len(cases.NMS_CASES)):
        x, vc, attrs = cases.nms_inputs(i)
        rc, shapes, _, msg = oracle.ref_infer("non_max_suppression", attrs, [x.shape, vc.shape])
        assert rc == 0, msg
        y = np.zeros(shapes[0], np.int32)
        rc, msg = oracle.ref_run_op("non_max_suppression", attrs, [x.copy(), vc], [y])
        assert rc == 0, msg
        op_cases.write_case(case_dir("non_max_suppression"), attrs, [x, vc], [y])
    kept = 0
    for op, attrs, shapes in REJECTED:
        rc, _, _, msg = oracle.ref_infer(op, attrs, shapes)
        if rc == 0:
            print("reference accepts, not written:", op, attrs, shapes)
            continue
        first = (msg.strip().splitlines() or ["rejected"])[0]
        op_cases.write_case(case_dir(op), attrs, [np.zeros(s, np.int32) for s in shapes], [], err=first[-160:] or "rejected")
        kept += 1
    total = sum(count.values())
    size = sum(os.path.getsize(os.path.join(d, f)) for d, _, fs in os.walk(root) for f in fs)
    print("wrote %d cases (%d rejections) for %d operators, %d KiB" % (total, kept, len(count), size // 1024))


if __name__ == "__main__":
    main()
