"""Operator case directories in the reference's own replay layout
(tests/test_op.cc:479-660).  The committed tree tests/golden/op_cases was written
from the compiled reference by tests/golden/make_op_cases.py; here it is replayed
(1) without a GPU up to shape inference, (2) against the oracle, (3) on the GPU."""
import os

import numpy as np
import pytest

import __graft_entry__

__graft_entry__.load_package()
import oracle  # noqa: E402
from cvm_runtime_amd import op_cases, runtime  # noqa: E402

TREE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "op_cases")
CASES = op_cases.list_cases(TREE)
IDS = ["%s-%s" % (op, os.path.basename(p)) for op, p in CASES]


def test_tensor_file_round_trip(tmp_path):
    for a in (np.arange(-6, 6, dtype=np.int32).reshape(2, 3, 2), np.array([2 ** 31 - 1, -2 ** 31], np.int32),
              np.zeros((3, 0, 2), np.int32), np.array(7, np.int32)):
        p = str(tmp_path / "t.txt")
        op_cases.write_tensor(p, a)
        b = op_cases.read_tensor(p)
        assert b.shape == a.shape and b.dtype == np.int32 and np.array_equal(a, b)
    # the reader takes any whitespace, as fscanf("%d ") does
    p = str(tmp_path / "u.txt")
    with open(p, "w") as f:
        f.write("2 2 3 1 2 3\n4 5\t6")
    assert np.array_equal(op_cases.read_tensor(p), np.arange(1, 7).reshape(2, 3))
    with open(p, "w") as f:
        f.write("1 4 1 2 3")
    with pytest.raises(ValueError):
        op_cases.read_tensor(p)


def test_case_directory_round_trip(tmp_path):
    d = str(tmp_path / "relu" / "00")
    op_cases.write_case(d, {"k": "v"}, [np.ones((2, 2), np.int32)], [np.zeros((2, 2), np.int32)])
    c = op_cases.read_case(d)
    assert c["attrs"] == {"k": "v"} and len(c["ins"]) == 1 and len(c["outs"]) == 1 and c["err"] == ""
    op_cases.write_case(d + "e", {}, [np.ones((2,), np.int32)], [], err="bad shape")
    assert op_cases.read_case(d + "e")["err"] == "bad shape"
    assert op_cases.list_cases(str(tmp_path)) == [("relu", d), ("relu", d + "e")]


def test_tree_is_complete():
    ops = {op for op, _ in CASES}
    registered = {n.split(".")[-1] for n in runtime.list_ops()}
    assert len(CASES) >= 130
    assert ops <= registered, ops - registered
    # every operator the reference's own main() replays (tests/test_op.cc:663-691) has cases here
    for op in ("max_pool2d", "upsampling", "dense", "conv2d", "sum", "max", "slice_like", "tile", "repeat", "get_valid_counts",
               "strided_slice", "concatenate", "transpose", "take", "elemwise_add", "non_max_suppression", "broadcast_sub",
               "broadcast_add", "broadcast_mul", "broadcast_max", "broadcast_div", "broadcast_greater"):
        assert op in ops, op
    assert sum(1 for _, p in CASES if op_cases.read_case(p)["err"]) >= 20


@pytest.mark.parametrize("index", range(len(CASES)), ids=IDS)
def test_shapes_and_rejections_without_gpu(index):
    op, path = CASES[index]
    ok, detail = op_cases.replay_case(op, path, execute=False)
    assert ok, detail


@pytest.mark.parametrize("index", range(len(CASES)), ids=IDS)
def test_oracle_reproduces_case(index):
    op, path = CASES[index]
    c = op_cases.read_case(path)
    if c["err"]:
        pytest.skip("rejected by shape inference")
    if op == "non_max_suppression":
        a = c["attrs"]
        y, _ = oracle.non_max_suppression(c["ins"][0], c["ins"][1], int(a["iou_threshold"]), a["force_suppress"] == "True",
                                          int(a["top_k"]), max_output_size=int(a["max_output_size"]),
                                          y_init=np.zeros_like(c["ins"][0]))
        outs = [y]
    else:
        init = np.zeros(c["outs"][0].shape, np.int32) if op == "where" else None
        outs = oracle.run_op(op, c["attrs"], c["ins"], init)
    assert len(outs) == len(c["outs"])
    for o, want in zip(outs, c["outs"]):
        assert o.shape == want.shape and np.array_equal(o, want)


@pytest.mark.gpu
def test_replay_tree_on_gpu():
    lines = []
    res = op_cases.replay_tree(TREE, log=lines.append)
    bad = [(op, os.path.basename(p), d) for op, p, ok, d in res if not ok]
    assert len(res) == len(CASES) and not bad, bad
