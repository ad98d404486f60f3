"""Operator cases shared by the golden generator and the tests.

Each case: (op, attrs, [input specs]) with an input spec (shape, lo, hi).
Inputs are regenerated from named splitmix64 streams, so a fixture only needs
to hold the expected outputs."""
import numpy as np

from cvm_runtime_amd import synth

OP_CASES = [
    ("conv2d", {"channels": "6", "kernel_size": "[3, 3]", "strides": "(2, 1)", "padding": "(1, 2)", "use_bias": "True"},
     [((2, 8, 9, 11), -127, 127), ((6, 8, 3, 3), -127, 127), ((6,), -30000, 30000)]),
    ("conv2d", {"channels": "6", "kernel_size": "[3, 3]", "dilation": "(2, 2)", "padding": "(1, 1)", "use_bias": "False"},
     [((2, 8, 9, 11), -127, 127), ((6, 8, 3, 3), -127, 127)]),
    ("conv2d", {"channels": "6", "kernel_size": "[3, 3]", "use_bias": "False"},      # operands wider than int8 are truncated
     [((2, 8, 9, 11), -1000, 1000), ((6, 8, 3, 3), -300, 300)]),
    ("conv2d", {"channels": "8", "kernel_size": "[3, 3]", "groups": "4", "use_bias": "True", "padding": "(1, 1)"},
     [((2, 8, 9, 11), -40000, 40000), ((8, 2, 3, 3), -40000, 40000), ((8,), -99, 99)]),
    ("conv2d", {"channels": "16", "kernel_size": "[3, 3]", "groups": "16", "use_bias": "False", "padding": "(1, 1)", "strides": "(2, 2)"},
     [((1, 16, 10, 10), -127, 127), ((16, 1, 3, 3), -127, 127)]),
    ("conv2d", {"channels": "4", "kernel_size": "[7, 7]", "strides": "(2, 2)", "padding": "(3, 3)", "use_bias": "True"},
     [((1, 3, 20, 20), -127, 127), ((4, 3, 7, 7), -127, 127), ((4,), -32768, 32768)]),
    ("dense", {"units": "5", "use_bias": "True"}, [((3, 17), -127, 127), ((5, 17), -127, 127), ((5,), -99, 99)]),
    ("dense", {"units": "4", "use_bias": "False"}, [((2, 9), -70000, 70000), ((4, 9), -70000, 70000)]),
    ("relu", {}, [((777,), -2 ** 31, 2 ** 31 - 1)]),
    ("abs", {}, [((777,), -2 ** 31, 2 ** 31 - 1)]),
    ("negative", {}, [((777,), -2 ** 31, 2 ** 31 - 1)]),
    ("cvm_precision", {}, [((777,), -2 ** 31, 2 ** 31 - 1)]),
    ("clip", {"a_min": "-5", "a_max": "100"}, [((777,), -300, 300)]),
    ("cvm_clip", {"precision": "8"}, [((777,), -300, 300)]),
    ("cvm_clip", {"precision": "1"}, [((50,), -3, 3)]),
    ("cvm_clip", {"precision": "32"}, [((50,), -2 ** 31, 2 ** 31 - 1)]),
    ("cvm_left_shift", {"precision": "8", "shift_bit": "3"}, [((777,), -60, 60)]),
    ("elemwise_add", {}, [((501,), -2 ** 31, 2 ** 31 - 1), ((501,), -2 ** 31, 2 ** 31 - 1)]),
    ("elemwise_sub", {}, [((501,), -2 ** 31, 2 ** 31 - 1), ((501,), -2 ** 31, 2 ** 31 - 1)]),
    ("max_pool2d", {"pool_size": "[3, 3]", "strides": "(2, 2)", "padding": "(1, 1)"}, [((2, 3, 10, 9), -2 ** 31, 2 ** 31 - 1)]),
    ("max_pool2d", {"pool_size": "[2, 2]", "strides": "(2, 2)", "padding": "(0, 0)", "ceil_mode": "True"}, [((1, 2, 7, 9), -99, 99)]),
    ("max_pool2d", {"pool_size": "[3, 2]", "strides": "(1, 2)", "padding": "(1,)"}, [((1, 2, 7, 7), -99, 99)]),
    ("concatenate", {"axis": "1"}, [((3, 1, 4, 5), -9, 9), ((3, 2, 4, 5), -9, 9), ((3, 1, 4, 5), -9, 9)]),
    ("concatenate", {"axis": "-1"}, [((3, 4, 5), -9, 9), ((3, 4, 2), -9, 9)]),
    ("transpose", {"axes": "(0, 2, 3, 1)"}, [((3, 2, 4, 5), -999, 999)]),
    ("transpose", {}, [((3, 2, 4, 5), -999, 999)]),
    ("transpose", {"axes": "(1, 2, 0)"}, [((3, 4, 5), -999, 999)]),
    ("strided_slice", {"begin": "(0, 0, 1)", "end": "(3, 1, 4)", "stride": "(2, 1, 2)"}, [((3, 1, 4, 5), -999, 999)]),
    ("strided_slice", {"begin": "(2, 0, 3)", "end": "(0, 1, 0)", "stride": "(-1, 1, -2)"}, [((3, 1, 4, 5), -999, 999)]),
    ("slice_like", {"axis": "(2, 3)"}, [((3, 1, 4, 5), -999, 999), ((1, 1, 2, 3), 0, 0)]),
    ("take", {}, [((3, 1, 4, 5), -999, 999), ((4, 3), -5, 70)]),
    ("take", {"axis": "2"}, [((3, 1, 4, 5), -999, 999), ((2, 3), -2, 6)]),
    ("take", {"axis": "0"}, [((3, 4), -999, 999), ((2, 3), -2, 6)]),
    ("cvm_lut", {"in_dim": "60"}, [((4, 3), -5, 70), ((60,), -999, 999)]),
    ("repeat", {"repeats": "3", "axis": "2"}, [((3, 1, 4, 5), -999, 999)]),
    ("tile", {"reps": "(2, 1, 3)"}, [((1, 4, 5), -999, 999)]),
    ("tile", {"reps": "(2, 1, 1, 3)"}, [((1, 4, 5), -999, 999)]),
    ("upsampling", {"scale": "2"}, [((2, 3, 4, 5), -999, 999)]),
    ("where", {}, [((3, 1, 4, 5), 0, 1), ((3, 1, 4, 5), -999, 999), ((3, 1, 4, 5), -999, 999)]),
    ("flatten", {}, [((3, 1, 4, 5), -999, 999)]),
    ("reshape", {"shape": "(-1, 5)"}, [((3, 1, 4, 5), -999, 999)]),
    ("reshape", {"shape": "(0, -3, -2)"}, [((3, 2, 4, 5), -999, 999)]),
    ("expand_dims", {"axis": "1", "num_newaxis": "2"}, [((3, 4), -999, 999)]),
    ("squeeze", {}, [((3, 1, 4, 1), -999, 999)]),
    ("squeeze", {"axis": "(1,)"}, [((3, 1, 4, 1), -999, 999)]),
    ("get_valid_counts", {"score_threshold": "10"}, [("boxes", 2, 300, 0)]),
    ("get_valid_counts", {"score_threshold": "-200"}, [("boxes", 1, 70, -1)]),
]
for _op in ("broadcast_add", "broadcast_sub", "broadcast_mul", "broadcast_max", "broadcast_div", "broadcast_greater"):
    OP_CASES.append((_op, {}, [((2, 3, 1, 5), -100, 100), ((3, 4, 1), -3, 3)]))
    OP_CASES.append((_op, {}, [((4, 7), -100, 100), ((1,), -3, -3)]))
    OP_CASES.append((_op, {}, [((1, 1), 7, 7), ((3, 1, 2), -3, 3)]))
for _op in ("sum", "max"):
    for _attrs in ({"axis": "(2, 3)"}, {}, {"axis": "(0,)", "keepdims": "True"}, {"axis": "(1, 3)", "exclude": "True"},
                   {"axis": "(0, 1, 2, 3)"}, {"axis": "(-1,)"}):
        OP_CASES.append((_op, _attrs, [((3, 1, 4, 5), -1000, -1)]))
        OP_CASES.append((_op, _attrs, [((3, 1, 4, 5), -1000, 1000)]))
for _p, _b in [(8, 8), (8, 1), (8, 24), (8, 23), (1, 5), (16, 16), (32, 1), (31, 1), (3, 31), (3, 32), (20, 11)]:
    OP_CASES.append(("cvm_right_shift", {"precision": str(_p), "shift_bit": str(_b)}, [((900,), -2 ** 31, 2 ** 31 - 1)]))

# (ids lower bound, iou, top_k, max_output_size, force_suppress, batches, anchors)
NMS_CASES = [(0, 45, -1, -1, False, 2, 120), (-1, 45, -1, -1, False, 2, 120), (-1, 30, 20, 10, True, 3, 64),
             (0, 50, 5, -1, False, 1, 64), (-1, 10, -1, 7, False, 2, 90), (0, 45, 0, -1, False, 1, 30),
             (-1, 60, 400, -1, True, 1, 600)]


def boxes(cid, b, n, id_lo, id_hi=3, extent=64):
    x = np.zeros((b, n, 6), np.int32)
    x[:, :, 0] = synth.tensor(cid, "id", (b, n), id_lo, id_hi)
    x[:, :, 1] = synth.tensor(cid, "score", (b, n), -20, 60)
    xy = np.sort(synth.tensor(cid, "xy", (b, n, 2, 2), 0, extent), axis=2)
    x[:, :, 2:] = xy.reshape(b, n, 4)
    return x


def make_inputs(index):
    op, attrs, specs = OP_CASES[index]
    ins = []
    for j, spec in enumerate(specs):
        if spec[0] == "boxes":
            ins.append(boxes("golden-%d" % index, spec[1], spec[2], spec[3]))
        else:
            shape, lo, hi = spec
            v = synth.tensor("golden-%d" % index, "in%d" % j, shape, lo, hi)
            if v.size >= 12 and lo == -2 ** 31:
                v.ravel()[:12] = [0, 1, -1, 127, -127, 128, -128, 2 ** 31 - 1, -2 ** 31, 2 ** 30, -2 ** 30, 255]
            ins.append(v)
    return ins


def nms_inputs(index):
    id_lo, iou, topk, mos, force, b, n = NMS_CASES[index]
    x = boxes("golden-nms-%d" % index, b, n, id_lo)
    vc = synth.tensor("golden-nms-%d" % index, "vc", (b,), n // 2, n).astype(np.int32)
    if index == 2:
        vc[1] = 0      # the call stops at the first batch without valid rows
    attrs = {"iou_threshold": str(iou), "top_k": str(topk), "max_output_size": str(mos), "force_suppress": str(force)}
    return x, vc, attrs


# host-logic cases: (op, attrs, input shapes, input precisions); expected status/shape/precision come from the reference
INFER_CASES = [
    ("conv2d", {"channels": "64", "kernel_size": "[3, 3]", "padding": "(1, 1)"}, [(1, 64, 56, 56), (64, 64, 3, 3), (64,)], [8, 8, 17]),
    ("conv2d", {"channels": "64", "kernel_size": "[3, 3]", "use_bias": "False"}, [(1, 64, 56, 56), (64, 64, 3, 3)], [8, 8]),
    ("conv2d", {"channels": "64", "kernel_size": "[3, 3]", "use_bias": "False"}, [(1, 64, 56, 56), (64, 64, 3, 3)], [9, 8]),
    ("conv2d", {"channels": "64", "kernel_size": "[3, 3]", "use_bias": "False"}, [(1, 64, 56, 56), (64, 32, 3, 3)], [8, 8]),
    ("conv2d", {"channels": "64", "kernel_size": "[3, 3]", "use_bias": "False", "layout": "NHWC"}, [(1, 64, 56, 56), (64, 64, 3, 3)], [8, 8]),
    ("conv2d", {"channels": "64", "kernel_size": "[9, 9]", "use_bias": "False"}, [(1, 64, 5, 5), (64, 64, 9, 9)], [8, 8]),
    ("conv2d", {"channels": "64", "kernel_size": "[3, 3]", "use_bias": "False", "groups": "64"}, [(1, 64, 56, 56), (64, 1, 3, 3)], [8, 8]),
    ("conv2d", {"channels": "64", "kernel_size": "[3, 3]", "use_bias": "False", "groups": "5"}, [(1, 64, 56, 56), (64, 1, 3, 3)], [8, 8]),
    ("conv2d", {"channels": "64", "kernel_size": "[3, 3]", "use_bias": "False", "strides": "(0, 1)"}, [(1, 64, 56, 56), (64, 64, 3, 3)], [8, 8]),
    ("conv2d", {"channels": "64", "kernel_size": "[3, 3]", "bogus": "1"}, [(1, 64, 56, 56), (64, 64, 3, 3), (64,)], [8, 8, 8]),
    ("conv2d", {"kernel_size": "[3, 3]"}, [(1, 64, 56, 56), (64, 64, 3, 3), (64,)], [8, 8, 8]),
    ("conv2d", {"channels": "x", "kernel_size": "[3, 3]"}, [(1, 64, 56, 56), (64, 64, 3, 3), (64,)], [8, 8, 8]),
    ("dense", {"units": "1000"}, [(16, 2048), (1000, 2048), (1000,)], [8, 8, 20]),
    ("dense", {"units": "1000", "use_bias": "False"}, [(16, 2048), (1000, 2047)], [8, 8]),
    ("dense", {"units": "0", "use_bias": "False"}, [(16, 2048), (1000, 2048)], [8, 8]),
    ("dense", {"units": "10", "use_bias": "0"}, [(16, 4, 4), (10, 4)], [8, 8]),
    ("max_pool2d", {"pool_size": "[3, 3]", "strides": "(2, 2)", "padding": "(1, 1)"}, [(16, 64, 112, 112)], [8]),
    ("max_pool2d", {"pool_size": "[2, 2]", "strides": "(2, 2)", "ceil_mode": "True"}, [(1, 3, 9, 11)], [8]),
    ("max_pool2d", {"pool_size": "[2, 2]", "padding": "(2, 2)"}, [(1, 3, 9, 11)], [8]),
    ("max_pool2d", {"pool_size": "[2, 2]", "padding": "(1,)"}, [(1, 3, 9, 11)], [8]),
    ("elemwise_add", {}, [(2, 3), (2, 3)], [8, 12]),
    ("elemwise_add", {}, [(2, 3), (3, 2)], [8, 8]),
    ("clip", {"a_min": "-5", "a_max": "100"}, [(2, 3)], [20]),
    ("clip", {"a_min": "5", "a_max": "1"}, [(2, 3)], [20]),
    ("cvm_clip", {"precision": "8"}, [(2, 3)], [20]),
    ("cvm_clip", {"precision": "33"}, [(2, 3)], [20]),
    ("cvm_right_shift", {"precision": "8", "shift_bit": "8"}, [(2, 3)], [28]),
    ("cvm_right_shift", {"precision": "8", "shift_bit": "0"}, [(2, 3)], [28]),
    ("cvm_left_shift", {"precision": "8", "shift_bit": "3"}, [(2, 3)], [8]),
    ("cvm_left_shift", {"precision": "8", "shift_bit": "3"}, [(2, 3)], [30]),
    ("cvm_precision", {}, [(2, 3)], [30]),
    ("broadcast_add", {}, [(2, 3, 1, 5), (3, 4, 1)], [8, 9]),
    ("broadcast_mul", {}, [(2, 3, 1, 5), (1,)], [8, 9]),
    ("broadcast_max", {}, [(2, 3), (4, 3)], [8, 9]),
    ("broadcast_div", {}, [(2, 3), (2, 3)], [8, 9]),
    ("sum", {"axis": "(2, 3)"}, [(16, 2048, 7, 7)], [8]),
    ("sum", {}, [(3, 4)], [8]),
    ("sum", {"axis": "(1,)", "keepdims": "True"}, [(3, 4, 5)], [8]),
    ("sum", {"axis": "(0, 0)"}, [(3, 4, 5)], [8]),
    ("sum", {"axis": "(3,)"}, [(3, 4, 5)], [8]),
    ("max", {"axis": "(0, 2)", "exclude": "True"}, [(3, 4, 5)], [8]),
    ("flatten", {}, [(2, 3, 4, 5)], [8]),
    ("reshape", {"shape": "(-1, 5)"}, [(2, 3, 4, 5)], [8]),
    ("reshape", {"shape": "(7, -1)"}, [(2, 3, 4, 5)], [8]),
    ("reshape", {"shape": "(-4, 1, 2, -2)"}, [(2, 3, 4)], [8]),
    ("expand_dims", {"axis": "-1"}, [(2, 3)], [8]),
    ("expand_dims", {"axis": "4"}, [(2, 3)], [8]),
    ("squeeze", {"axis": "(0,)"}, [(2, 1, 3)], [8]),
    ("squeeze", {}, [(1, 1)], [8]),
    ("concatenate", {"axis": "1"}, [(2, 3, 4), (2, 5, 4)], [8, 10]),
    ("concatenate", {"axis": "1"}, [(2, 3, 4), (2, 5, 5)], [8, 10]),
    ("transpose", {"axes": "(1, 0, 2)"}, [(2, 3, 4)], [8]),
    ("transpose", {"axes": "(1, 1, 2)"}, [(2, 3, 4)], [8]),
    ("strided_slice", {"begin": "(0, 1)", "end": "(2, 4)", "stride": "(1, 2)"}, [(3, 5)], [8]),
    ("strided_slice", {"begin": "(2,)", "end": "(1,)"}, [(3, 5)], [8]),
    ("take", {"axis": "1"}, [(3, 4, 5), (2, 2)], [8, 32]),
    ("take", {}, [(3, 4, 5), (7,)], [8, 32]),
    ("cvm_lut", {"in_dim": "256"}, [(3, 4), (256,)], [8, 20]),
    ("cvm_lut", {"in_dim": "255"}, [(3, 4), (256,)], [8, 20]),
    ("slice_like", {"axis": "(2, 3)"}, [(1, 3, 8, 8), (1, 5, 4, 4)], [8, 8]),
    ("slice_like", {}, [(1, 3, 8, 8), (1, 5, 4, 4)], [8, 8]),
    ("repeat", {"repeats": "2", "axis": "-1"}, [(2, 3)], [8]),
    ("repeat", {"repeats": "0"}, [(2, 3)], [8]),
    ("tile", {"reps": "(2, 3, 1)"}, [(4, 5)], [8]),
    ("tile", {"reps": "(0,)"}, [(4, 5)], [8]),
    ("upsampling", {"scale": "2"}, [(1, 3, 4, 4)], [8]),
    ("upsampling", {"scale": "2", "method": "BILINEAR"}, [(1, 3, 4, 4)], [8]),
    ("where", {}, [(3,), (3, 4), (3, 4)], [1, 8, 9]),
    ("where", {}, [(4,), (3, 4), (3, 4)], [1, 8, 9]),
    ("get_valid_counts", {"score_threshold": "10"}, [(1, 24564, 6)], [12]),
    ("get_valid_counts", {}, [(1, 24564, 40)], [12]),
    ("non_max_suppression", {"iou_threshold": "45", "top_k": "400"}, [(1, 24564, 6), (1,)], [12, 16]),
    ("non_max_suppression", {"iou_threshold": "0"}, [(1, 24564, 6), (1,)], [12, 16]),
    ("non_max_suppression", {"return_indices": "True"}, [(1, 24564, 6), (1,)], [12, 16]),
    ("non_max_suppression", {}, [(1, 24564, 5), (1,)], [12, 16]),
]
