"""GPU parity: every operator of the C ABI (include/cvm_hip_ops.h) against the
CPU oracle on the same seeded inputs.  Bit-exact (integer work): the only
accepted difference is none.  Cases follow the reference's per-op test list
(tests/test_op.cc:662-693) plus the ops it has no cases for."""
import numpy as np
import pytest
import torch

import oracle
from cvm_runtime_amd import hipops, synth

pytestmark = pytest.mark.gpu


def T(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(dev)


def same(t, ref, what=""):
    torch.cuda.synchronize()
    got = t.cpu().numpy()
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    if not np.array_equal(got, ref):
        bad = np.argwhere(got != ref)
        raise AssertionError("%s: %d of %d differ, first at %s: got %d want %d" % (
            what, len(bad), ref.size, bad[0], got[tuple(bad[0])], ref[tuple(bad[0])]))


CONV_CASES = [
    # n, ic, h, w, oc, kh, kw, stride, pad, dil, bias
    (1, 64, 56, 56, 64, 3, 3, (1, 1), (1, 1), (1, 1), True),     # BASELINE config 1
    (2, 3, 32, 32, 16, 3, 3, (1, 1), (1, 1), (1, 1), True),      # first layer, 3 channels (4-byte granules)
    (1, 3, 64, 64, 64, 7, 7, (2, 2), (3, 3), (1, 1), False),     # ResNet-50 stem shape, shrunk
    (3, 8, 15, 17, 24, 3, 3, (2, 1), (1, 2), (1, 1), True),      # 8 channels (8-byte granules), ragged
    (2, 16, 9, 11, 10, 1, 1, (1, 1), (0, 0), (1, 1), False),     # 1x1
    (1, 48, 13, 13, 70, 3, 3, (1, 1), (2, 2), (2, 2), True),     # dilation, channel count not a multiple of 64
    (2, 20, 14, 14, 130, 5, 3, (2, 2), (2, 1), (1, 1), True),    # channels padded 20 -> 32, oc > 128
    (16, 256, 7, 7, 512, 1, 1, (1, 1), (0, 0), (1, 1), False),   # small-spatial bottleneck
    (1, 1, 5, 5, 1, 3, 3, (1, 1), (0, 0), (1, 1), False),        # minimum sizes
    (1, 128, 28, 28, 128, 3, 3, (2, 2), (1, 1), (1, 1), True),   # strided 3x3
]


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "n%dc%dh%dw%d_o%dk%dx%d" % c[:7])
def test_conv2d(case, dev):
    n, ic, h, w, oc, kh, kw, st, pd, dl, bias = case
    cid = "conv-%s" % (case,)
    x = synth.tensor(cid, "x", (n, ic, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (oc, ic, kh, kw), -127, 127)
    b = synth.tensor(cid, "b", (oc,), -32768, 32768) if bias else None
    ref = oracle.conv2d(x, wt, b, st, pd, dl, 1)
    y = hipops.conv2d(T(x, dev), T(wt, dev), T(b, dev) if bias else None, st, pd, dl, 1)
    same(y, ref, "conv2d")


def test_conv2d_closed_form_ones(dev):
    # all-ones data and filter: every output equals the number of in-bounds taps x IC
    x = np.ones((1, 32, 6, 6), np.int32)
    w = np.ones((8, 32, 3, 3), np.int32)
    y = hipops.conv2d(T(x, dev), T(w, dev), None, (1, 1), (1, 1)).cpu().numpy()
    cnt = np.full((6, 6), 9)
    cnt[0, :] = cnt[-1, :] = cnt[:, 0] = cnt[:, -1] = 6
    cnt[0, 0] = cnt[0, -1] = cnt[-1, 0] = cnt[-1, -1] = 4
    assert np.array_equal(y[0, 3], cnt * 32)


def test_conv2d_narrows_like_the_reference(dev):
    # values outside int8 are truncated with static_cast<int8_t> in the groups == 1 path
    x = synth.tensor("conv-trunc", "x", (1, 16, 8, 8), -1000, 1000)
    w = synth.tensor("conv-trunc", "w", (8, 16, 3, 3), -300, 300)
    same(hipops.conv2d(T(x, dev), T(w, dev), None, (1, 1), (1, 1)), oracle.conv2d(x, w, None, (1, 1), (1, 1)), "trunc")


def test_conv2d_accumulator_wraps(dev):
    x = np.full((1, 4096, 3, 3), -128, np.int32)
    w = np.full((2, 4096, 3, 3), -128, np.int32)
    b = np.array([2 ** 31 - 1, -2 ** 31], np.int32)
    same(hipops.conv2d(T(x, dev), T(w, dev), T(b, dev), (1, 1), (1, 1)), oracle.conv2d(x, w, b, (1, 1), (1, 1)), "wrap")


GROUP_CASES = [
    (2, 32, 14, 14, 32, 3, 3, (1, 1), (1, 1), (1, 1), 32, True),   # depthwise
    (1, 32, 16, 16, 32, 3, 3, (2, 2), (1, 1), (1, 1), 32, False),  # depthwise stride 2
    (2, 12, 9, 9, 8, 3, 3, (1, 1), (0, 0), (1, 1), 4, True),       # grouped
    (1, 8, 7, 7, 8, 3, 3, (1, 1), (2, 2), (2, 2), 2, False),       # grouped + dilation
]


@pytest.mark.parametrize("case", GROUP_CASES, ids=lambda c: "g%d_c%d" % (c[10], c[1]))
def test_conv2d_grouped_is_exact_int32(case, dev):
    n, ic, h, w, oc, kh, kw, st, pd, dl, groups, bias = case
    cid = "gconv-%s" % (case,)
    x = synth.tensor(cid, "x", (n, ic, h, w), -40000, 40000)   # no narrowing in this path
    wt = synth.tensor(cid, "w", (oc, ic // groups, kh, kw), -40000, 40000)
    b = synth.tensor(cid, "b", (oc,), -2 ** 30, 2 ** 30) if bias else None
    ref = oracle.conv2d(x, wt, b, st, pd, dl, groups)
    same(hipops.conv2d(T(x, dev), T(wt, dev), T(b, dev) if bias else None, st, pd, dl, groups), ref, "grouped")


@pytest.mark.parametrize("m,k,n,bias", [(1, 2048, 1000, True), (16, 2048, 1000, True), (1, 64, 10, False),
                                        (64, 64, 10, True), (3, 100, 7, True), (1, 25088, 64, False)])
def test_dense(m, k, n, bias, dev):
    cid = "dense-%d-%d-%d" % (m, k, n)
    x = synth.tensor(cid, "x", (m, k), -127, 127)
    w = synth.tensor(cid, "w", (n, k), -127, 127)
    b = synth.tensor(cid, "b", (n,), -100000, 100000) if bias else None
    same(hipops.dense(T(x, dev), T(w, dev), T(b, dev) if bias else None), oracle.dense(x, w, b), "dense")


def test_dense_wide_operands_exact(dev):
    x = synth.tensor("dense-wide", "x", (5, 333), -70000, 70000)
    w = synth.tensor("dense-wide", "w", (9, 333), -70000, 70000)
    b = synth.tensor("dense-wide", "b", (9,), -5, 5)
    same(hipops.dense(T(x, dev), T(w, dev), T(b, dev), operand_bits=32), oracle.dense(x, w, b), "dense32")


def _edge_values(n, seed):
    v = synth.tensor("edges", "v%d" % seed, (n,), -2 ** 31, 2 ** 31 - 1)
    v[:12] = [0, 1, -1, 127, -127, 128, -128, 2 ** 31 - 1, -2 ** 31, 2 ** 30, -2 ** 30, 255]
    return v


@pytest.mark.parametrize("size", [1, 3, 4, 1023, 200704])
def test_unary_ops(size, dev):
    v = _edge_values(max(size, 12), size)[:size].copy()
    t = T(v, dev)
    same(hipops.relu(t), oracle.relu(v), "relu")
    same(hipops.abs_(t), oracle.abs_(v), "abs")
    same(hipops.negative(t), oracle.negative(v), "negative")
    same(hipops.cvm_precision(t), oracle.cvm_precision(v), "cvm_precision")
    same(hipops.clip(t, -5, 100), oracle.clip(v, -5, 100), "clip")
    for p in (1, 2, 8, 16, 31, 32):
        same(hipops.cvm_clip(t, p), oracle.cvm_clip(v, p), "cvm_clip p=%d" % p)
        same(hipops.cvm_left_shift(t, p, 3), oracle.cvm_left_shift(v, p, 3), "lshift")


def test_cvm_right_shift_all_parameter_pairs(dev):
    v = _edge_values(4096, 7)
    t = T(v, dev)
    for p in range(1, 33):
        for b in range(1, 33):
            same(hipops.cvm_right_shift(t, p, b), oracle.cvm_right_shift(v, p, b), "rshift p=%d b=%d" % (p, b))


def test_unary_in_place_and_unaligned(dev):
    v = _edge_values(1001, 3)
    t = T(v, dev)
    hipops.cvm_right_shift(t, 8, 5, out=t)       # in place: whitelisted by the graph runtime
    same(t, oracle.cvm_right_shift(v, 8, 5), "in place")
    big = T(np.concatenate([[0], v]), dev)
    view = big[1:]                                # 4-byte aligned only
    same(hipops.relu(view.contiguous() if not view.is_contiguous() else view), oracle.relu(v), "unaligned")


def test_elemwise(dev):
    a = _edge_values(5003, 1)
    b = _edge_values(5003, 2)[::-1].copy()
    ta, tb = T(a, dev), T(b, dev)
    same(hipops.elemwise("elemwise_add", ta, tb), oracle.elemwise("elemwise_add", a, b), "add")
    same(hipops.elemwise("elemwise_sub", ta, tb), oracle.elemwise("elemwise_sub", a, b), "sub")
    hipops.elemwise("elemwise_add", ta, tb, out=ta)
    same(ta, oracle.elemwise("elemwise_add", a, b), "add in place")


BSHAPES = [((2, 3, 4, 5), (2, 3, 4, 5)), ((2, 3, 1, 5), (3, 4, 1)), ((4, 7), (1,)), ((1,), (4, 7)),
           ((1, 1), (3, 1, 2)), ((16, 64, 7, 7), (64, 1, 1)), ((5,), (5,)), ((2, 1, 3, 1, 2, 1), (1, 4, 1, 5, 1, 3))]


@pytest.mark.parametrize("op", list(hipops.BCAST))
def test_broadcast(op, dev):
    for i, (sa, sb) in enumerate(BSHAPES):
        a = synth.tensor("bcast", "a%d" % i, sa, -2000, 2000)
        b = synth.tensor("bcast", "b%d" % i, sb, -3, 3)   # zeros exercise div-by-zero -> 0
        same(hipops.broadcast(op, T(a, dev), T(b, dev)), oracle.broadcast(op, a, b), "%s %s %s" % (op, sa, sb))
    a = np.array([-2 ** 31, 2 ** 31 - 1, 7], np.int32)
    b = np.array([-1, -1, -1], np.int32)
    same(hipops.broadcast(op, T(a, dev), T(b, dev)), oracle.broadcast(op, a, b), op + " extremes")


@pytest.mark.parametrize("case", [((16, 64, 112, 112), (3, 3), (2, 2), (1, 1), False),
                                  ((2, 8, 14, 14), (2, 2), (2, 2), (0, 0), False),
                                  ((1, 3, 9, 11), (2, 2), (2, 2), (0, 0), True),
                                  ((1, 2, 7, 7), (3, 2), (1, 2), (1,), False),
                                  # 3x3 stride 2 on rows of a multiple of 4 (the paired kernel): both paddings,
                                  # odd output widths, one-pair rows, ceil_mode (falls back to the general kernel)
                                  ((2, 5, 12, 12), (3, 3), (2, 2), (0, 0), False),
                                  ((3, 4, 9, 8), (3, 3), (2, 2), (1, 1), False),
                                  ((1, 7, 5, 4), (3, 3), (2, 2), (1, 1), False),
                                  ((1, 3, 16, 20), (3, 3), (2, 2), (0, 1), False),
                                  ((1, 3, 16, 20), (3, 3), (2, 2), (1, 0), False),
                                  ((2, 3, 12, 12), (3, 3), (2, 2), (1, 1), True),
                                  ((1, 2, 11, 16), (3, 3), (2, 2), (0, 0), True),
                                  # 2x2 stride 2 without padding on rows of a multiple of 4 (the paired kernel): an odd
                                  # height, one pair per row, ceil_mode with a last window past the image (general kernel)
                                  ((2, 3, 16, 16), (2, 2), (2, 2), (0, 0), False),
                                  ((1, 5, 9, 12), (2, 2), (2, 2), (0, 0), False),
                                  ((3, 2, 8, 4), (2, 2), (2, 2), (0, 0), False),
                                  ((1, 2, 8, 20), (2, 2), (2, 2), (0, 0), True),
                                  ((1, 2, 7, 12), (2, 2), (2, 2), (0, 0), True),
                                  ((2, 64, 56, 56), (2, 2), (2, 2), (0, 0), False)])
def test_max_pool2d(case, dev):
    shape, k, s, p, ceil = case
    x = synth.tensor("pool", str(case), shape, -2 ** 31, 2 ** 31 - 1)
    same(hipops.max_pool2d(T(x, dev), k, s, p, ceil), oracle.max_pool2d(x, k, s, p, ceil), "max_pool2d")


@pytest.mark.parametrize("op", ["sum", "max"])
def test_reduce(op, dev):
    x = synth.tensor("reduce", "x", (3, 1, 4, 5), -1000, 1000)
    neg = -np.abs(x) - 1
    for v in (x, neg):
        t = T(v, dev)
        for axes, keep, excl in [((2, 3), False, False), ((), False, False), ((0,), True, False),
                                 ((1, 3), False, True), ((0, 1, 2, 3), False, False), ((-1,), False, False),
                                 ((0, 1, 2, 3), False, True)]:
            same(hipops.reduce(op, t, axes, keep, excl), oracle.reduce(op, v, axes, keep, excl),
                 "%s axes=%s keep=%s excl=%s" % (op, axes, keep, excl))
    gap = synth.tensor("reduce", "gap", (16, 2048, 7, 7), -127, 127)
    same(hipops.reduce(op, T(gap, dev), (2, 3)), oracle.reduce(op, gap, (2, 3)), "global pool")
    # short contiguous runs on both sides of the lane-group sizes (1, 8, 9, 21, 64, 65, 300, 512, 513 elements)
    for run in (1, 8, 9, 21, 64, 65, 300, 512, 513):
        v = synth.tensor("reduce", "run%d" % run, (37, run), -2 ** 31, 2 ** 31 - 1)
        same(hipops.reduce(op, T(v, dev), (1,)), oracle.reduce(op, v, (1,)), "run of %d" % run)
        w = -np.abs(synth.tensor("reduce", "neg%d" % run, (5, 3, run), -1000, 1000)) - 1   # all negative: max stays negative
        same(hipops.reduce(op, T(w, dev), (2,)), oracle.reduce(op, w, (2,)), "negative run of %d" % run)
    big = synth.tensor("reduce", "big", (1 << 20,), -2 ** 31, 2 ** 31 - 1)   # full reduction wraps
    same(hipops.reduce(op, T(big, dev)), oracle.reduce(op, big), "full")


def test_remap_ops(dev):
    x = synth.tensor("remap", "x", (3, 1, 4, 5), -1000, 1000)
    t = T(x, dev)
    same(hipops.concatenate([t, t, t], 1), oracle.concatenate([x, x, x], 1), "concat axis 1")
    same(hipops.concatenate([t, t], -1), oracle.concatenate([x, x], -1), "concat axis -1")
    y = synth.tensor("remap", "y", (3, 2, 4, 5), -9, 9)
    same(hipops.concatenate([t, T(y, dev)], 1), oracle.concatenate([x, y], 1), "concat ragged")
    for axes in [(0, 2, 3, 1), (), (3, 2, 1, 0), (0, -1, 1, 2)]:
        same(hipops.transpose(t, axes), oracle.transpose(x, axes), "transpose %s" % (axes,))
    x3 = x[:, 0]
    same(hipops.transpose(T(x3, dev), (1, 2, 0)), oracle.transpose(x3, (1, 2, 0)), "transpose (1,2,0)")
    # the tiled path (a trailing group of dims moved in front of the group before it), ragged against the 32x32 tile
    for shape, axes in [((2, 33, 7, 9), (0, 2, 3, 1)), ((1, 126, 64, 64), (0, 2, 3, 1)), ((3, 5, 6, 40), (0, 3, 1, 2)),
                        ((65, 31), (1, 0)), ((4, 3, 70), (2, 0, 1)), ((2, 3, 4, 5, 6), (0, 1, 4, 2, 3)),
                        ((2, 1, 50), (0, 2, 1)), ((5, 1, 1, 8), (0, 3, 1, 2))]:
        v = synth.tensor("remap", "t%s" % (shape,), shape, -2 ** 31, 2 ** 31 - 1)
        same(hipops.transpose(T(v, dev), axes), oracle.transpose(v, axes), "transpose %s %s" % (shape, axes))
    for b, e, s in [((0, 0, 1), (3, 1, 4), (2, 1, 2)), ((2, 0, 3), (0, 1, 0), (-1, 1, -2)), ((1,), (3,), ())]:
        ref = oracle.strided_slice(x, b, e, s)
        same(hipops.strided_slice(t, b, e, s, ref.shape), ref, "strided_slice")
    ref = oracle.slice_like(x, (1, 1, 2, 3), (2, 3))
    same(hipops.slice_like(t, ref.shape), ref, "slice_like")
    same(hipops.repeat(t, 3, 2), oracle.repeat(x, 3, 2), "repeat")
    same(hipops.repeat(t, 2, -1), oracle.repeat(x, 2, -1), "repeat -1")
    same(hipops.tile(T(x[0], dev), (2, 1, 3)), oracle.tile(x[0], (2, 1, 3)), "tile")
    same(hipops.tile(T(x[0], dev), (2, 1, 1, 3)), oracle.tile(x[0], (2, 1, 1, 3)), "tile lead")
    same(hipops.upsampling(t, 2), oracle.upsampling(x, 2), "upsampling")
    same(hipops.copy(t, (3, 20)), x.reshape(3, 20), "flatten")
    idx = synth.tensor("remap", "i", (4, 3), -5, 70)
    same(hipops.take(t, T(idx, dev)), oracle.take(x, idx), "take flat")
    idx2 = synth.tensor("remap", "i2", (2, 3), -2, 6)
    same(hipops.take(t, T(idx2, dev), 2), oracle.take(x, idx2, 2), "take axis 2")
    x2 = np.ascontiguousarray(x[:, 0, :, 0])
    same(hipops.take(T(x2, dev), T(idx2, dev), 0), oracle.take(x2, idx2, 0), "take axis 0")
    cond = synth.tensor("remap", "c", x.shape, 0, 1)
    out = torch.zeros_like(t)
    same(hipops.where(T(cond, dev), t, T(-x, dev), out), oracle.where(cond, x, -x), "where")
    init = np.full_like(x, 9)
    c1 = np.array([0, 1, 0], np.int32)
    out = T(init, dev)
    same(hipops.where(T(c1, dev), t, T(-x, dev), out), oracle.where(c1, x, -x, init), "where 1-D condition")


def _boxes(cid, b, n, id_lo, id_hi=20, score=(-127, 127), extent=512):
    x = np.zeros((b, n, 6), np.int32)
    x[:, :, 0] = synth.tensor(cid, "id", (b, n), id_lo, id_hi)
    x[:, :, 1] = synth.tensor(cid, "score", (b, n), score[0], score[1])
    xy = synth.tensor(cid, "xy", (b, n, 2, 2), 0, extent)
    xy = np.sort(xy, axis=2)   # (x1,y1) <= (x2,y2)
    x[:, :, 2:] = xy.reshape(b, n, 4)
    return x


@pytest.mark.parametrize("b,n,thr", [(1, 24564, 10), (2, 1000, 0), (3, 255, -200), (1, 257, 200), (2, 1, 0)])
def test_get_valid_counts(b, n, thr, dev):
    x = _boxes("gvc-%d-%d" % (b, n), b, n, 0)
    vc_ref, y_ref = oracle.get_valid_counts(x, thr)
    vc, y = hipops.get_valid_counts(T(x, dev), thr)
    same(vc, vc_ref, "valid_count")
    same(y, y_ref, "compacted rows")


NMS_CASES = [
    # b, n, id_lo, iou, topk, mos, force, extent
    (1, 24564, 0, 45, 400, -1, False, 512),    # BASELINE config 5
    (1, 24564, -1, 45, 400, -1, False, 512),   # negative ids: the CPU early-break semantics
    (2, 300, -1, 30, -1, -1, False, 64),
    (2, 300, -1, 30, -1, -1, True, 64),
    (2, 300, 0, 50, 20, 10, False, 64),
    (3, 64, -1, 10, 5, 3, True, 32),
    (1, 2000, -1, 45, -1, 100, False, 128),
    (2, 50, 0, 45, 0, -1, False, 64),          # top_k == 0 keeps nothing
    (1, 1, 0, 45, -1, -1, False, 64),
    (1, 4000, -1, 45, -1, -1, False, 256),     # more candidate rows than the kernel stages on chip
    (1, 3000, -1, 45, 512, -1, False, 128),    # the largest top_k that takes the bit-matrix walk
    (2, 3000, -1, 45, 513, 200, False, 128),   # one more: the row-by-row walk
    (2, 700, 0, 45, 65, -1, True, 48),         # top_k straddling a 64-row ballot
]


@pytest.mark.parametrize("case", NMS_CASES, ids=lambda c: "b%dn%d_id%d_iou%d_k%d_m%d_f%d" % c[:7])
def test_non_max_suppression(case, dev):
    b, n, id_lo, iou, topk, mos, force, extent = case
    x = _boxes("nms-%s" % (case,), b, n, id_lo, 20 if n > 1000 else 3, extent=extent)
    vc, xs = oracle.get_valid_counts(x, 10)
    init = np.full_like(xs, 5)
    y_ref, x_after = oracle.non_max_suppression(xs, vc, iou, force, topk, max_output_size=mos, y_init=init)
    tx, ty = T(xs, dev), T(init, dev)
    hipops.non_max_suppression(tx, T(vc, dev), ty, iou, force, topk, max_output_size=mos)
    same(ty, y_ref, "nms output")
    same(tx, x_after, "nms input after the call")


@pytest.mark.parametrize("score,topk,n", [((-2 ** 31, 2 ** 31 - 1), 400, 5000),   # keys differ in every bit
                                          ((7, 7), 50, 900),                      # all scores equal: order by index alone
                                          ((-3, 3), 300, 4000),                   # long runs of equal scores around the cut
                                          ((2 ** 31 - 5, 2 ** 31 - 1), 2048, 3000),  # the largest top_k of the selection path
                                          ((-2 ** 31, -2 ** 31 + 2), 2049, 3000),    # one more: all-pairs ranking
                                          ((0, 1000), 1, 700),
                                          ((-50, 50), 400, 300),                  # top_k above the row count: every row ranked in the list
                                          ((-2 ** 31, 2 ** 31 - 1), 2048, 2048),  # ... with the list full
                                          ((-2 ** 31, 2 ** 31 - 1), 400, 32768),  # the most rows the selection path takes: 32 per thread
                                          ((-2 ** 31, -2 ** 31 + 3), 1000, 20000),  # the lowest scores there are, in long runs; 20 rows per thread
                                          ((-100, 100), 2048, 28700),             # 29 rows per thread, the last block of four partly filled
                                          ((0, 2 ** 20), 600, 14000)])            # 14 rows per thread
def test_nms_top_k_selection(score, topk, n, dev):
    """Rows past top_k only need to be known as such; the first top_k must come out in the stable-sort order."""
    x = _boxes("nms-topk-%s-%d" % (score, topk), 2, n, -1, 3, score=score, extent=256)
    vc = np.array([n, n - 7], np.int32)
    init = np.full_like(x, 5)
    y_ref, x_after = oracle.non_max_suppression(x, vc, 60, False, topk, y_init=init)
    tx, ty = T(x, dev), T(init, dev)
    hipops.non_max_suppression(tx, T(vc, dev), ty, 60, False, topk)
    same(ty, y_ref, "nms output")
    same(tx, x_after, "nms input after the call")


@pytest.mark.parametrize("b,n,score,topk,extent", [
    (1, 24564, (-127, 127), -1, 16),             # the detector's anchor count without top_k: long runs of equal scores
    (2, 100000, (-1000, 1000), -1, 12),
    (1, 20000, (-2 ** 31, 2 ** 31 - 1), 3000, 24),   # top_k above what the selection path takes; keys differ in every bit
    (2, 8192, (0, 3), -1, 8),                     # the fewest rows that are sorted; four distinct scores
    (2, 8191, (0, 3), -1, 8),                     # one fewer: ranked by counting
    (1, 70000, (5, 5), 40000, 10),                # every score equal: the order is the row index alone
])
def test_nms_many_rows_without_usable_top_k_are_ranked_by_a_stable_sort(b, n, score, topk, extent, dev):
    """From 8192 rows on, rows are ranked by a least-significant-digit radix sort on (score descending) that keeps rows
    of equal score in index order -- the order of the reference's std::stable_sort (nms.cc:89-91)."""
    x = _boxes("nms-sort-%d-%d-%s" % (b, n, score), b, n, -1, 3, score=score, extent=extent)
    vc = np.array([n - 777 * i for i in range(b)], np.int32)
    init = np.full_like(x, 5)
    y_ref, x_after = oracle.non_max_suppression(x, vc, 45, False, topk, y_init=init)
    tx, ty = T(x, dev), T(init, dev)
    hipops.non_max_suppression(tx, T(vc, dev), ty, 45, False, topk)
    same(ty, y_ref, "nms output")
    same(tx, x_after, "nms input after the call")


def test_nms_stops_at_first_batch_without_valid_rows(dev):
    x = _boxes("nms-early", 3, 40, 0, 3, extent=32)
    vc = np.array([12, 0, 30], np.int32)
    init = np.full_like(x, 5)
    y_ref, x_after = oracle.non_max_suppression(x, vc, 45, y_init=init)
    assert np.all(y_ref[2] == 5)   # the reference leaves later batches untouched
    tx, ty = T(x, dev), T(init, dev)
    hipops.non_max_suppression(tx, T(vc, dev), ty, 45)
    same(ty, y_ref, "early exit")
    vc2 = np.array([45, -3, 7], np.int32)   # clamped to [0, n]
    y_ref, _ = oracle.non_max_suppression(x, vc2, 45, y_init=init)
    ty = T(init, dev)
    hipops.non_max_suppression(T(x, dev), T(vc2, dev), ty, 45)
    same(ty, y_ref, "clamped counts")


def test_argument_errors_are_reported_not_launched(dev):
    from cvm_runtime_amd import CvmHipError
    t = T(np.zeros((4,), np.int32), dev)
    with pytest.raises(CvmHipError):
        hipops.cvm_clip(t, 0)
    with pytest.raises(CvmHipError):
        hipops.cvm_right_shift(t, 8, 33)
    x = T(np.zeros((1, 4, 6), np.int32), dev)
    with pytest.raises(CvmHipError):
        hipops.non_max_suppression(x, T(np.ones((1,), np.int32), dev), torch.empty_like(x), iou_threshold=0)
    # more candidate rows than the greedy walk is allowed: refused unless top_k bounds them
    big = torch.zeros((1, (1 << 18) + 1, 6), dtype=torch.int32, device=dev)
    with pytest.raises(CvmHipError):
        hipops.non_max_suppression(big, T(np.ones((1,), np.int32), dev), torch.empty_like(big), iou_threshold=45)
    hipops.non_max_suppression(big, T(np.ones((1,), np.int32), dev), torch.empty_like(big), iou_threshold=45, top_k=100)
