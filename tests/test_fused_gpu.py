"""GPU parity of the fused int8 entry points (include/cvm_hip_ops.h, "fused int8
path") against the CPU oracle running the same nodes one by one, and of the
fused graph executor against the node-by-node executor.  Bit-exact."""
import os

import numpy as np
import pytest
import torch

import oracle
import oracle.graph as og
from cvm_runtime_amd import CvmHipError, graphgen, hipops, runtime, synth

pytestmark = pytest.mark.gpu


def T(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(dev)


def act_to_nchw(t, n, c, h, w):
    """int8 activation buffer (library layout) -> int32 NCHW numpy; padding channels are checked to be zero."""
    torch.cuda.synchronize()
    a = t.cpu().numpy()
    cp = hipops.pad_channels(c)
    p = np.arange(n * h * w, dtype=np.int64)[:, None]
    ch = np.arange(cp, dtype=np.int64)[None, :]
    full = a[hipops.act_offset(p, ch, cp)].astype(np.int32)          # (pixels, cp)
    assert not full[:, c:].any(), "padding channels must stay zero"
    return np.ascontiguousarray(full[:, :c].reshape(n, h, w, c).transpose(0, 3, 1, 2))


def run_chain(v, stages):
    for st in stages:
        if st[0] == "relu":
            v = oracle.relu(v)
        elif st[0] == "cvm_right_shift":
            v = oracle.cvm_right_shift(v, st[1], st[2])
        elif st[0] == "cvm_clip":
            v = oracle.cvm_clip(v, st[1])
        elif st[0] == "mul":
            v = oracle.broadcast("broadcast_mul", v, np.array([st[1]], np.int32))
        else:
            v = oracle.clip(v, st[1], st[2])
    return v


def eq(got, ref, what):
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    if not np.array_equal(got, ref):
        bad = np.argwhere(got != ref)
        raise AssertionError("%s: %d of %d differ, first at %s: got %d want %d" % (
            what, len(bad), ref.size, bad[0], got[tuple(bad[0])], ref[tuple(bad[0])]))


@pytest.mark.parametrize("c", [1, 3, 5, 8, 13, 20, 64, 100])
def test_pack_unpack_round_trip(c, dev):
    x = synth.tensor("pack-%d" % c, "x", (3, c, 7, 5), -128, 127)
    xp = hipops.pack_act_i8(T(x, dev))
    assert hipops.pad_channels(c) >= c
    eq(act_to_nchw(xp, 3, c, 7, 5), x, "pack")
    y = hipops.unpack_act_i8(xp, 3, c, 7, 5)
    torch.cuda.synchronize()
    eq(y.cpu().numpy(), x, "unpack")


def test_pack_narrows_like_static_cast(dev):
    # values outside int8 are truncated exactly as the reference's static_cast<int8_t> (ops.cc:234)
    x = np.array([127, 128, 255, 256, -128, -129, 1000, -1000, 2**31 - 1, -2**31], np.int64).astype(np.int32).reshape(1, 10, 1, 1)
    xp = hipops.pack_act_i8(T(x, dev))
    eq(act_to_nchw(xp, 1, 10, 1, 1), x.astype(np.int8).astype(np.int32), "narrow")


FUSED_CONV = [
    # n, ic, h, w, oc, k, stride, pad, bias, chain, residual chain, int8 out
    (2, 64, 14, 14, 64, 3, 1, 1, True, [("relu",), ("cvm_right_shift", 8, 9)], None, True),
    (2, 64, 14, 14, 256, 1, 1, 0, False, [("cvm_right_shift", 8, 7)], [("relu",), ("cvm_right_shift", 8, 1)], True),
    (1, 3, 33, 31, 16, 7, 2, 3, True, [("relu",), ("cvm_right_shift", 8, 10), ("cvm_clip", 8)], None, True),
    (3, 8, 9, 9, 24, 3, 2, 1, True, [("cvm_right_shift", 8, 6), ("clip", -100, 90)], None, True),
    (1, 32, 12, 12, 40, 3, 1, 1, True, [("cvm_right_shift", 16, 3)], None, False),      # int32 NCHW output, wide values
    (1, 32, 12, 12, 40, 3, 1, 1, False, [], None, False),                                # no chain at all
    (2, 128, 7, 7, 130, 1, 1, 0, True, [("cvm_right_shift", 8, 8)], [("cvm_right_shift", 8, 1), ("relu",)], True),
    (1, 16, 6, 6, 20, 3, 1, 1, True, [("cvm_right_shift", 8, 31)], None, True),          # shift regime b >= 31
    (1, 16, 6, 6, 20, 3, 1, 1, True, [("cvm_right_shift", 8, 24), ("cvm_clip", 8)], None, True),  # regime p + b >= 32
    (16, 512, 7, 7, 512, 3, 1, 1, True, [("relu",), ("cvm_right_shift", 8, 12)], None, True),      # deep K (4608), few pixels
    (2, 64, 9, 9, 48, 3, 1, 1, True, [("relu",), ("mul", 93), ("cvm_right_shift", 8, 17)], None, True),   # scale then shift
    (1, 32, 8, 8, 32, 1, 1, 0, True, [("mul", -70001), ("cvm_right_shift", 8, 20), ("cvm_clip", 8)],
     [("mul", 3), ("cvm_right_shift", 8, 2)], True),                                               # products that wrap
    (4, 1024, 14, 14, 256, 1, 1, 0, False, [("relu",), ("cvm_right_shift", 8, 11)], None, True),
    # tap masks at their limits: a 32-tap filter side (bit 31 of the mask), and padding wider than the
    # filter so that whole receptive fields lie outside the image
    (1, 32, 8, 8, 32, 32, 1, 12, True, [("cvm_right_shift", 8, 14)], None, True),
    (2, 64, 5, 5, 64, 3, 1, 5, True, [("cvm_right_shift", 8, 9)], None, True),
    (1, 32, 6, 6, 64, 3, 2, 40, True, [("cvm_right_shift", 8, 9)], None, True),
]


@pytest.fixture(params=["auto", "lds", "wave", "big"])
def conv_kernel(request):
    """Both implicit-GEMM kernels must give the same bits: force each in turn (the library reads the hook per call)."""
    if request.param == "auto":
        os.environ.pop("CVM_HIP_CONV", None)
    else:
        os.environ["CVM_HIP_CONV"] = request.param
    yield request.param
    os.environ.pop("CVM_HIP_CONV", None)


@pytest.mark.parametrize("case", FUSED_CONV, ids=lambda c: "n%dc%dh%dw%d_o%dk%d" % c[:6])
def test_conv2d_i8(case, conv_kernel, dev):
    n, ic, h, w, oc, k, st, pd, bias, ch1, ch2, i8 = case
    cid = "fconv-%s" % (case[:8],)
    x = synth.tensor(cid, "x", (n, ic, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (oc, ic, k, k), -127, 127)
    b = synth.tensor(cid, "b", (oc,), -32768, 32768) if bias else None
    ref = run_chain(oracle.conv2d(x, wt, b, (st, st), (pd, pd), (1, 1), 1), ch1)
    oh, ow = ref.shape[2:]
    res_t = None
    if ch2 is not None:
        r = synth.tensor(cid, "r", ref.shape, -127, 127)
        ref = run_chain(oracle.elemwise("elemwise_add", ref, r), ch2)
        res_t = hipops.pack_act_i8(T(r, dev))
    xp = hipops.pack_act_i8(T(x, dev))
    wp = hipops.pack_weights(T(wt, dev))
    out = hipops.conv2d_i8(xp, n, ic, h, w, wp, oc, k, k, T(b, dev) if bias else None,
                           hipops.chain(*ch1) if ch1 else None, res_t, hipops.chain(*ch2) if ch2 else None,
                           out_is_i8=i8, strides=(st, st), padding=(pd, pd))
    if i8:
        assert ref.min() >= -128 and ref.max() <= 127, "case must be representable"
        eq(act_to_nchw(out, n, oc, oh, ow), ref, "conv2d_i8")
    else:
        torch.cuda.synchronize()
        eq(out.cpu().numpy(), ref, "conv2d_i8 -> int32")


def _random_conv_cases(count):
    """Seeded geometries across the addressing modes of both kernels: 1x1 / strided / padded / dilated,
    channel counts on both sides of the 4-8-16-32 padding steps, ragged pixel counts."""
    rng = np.random.RandomState(20240611)
    cases = []
    while len(cases) < count:
        ic = int(rng.choice([1, 3, 5, 8, 13, 16, 24, 32, 40, 64, 96, 160]))
        oc = int(rng.choice([1, 7, 16, 31, 32, 33, 64, 100, 130]))
        k = int(rng.choice([1, 1, 2, 3, 3, 5]))
        st = int(rng.choice([1, 1, 2, 3]))
        pd = int(rng.choice([0, 0, 1, 2]))
        dl = int(rng.choice([1, 1, 1, 2]))
        n = int(rng.choice([1, 2, 3]))
        h, w = int(rng.randint(1, 15)), int(rng.randint(1, 15))
        if h + 2 * pd < dl * (k - 1) + 1 or w + 2 * pd < dl * (k - 1) + 1:
            continue
        cases.append((n, ic, h, w, oc, k, st, pd, dl, bool(rng.randint(2)), bool(rng.randint(2)), bool(rng.randint(2))))
    return cases


@pytest.mark.parametrize("case", _random_conv_cases(48), ids=lambda c: "n%dc%dh%dw%d_o%dk%ds%dp%dd%d" % c[:9])
def test_conv2d_i8_random_geometries(case, dev):
    n, ic, h, w, oc, k, st, pd, dl, bias, with_res, i8 = case
    cid = "rconv-%s" % (case,)
    x = synth.tensor(cid, "x", (n, ic, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (oc, ic, k, k), -127, 127)
    b = synth.tensor(cid, "b", (oc,), -32768, 32768) if bias else None
    shift = max(1, int(np.ceil(np.log2(ic * k * k * 127 * 127 / 100.0))))
    ch1 = [("cvm_right_shift", 8, shift)]
    ch2 = [("relu",), ("cvm_right_shift", 8, 1)]
    ref = run_chain(oracle.conv2d(x, wt, b, (st, st), (pd, pd), (dl, dl), 1), ch1)
    oh, ow = ref.shape[2:]
    res_t = None
    if with_res:
        r = synth.tensor(cid, "r", ref.shape, -127, 127)
        ref = run_chain(oracle.elemwise("elemwise_add", ref, r), ch2)
        res_t = hipops.pack_act_i8(T(r, dev))
    xp, wp = hipops.pack_act_i8(T(x, dev)), hipops.pack_weights(T(wt, dev))
    for kind in ("lds", "wave", "big"):
        os.environ["CVM_HIP_CONV"] = kind
        try:
            out = hipops.conv2d_i8(xp, n, ic, h, w, wp, oc, k, k, T(b, dev) if bias else None, hipops.chain(*ch1), res_t,
                                   hipops.chain(*ch2) if with_res else None, out_is_i8=i8, strides=(st, st),
                                   padding=(pd, pd), dilation=(dl, dl))
        finally:
            os.environ.pop("CVM_HIP_CONV", None)
        if i8:
            eq(act_to_nchw(out, n, oc, oh, ow), ref, "conv2d_i8 (%s)" % kind)
        else:
            torch.cuda.synchronize()
            eq(out.cpu().numpy(), ref, "conv2d_i8 -> int32 (%s)" % kind)


KSLICE_CASES = [
    # n, ic, h, w, oc, k   (output 1x1: a dense layer over the flattened map, or a plain dense layer)
    (16, 512, 7, 7, 256, 7),      # the shape of VGG-16's first dense layer, fewer units
    (5, 8192, 1, 1, 100, 1),      # plain dense, ragged unit count, K exactly at the threshold
    (32, 8192, 1, 1, 96, 1),      # 32 rows: the one-pixel-block tile (at most 32 pixels, 1x1) completely full
    (16, 12544, 1, 1, 520, 1),    # 392 chunks of K over four slices and four wavefronts each, 17 channel tiles
    (33, 1024, 3, 3, 64, 3),      # 33 rows: second half of the pixel tile partly empty
    (1, 9216, 1, 1, 8192, 1),     # more than 256 tiles: not sliced, same answer
    (2, 4096, 1, 1, 64, 1),       # K below the threshold: no workspace
]


@pytest.mark.parametrize("i8", [True, False])
@pytest.mark.parametrize("case", KSLICE_CASES, ids=lambda c: "n%dc%dh%dw%d_o%dk%d" % c)
def test_conv2d_i8_in_k_slices_equals_the_plain_launch(case, i8, dev):
    n, ic, h, w, oc, k = case
    cid = "kslice-%s" % (case,)
    x = synth.tensor(cid, "x", (n, ic, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (oc, ic, k, k), -127, 127)
    b = synth.tensor(cid, "b", (oc,), -32768, 32768)
    shift = max(1, int(np.ceil(np.log2(ic * k * k * 127 * 127 / 100.0))))
    ch = [("relu",), ("cvm_right_shift", 8, shift)] if i8 else []
    ref = run_chain(oracle.conv2d(x, wt, b, (1, 1), (0, 0), (1, 1), 1), ch)
    xp, wp = hipops.pack_act_i8(T(x, dev)), hipops.pack_weights(T(wt, dev))
    out, used = hipops.conv2d_i8_ws(xp, n, ic, h, w, wp, oc, k, k, T(b, dev), hipops.chain(*ch) if ch else None, i8)
    tiles = (oc + 31) // 32
    assert (used > 0) == (ic * k * k >= 8192 and tiles <= 256)
    if i8:
        eq(act_to_nchw(out, n, oc, 1, 1), ref, "K-sliced conv2d_i8")
    else:
        torch.cuda.synchronize()
        eq(out.cpu().numpy(), ref, "K-sliced conv2d_i8 -> int32")


HEAD_CASES = [
    # n, ic, h, w, oc, k, pad, elements before the slice, elements after it
    (1, 64, 8, 8, 84, 3, 1, 0, 0),        # SSD class head: 4 anchors x 21 classes
    (2, 128, 5, 7, 24, 3, 1, 11, 30),     # two images, a slice in the middle of each image's row
    (3, 32, 4, 4, 126, 1, 0, 5, 0),       # 1x1 head, odd channel count past 96
    (1, 512, 3, 3, 16, 3, 1, 7, 9),       # deep K, very few pixels
]


@pytest.mark.parametrize("case", HEAD_CASES, ids=lambda c: "n%dc%dh%dw%d_o%dk%d" % c[:6])
def test_conv2d_i8_writes_a_detection_head_in_place(case, conv_kernel, dev):
    """conv2d -> chain -> transpose(0,2,3,1) -> reshape -> concatenate, done by one launch that writes
    the pixel-major rows into the concatenated tensor; everything outside the slice stays untouched."""
    n, ic, h, w, oc, k, pd, before, after = case
    cid = "head-%s" % (case,)
    x = synth.tensor(cid, "x", (n, ic, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (oc, ic, k, k), -127, 127)
    b = synth.tensor(cid, "b", (oc,), -32768, 32768)
    ch = [("cvm_right_shift", 8, 9), ("cvm_clip", 8)]
    ref = run_chain(oracle.conv2d(x, wt, b, (1, 1), (pd, pd), (1, 1), 1), ch)
    part = np.ascontiguousarray(ref.transpose(0, 2, 3, 1)).reshape(n, -1)
    stride = before + part.shape[1] + after
    want = np.full((n, stride), 77, np.int32)
    want[:, before:before + part.shape[1]] = part
    out = T(np.full((n, stride), 77, np.int32), dev)
    hipops.conv2d_i8_nhwc(hipops.pack_act_i8(T(x, dev)), n, ic, h, w, hipops.pack_weights(T(wt, dev)), oc, k, k, out, before,
                          stride, T(b, dev), hipops.chain(*ch), padding=(pd, pd))
    torch.cuda.synchronize()
    eq(out.cpu().numpy(), want, "conv2d_i8_nhwc")


HEAD_PAIR_CASES = [
    # n, ic, h, w, oc_a, oc_b, k, pad
    (1, 64, 8, 8, 84, 16, 3, 1),        # SSD: 4 anchors x (21 classes, 4 coordinates)
    (2, 128, 5, 7, 126, 24, 3, 1),      # 6 anchors, two images
    (3, 32, 4, 4, 32, 5, 1, 0),         # the first head ends exactly on a tile boundary
    (1, 512, 3, 3, 16, 126, 3, 1),      # the small head first, deep K
    (1, 96, 16, 16, 200, 70, 3, 1),     # both heads span several tiles
]
HEAD_PAIR_KERNELS = [("auto", None, None), ("lds", None, None)] + [("wave", str(c), None) for c in range(8)] + [("big", None, t) for t in (1, 2, 3)]


@pytest.mark.parametrize("kern", HEAD_PAIR_KERNELS, ids=lambda k: "%s%s%s" % (k[0], "-cfg" + k[1] if k[1] else "", "-tile%d" % k[2] if k[2] else ""))
@pytest.mark.parametrize("case", HEAD_PAIR_CASES, ids=lambda c: "n%dc%dh%dw%d_a%db%dk%d" % c[:7])
def test_two_detection_heads_in_one_launch(case, kern, dev):
    """Two convolutions over the same tensor, each written pixel-major into its own slice of its own concatenated
    tensor, computed as one convolution: equal to the oracle's two, nothing outside the slices touched."""
    n, ic, h, w, oc_a, oc_b, k, pd = case
    cid = "headpair-%s" % (case,)
    x = synth.tensor(cid, "x", (n, ic, h, w), -127, 127)
    wa, wb = synth.tensor(cid, "wa", (oc_a, ic, k, k), -127, 127), synth.tensor(cid, "wb", (oc_b, ic, k, k), -127, 127)
    ba, bb = synth.tensor(cid, "ba", (oc_a,), -32768, 32768), synth.tensor(cid, "bb", (oc_b,), -32768, 32768)
    ch = [("cvm_right_shift", 8, 9), ("cvm_clip", 8)]
    wants, outs = [], []
    for wt, b, before, after in ((wa, ba, 3, 11), (wb, bb, 0, 5)):
        ref = run_chain(oracle.conv2d(x, wt, b, (1, 1), (pd, pd), (1, 1), 1), ch)
        part = np.ascontiguousarray(ref.transpose(0, 2, 3, 1)).reshape(n, -1)
        stride = before + part.shape[1] + after
        want = np.full((n, stride), 77, np.int32)
        want[:, before:before + part.shape[1]] = part
        wants.append((want, before, stride))
        outs.append(T(np.full((n, stride), 77, np.int32), dev))
    split = (oc_a + 31) // 32 * 32
    bias = np.zeros(split + oc_b, np.int32)
    bias[:oc_a], bias[split:] = ba, bb
    if kern[0] != "auto":
        os.environ["CVM_HIP_CONV"] = kern[0]
    if kern[1]:
        os.environ["CVM_HIP_WAVECFG"] = kern[1]
    if kern[2]:
        os.environ["CVM_HIP_TILE"] = "%d,0" % kern[2]
    try:
        hipops.conv2d_i8_nhwc_pair(hipops.pack_act_i8(T(x, dev)), n, ic, h, w, hipops.pack_weights_pair(T(wa, dev), T(wb, dev)), k, k,
                                   outs[0], wants[0][1], wants[0][2], oc_a, outs[1], wants[1][1], wants[1][2], oc_b,
                                   T(bias, dev), hipops.chain(*ch), padding=(pd, pd))
        torch.cuda.synchronize()
    finally:
        os.environ.pop("CVM_HIP_CONV", None)
        os.environ.pop("CVM_HIP_WAVECFG", None)
        os.environ.pop("CVM_HIP_TILE", None)
    eq(outs[0].cpu().numpy(), wants[0][0], "first head, %s" % (kern,))
    eq(outs[1].cpu().numpy(), wants[1][0], "second head, %s" % (kern,))


def test_independent_detection_heads_share_one_launch(dev):
    """Seven head layers of different feature maps (pairs and single heads, 64- and 32-channel tiles, padded and 1x1) recorded
    into one table and launched once: every slice equals the oracle, nothing else is touched."""
    specs = [
        # n, ic, h, w, oc_a, oc_b (0: single head), k, pad
        (1, 256, 16, 16, 84, 16, 3, 1),
        (1, 512, 8, 8, 126, 24, 3, 1),
        (1, 1024, 4, 4, 126, 24, 3, 1),
        (1, 64, 6, 5, 20, 0, 3, 1),
        (1, 128, 2, 2, 84, 16, 3, 1),
        (1, 96, 1, 1, 40, 0, 1, 0),
        (1, 32, 9, 9, 16, 100, 1, 0),
    ]
    grp = hipops.HeadGroup(dev)
    checks = []
    ch = [("cvm_right_shift", 8, 9), ("cvm_clip", 8)]
    for i, (n, ic, h, w, oc_a, oc_b, k, pd) in enumerate(specs):
        cid = "headgroup-%d" % i
        x = synth.tensor(cid, "x", (n, ic, h, w), -127, 127)
        outs = []
        ws, bs = [], []
        for name, oc, before, after in (("a", oc_a, 3 + i, 2), ("b", oc_b, i, 7)):
            if oc == 0:
                continue
            wt = synth.tensor(cid, "w" + name, (oc, ic, k, k), -127, 127)
            b = synth.tensor(cid, "b" + name, (oc,), -32768, 32768)
            ref = run_chain(oracle.conv2d(x, wt, b, (1, 1), (pd, pd), (1, 1), 1), ch)
            part = np.ascontiguousarray(ref.transpose(0, 2, 3, 1)).reshape(n, -1)
            stride = before + part.shape[1] + after
            want = np.full((n, stride), 77, np.int32)
            want[:, before:before + part.shape[1]] = part
            out = T(np.full((n, stride), 77, np.int32), dev)
            outs.append((out, before, stride))
            checks.append((out, want, "%d%s" % (i, name)))
            ws.append(wt)
            bs.append(b)
        xp = hipops.pack_act_i8(T(x, dev))
        if oc_b:
            split = (oc_a + 31) // 32 * 32
            bias = np.zeros(split + oc_b, np.int32)
            bias[:oc_a], bias[split:] = bs[0], bs[1]
            grp.add(xp, n, ic, h, w, hipops.pack_weights_pair(T(ws[0], dev), T(ws[1], dev)), k, k, outs[0][0], outs[0][1], outs[0][2], oc_a,
                    outs[1][0], outs[1][1], outs[1][2], oc_b, T(bias, dev), hipops.chain(*ch), padding=(pd, pd))
        else:
            grp.add(xp, n, ic, h, w, hipops.pack_weights(T(ws[0], dev)), k, k, outs[0][0], outs[0][1], outs[0][2], oc_a,
                    bias=T(bs[0], dev), chain1=hipops.chain(*ch), padding=(pd, pd))
    assert grp.count == len(specs)
    grp.launch()
    for out, want, what in checks:
        eq(out.cpu().numpy(), want, "grouped head " + what)


def test_independent_int8_convolutions_share_one_launch(dev):
    """Convolutions with int8 output that do not depend on one another (a 1x1 layer, a strided projection, a 3x3 layer with a
    residual, a dilated one) recorded into one table and launched once: each equals the oracle's conv2d + chains."""
    specs = [
        # n, ic, h, w, oc, k, stride, pad, dilation, residual
        (1, 64, 14, 14, 64, 1, 1, 0, 1, False),
        (1, 64, 14, 14, 256, 1, 2, 0, 1, False),
        (2, 128, 9, 7, 100, 3, 1, 1, 1, True),
        (1, 32, 12, 12, 40, 3, 1, 2, 2, False),
        (3, 256, 4, 4, 512, 1, 1, 0, 1, True),
    ]
    grp = hipops.HeadGroup(dev)
    checks = []
    ch1, ch2 = [("cvm_right_shift", 8, 11)], [("relu",), ("cvm_right_shift", 8, 1)]
    for i, (n, ic, h, w, oc, k, st, pd, dl, res) in enumerate(specs):
        cid = "convgroup-%d" % i
        x = synth.tensor(cid, "x", (n, ic, h, w), -127, 127)
        wt = synth.tensor(cid, "w", (oc, ic, k, k), -127, 127)
        b = synth.tensor(cid, "b", (oc,), -32768, 32768)
        ref = run_chain(oracle.conv2d(x, wt, b, (st, st), (pd, pd), (dl, dl), 1), ch1)
        rp = None
        if res:
            r = synth.tensor(cid, "r", ref.shape, -127, 127)
            ref = run_chain(oracle.elemwise("elemwise_add", ref, r), ch2)
            rp = hipops.pack_act_i8(T(r, dev))
        out = grp.add_conv_i8(hipops.pack_act_i8(T(x, dev)), n, ic, h, w, hipops.pack_weights(T(wt, dev)), oc, k, k, T(b, dev),
                              hipops.chain(*ch1), rp, hipops.chain(*ch2) if res else None, (st, st), (pd, pd), (dl, dl))
        checks.append((out, ref, n, oc))
    grp.launch(i8=True)
    for i, (out, ref, n, oc) in enumerate(checks):
        eq(act_to_nchw(out, n, oc, ref.shape[2], ref.shape[3]), ref, "grouped int8 convolution %d" % i)


def test_planner_groups_the_projection_with_the_first_layer_of_its_block(dev):
    """At a batch no layer sequence takes, the shortcut projection of a ResNet block moves next to the block's first 1x1
    layer and the two share a launch (one per stage); CVM_HIP_CONVGROUP=0 keeps the graph's order."""
    g, heads = graphgen.resnet50(3, width=32, blocks=(1, 2, 1, 1), size=64, classes=20, config_id="convgroup-r50")
    js, pb = g.build(heads)
    x = synth.tensor("convgroup-r50", "data", g.shape((0, 0)), -127, 127)
    outs, launches = {}, {}
    for mode in ("1", "0"):
        os.environ["CVM_HIP_CONVGROUP"] = mode
        try:
            m = runtime.HipModel(js, pb)
            outs[mode] = [m.inference(x.astype(np.int8).tobytes()) for _ in range(3)]
            launches[mode] = m.launch_counts()[0]
            tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
            m.close()
        finally:
            os.environ.pop("CVM_HIP_CONVGROUP", None)
    assert outs["1"][0] == outs["0"][0] and outs["1"][1] == outs["1"][0] and outs["1"][2] == outs["1"][0]
    assert launches["1"] == launches["0"] - 4, launches
    ref = og.run_graph(js, graphgen.load_params(pb), x)
    got = np.frombuffer(outs["1"][0], np.int32 if tsize == 4 else np.int8).astype(np.int32)
    assert np.array_equal(got, np.concatenate([r.ravel() for r in ref]))


def test_head_group_refuses_few_channel_inputs(dev):
    grp = hipops.HeadGroup(dev)
    x = hipops.pack_act_i8(T(synth.tensor("hg-bad", "x", (1, 16, 4, 4), -127, 127), dev))
    w = hipops.pack_weights(T(synth.tensor("hg-bad", "w", (8, 16, 1, 1), -127, 127), dev))
    out = T(np.zeros((1, 128), np.int32), dev)
    with pytest.raises(CvmHipError):
        grp.add(x, 1, 16, 4, 4, w, 1, 1, out, 0, 128, 8)
    assert grp.count == 0


STEM_CASES = [
    # n, c, h, w, oc, kh, kw, stride, pad
    (2, 3, 32, 32, 64, 7, 7, 2, 3),      # ResNet stem shape, shrunk
    (1, 3, 20, 24, 16, 3, 3, 1, 1),      # VGG / CIFAR stem: 16-byte windows, two filter rows per chunk
    (3, 1, 9, 11, 40, 5, 3, 1, 0),       # one channel, no padding, odd sizes
    (2, 4, 12, 12, 70, 3, 8, 1, 4),      # four channels, the widest window
    (1, 3, 13, 13, 32, 1, 1, 2, 0),      # 1x1, strided
    (2, 2, 8, 30, 24, 4, 2, 3, 1),       # stride 3, asymmetric filter
]


@pytest.mark.parametrize("case", STEM_CASES, ids=lambda c: "n%dc%dh%dw%d_o%dk%dx%ds%dp%d" % c)
def test_conv2d_stem_i8(case, dev):
    """Row-window convolution of the few-channel input layer against the oracle's conv2d + chain."""
    n, c, h, w, oc, kh, kw, st, pd = case
    cid = "stem-%s" % (case,)
    x = synth.tensor(cid, "x", (n, c, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (oc, c, kh, kw), -127, 127)
    b = synth.tensor(cid, "b", (oc,), -32768, 32768)
    conv = oracle.conv2d(x, wt, b, (st, st), (pd, pd), (1, 1), 1)
    stages = [("relu",), ("cvm_right_shift", 8, 9)]
    out32 = hipops.conv2d_stem_i8(T(x, dev), T(wt, dev), T(b, dev), None, False, (st, st), (pd, pd))
    torch.cuda.synchronize()
    eq(out32.cpu().numpy(), conv, "stem int32")
    out8 = hipops.conv2d_stem_i8(T(x, dev), T(wt, dev), T(b, dev), hipops.chain(*stages), True, (st, st), (pd, pd))
    eq(act_to_nchw(out8, n, oc, conv.shape[2], conv.shape[3]), run_chain(conv, stages), "stem int8")


STEM_POOL_CASES = [
    # n, c, h, w, oc, kh, kw, stride, pad, ceil_mode
    (2, 3, 64, 64, 64, 7, 7, 2, 3, False),    # ResNet stem shape, shrunk: 32x32 -> 16x16, two patches by four
    (1, 3, 224, 224, 64, 7, 7, 2, 3, False),  # the real one
    (3, 3, 30, 42, 32, 3, 3, 1, 1, False),    # one channel tile, ragged patches on both axes
    (1, 1, 19, 23, 64, 5, 3, 1, 0, True),     # odd convolution extent, ceil mode: the last windows hang over the edge
    (2, 4, 12, 12, 64, 3, 8, 1, 4, False),    # the widest window
    (1, 3, 9, 9, 64, 3, 3, 2, 1, True),       # 5x5 -> 3x3
]


@pytest.mark.parametrize("case", STEM_POOL_CASES, ids=lambda c: "n%dc%dh%dw%d_o%dk%dx%ds%dp%dceil%d" % c)
def test_conv2d_stem_with_fused_3x3_max_pool(case, dev):
    """Row-window convolution -> requantisation -> max_pool2d(3x3, stride 2, padding 1) in one launch against the oracle."""
    n, c, h, w, oc, kh, kw, st, pd, ceil = case
    cid = "stempool-%s" % (case,)
    x = synth.tensor(cid, "x", (n, c, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (oc, c, kh, kw), -127, 127)
    b = synth.tensor(cid, "b", (oc,), -32768, 32768)
    stages = [("relu",), ("cvm_right_shift", 8, 9)] if n != 3 else [("cvm_right_shift", 8, 9)]   # with and without negative values
    conv = run_chain(oracle.conv2d(x, wt, b, (st, st), (pd, pd), (1, 1), 1), stages)
    ref = oracle.max_pool2d(conv, (3, 3), (2, 2), (1, 1), ceil)
    qh, qw = ref.shape[2:]
    assert hipops.conv2d_stem_pool3_eligible(n, c, h, w, oc, kh, kw, (st, st), (pd, pd), qh, qw)
    out = hipops.conv2d_stem_pool3_i8(T(x, dev), T(wt, dev), T(b, dev), hipops.chain(*stages), (st, st), (pd, pd), qh, qw)
    torch.cuda.synchronize()
    eq(act_to_nchw(out, n, oc, qh, qw), ref, "stem + 3x3 max-pool")


def test_conv2d_stem_pool_eligibility(dev):
    assert not hipops.conv2d_stem_pool3_eligible(1, 3, 32, 32, 16, 3, 3, (1, 1), (1, 1), 16, 16)    # too few output channels
    assert not hipops.conv2d_stem_pool3_eligible(1, 3, 32, 32, 96, 3, 3, (1, 1), (1, 1), 16, 16)    # too many
    assert not hipops.conv2d_stem_pool3_eligible(1, 8, 32, 32, 64, 3, 3, (1, 1), (1, 1), 16, 16)    # not a few-channel input
    assert not hipops.conv2d_stem_pool3_eligible(1, 3, 32, 32, 64, 3, 3, (1, 1), (1, 1), 18, 16)    # a window past the output


def test_planner_folds_the_resnet_head_max_pool(dev):
    """conv 7x7/2 -> relu -> shift -> max_pool 3x3/2 at the head of a ResNet-50 is one launch; CVM_HIP_POOLFUSE=0 keeps two."""
    g, heads = graphgen.resnet50(2, width=64, blocks=(1, 1, 1, 1), size=64, classes=20, config_id="stempool-r50")
    js, pb = g.build(heads)
    x = synth.tensor("stempool-r50", "data", g.shape((0, 0)), -127, 127)
    outs, launches = {}, {}
    for mode in ("1", "0"):
        os.environ["CVM_HIP_POOLFUSE"] = mode
        try:
            m = runtime.HipModel(js, pb)
            outs[mode] = m.inference(x.astype(np.int8).tobytes())
            launches[mode] = m.launch_counts()[0]
            tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
            m.close()
        finally:
            os.environ.pop("CVM_HIP_POOLFUSE", None)
    assert outs["1"] == outs["0"]
    assert launches["1"] == launches["0"] - 1, launches
    ref = og.run_graph(js, graphgen.load_params(pb), x)
    got = np.frombuffer(outs["1"], np.int32 if tsize == 4 else np.int8).astype(np.int32)
    assert np.array_equal(got, np.concatenate([r.ravel() for r in ref]))


@pytest.mark.parametrize("cfg", range(8))
def test_conv2d_stem_i8_every_configuration(cfg, dev):
    """The row-window input layer under every tile / K-split configuration of the wavefront kernel."""
    n, c, h, w, oc, kh, kw, st, pd = (2, 3, 40, 36, 64, 7, 7, 2, 3)
    cid = "stem-cfg"
    x = synth.tensor(cid, "x", (n, c, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (oc, c, kh, kw), -127, 127)
    b = synth.tensor(cid, "b", (oc,), -32768, 32768)
    conv = oracle.conv2d(x, wt, b, (st, st), (pd, pd), (1, 1), 1)
    stages = [("relu",), ("cvm_right_shift", 8, 9)]
    os.environ["CVM_HIP_WAVECFG"] = str(cfg)
    try:
        out32 = hipops.conv2d_stem_i8(T(x, dev), T(wt, dev), T(b, dev), None, False, (st, st), (pd, pd))
        out8 = hipops.conv2d_stem_i8(T(x, dev), T(wt, dev), T(b, dev), hipops.chain(*stages), True, (st, st), (pd, pd))
        torch.cuda.synchronize()
    finally:
        os.environ.pop("CVM_HIP_WAVECFG", None)
    eq(out32.cpu().numpy(), conv, "stem cfg %d int32" % cfg)
    eq(act_to_nchw(out8, n, oc, conv.shape[2], conv.shape[3]), run_chain(conv, stages), "stem cfg %d int8" % cfg)


def test_conv2d_stem_i8_benchmark_shape(dev):
    """ResNet-50's input layer at the benchmark's batch 16 (the shape for which the 64 x 128 tile is chosen
    automatically: 784 workgroups of 64 x 64 tiles for 512 places)."""
    n, c, h, w, oc, kh, kw, st, pd = (16, 3, 224, 224, 64, 7, 7, 2, 3)
    cid = "stem-b16"
    x = synth.tensor(cid, "x", (n, c, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (oc, c, kh, kw), -127, 127)
    b = synth.tensor(cid, "b", (oc,), -32768, 32768)
    conv = oracle.conv2d(x, wt, b, (st, st), (pd, pd), (1, 1), 1)
    stages = [("relu",), ("cvm_right_shift", 8, 9)]
    out8 = hipops.conv2d_stem_i8(T(x, dev), T(wt, dev), T(b, dev), hipops.chain(*stages), True, (st, st), (pd, pd))
    torch.cuda.synchronize()
    eq(act_to_nchw(out8, n, oc, conv.shape[2], conv.shape[3]), run_chain(conv, stages), "stem batch 16 int8")


@pytest.mark.parametrize("cfg", range(8))
@pytest.mark.parametrize("case", [(3, 96, 11, 13, 100, 3, 1, 1, True), (2, 256, 9, 9, 72, 1, 2, 0, False),
                                  (1, 64, 8, 8, 40, 3, 2, 1, True)],
                         ids=lambda c: "n%dc%dh%dw%d_o%dk%ds%dp%d" % c[:8])
def test_conv_wave_kernel_every_configuration(case, cfg, dev):
    """All tile / K-split configurations of the wavefront-private kernel, int8 and int32 output, with a residual."""
    n, ic, h, w, oc, k, st, pd, bias = case
    cid = "wavecfg-%s" % (case,)
    x = synth.tensor(cid, "x", (n, ic, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (oc, ic, k, k), -127, 127)
    b = synth.tensor(cid, "b", (oc,), -32768, 32768) if bias else None
    ch1, ch2 = [("cvm_right_shift", 8, 11)], [("relu",), ("cvm_right_shift", 8, 1)]
    conv = oracle.conv2d(x, wt, b, (st, st), (pd, pd), (1, 1), 1)
    r = synth.tensor(cid, "r", conv.shape, -127, 127)
    ref8 = run_chain(oracle.elemwise("elemwise_add", run_chain(conv, ch1), r), ch2)
    xp, wp, rp = hipops.pack_act_i8(T(x, dev)), hipops.pack_weights(T(wt, dev)), hipops.pack_act_i8(T(r, dev))
    os.environ["CVM_HIP_CONV"] = "wave"
    os.environ["CVM_HIP_WAVECFG"] = str(cfg)
    try:
        out8 = hipops.conv2d_i8(xp, n, ic, h, w, wp, oc, k, k, T(b, dev) if bias else None, hipops.chain(*ch1), rp,
                                hipops.chain(*ch2), True, (st, st), (pd, pd))
        out32 = hipops.conv2d_i8(xp, n, ic, h, w, wp, oc, k, k, T(b, dev) if bias else None, None, None, None, False,
                                 (st, st), (pd, pd))
        torch.cuda.synchronize()
    finally:
        os.environ.pop("CVM_HIP_CONV", None)
        os.environ.pop("CVM_HIP_WAVECFG", None)
    eq(act_to_nchw(out8, n, oc, conv.shape[2], conv.shape[3]), ref8, "wave cfg %d int8" % cfg)
    eq(out32.cpu().numpy(), conv, "wave cfg %d int32" % cfg)


BIG_TILE_CASES = [
    # n, ic, h, w, oc, k, stride, pad, dilation, bias
    (2, 64, 20, 20, 160, 3, 1, 1, 1, True),     # channels past one 128-row tile, ragged pixel count
    (1, 96, 17, 15, 300, 3, 1, 1, 1, True),     # 300 channels: blocks past the packed filter are repeated, never stored
    (3, 32, 9, 9, 64, 5, 2, 2, 1, False),       # 25 taps over one channel block, stride 2
    (1, 128, 12, 12, 128, 3, 1, 2, 2, True),    # dilated
    (2, 256, 7, 7, 96, 1, 1, 0, 1, True),       # 1x1: eight channel blocks per tap
    (1, 64, 33, 31, 40, 3, 1, 0, 1, True),      # no padding, few channels
    (4, 160, 14, 14, 256, 3, 1, 1, 1, True),    # five channel blocks per tap (odd: a step of K straddles two taps)
]


@pytest.mark.parametrize("tile", [1, 2, 3])
@pytest.mark.parametrize("case", BIG_TILE_CASES, ids=lambda c: "n%dc%dh%dw%d_o%dk%ds%dp%dd%d" % c[:9])
def test_large_tile_kernel_every_tile(case, tile, dev):
    """The large-tile kernel (operands through a ring of LDS stages filled by global -> LDS requests), forced for
    layers of any size, for each of its three tiles: int8 output with a residual, and int32 output."""
    n, ic, h, w, oc, k, st, pd, dl, bias = case
    cid = "bigtile-%s" % (case,)
    x = synth.tensor(cid, "x", (n, ic, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (oc, ic, k, k), -127, 127)
    b = synth.tensor(cid, "b", (oc,), -32768, 32768) if bias else None
    ch1, ch2 = [("cvm_right_shift", 8, 12)], [("relu",), ("cvm_right_shift", 8, 1)]
    conv = oracle.conv2d(x, wt, b, (st, st), (pd, pd), (dl, dl), 1)
    r = synth.tensor(cid, "r", conv.shape, -127, 127)
    ref8 = run_chain(oracle.elemwise("elemwise_add", run_chain(conv, ch1), r), ch2)
    xp, wp, rp = hipops.pack_act_i8(T(x, dev)), hipops.pack_weights(T(wt, dev)), hipops.pack_act_i8(T(r, dev))
    os.environ["CVM_HIP_CONV"] = "big"
    os.environ["CVM_HIP_TILE"] = "%d,0" % tile
    try:
        out8 = hipops.conv2d_i8(xp, n, ic, h, w, wp, oc, k, k, T(b, dev) if bias else None, hipops.chain(*ch1), rp,
                                hipops.chain(*ch2), True, (st, st), (pd, pd), (dl, dl))
        out32 = hipops.conv2d_i8(xp, n, ic, h, w, wp, oc, k, k, T(b, dev) if bias else None, None, None, None, False,
                                 (st, st), (pd, pd), (dl, dl))
        torch.cuda.synchronize()
    finally:
        os.environ.pop("CVM_HIP_CONV", None)
        os.environ.pop("CVM_HIP_TILE", None)
    eq(act_to_nchw(out8, n, oc, conv.shape[2], conv.shape[3]), ref8, "large tile %d int8" % tile)
    eq(out32.cpu().numpy(), conv, "large tile %d int32" % tile)


POOL_FUSED_CASES = [
    # n, ic, h, w, oc, k, stride, pad, dilation, bias
    (2, 64, 20, 20, 160, 3, 1, 1, 1, True),     # 3x3 with padding, channels past one tile
    (1, 96, 18, 14, 300, 3, 1, 1, 1, True),     # ragged channel count, windows that straddle pixel tiles
    (3, 32, 9, 9, 64, 5, 2, 2, 1, False),       # stride 2; the 5x5 output has no whole 2x2 windows: refused
    (1, 128, 12, 12, 128, 3, 1, 2, 2, True),    # dilated
    (2, 256, 8, 6, 96, 1, 1, 0, 1, True),       # 1x1 without padding (the identity addressing must not be used)
    (1, 64, 34, 30, 40, 3, 1, 0, 1, True),      # no padding, few channels
    (4, 160, 14, 14, 256, 3, 1, 1, 1, True),    # five channel blocks per tap
    (1, 32, 4, 4, 32, 3, 1, 1, 1, True),        # a single pixel tile, mostly empty
    (2, 64, 16, 16, 160, 3, 1, 1, 1, True),     # 512 pixels: whole 128-pixel wavefront tiles, the maximum between registers
    (1, 128, 32, 32, 96, 3, 1, 1, 1, False),    # 1024 pixels, 96 channels (ragged last 128-channel tile of the large-tile kernel)
    (3, 32, 16, 8, 64, 1, 1, 0, 1, True),       # 384 pixels, 1x1
]
# kernel, wavefront configuration, large tile
POOL_FUSED_KERNELS = [("auto", None, None)] + [("wave", str(c), None) for c in range(8)] + [("big", None, t) for t in (1, 2, 3)]


@pytest.mark.parametrize("kern", POOL_FUSED_KERNELS, ids=lambda k: "%s%s%s" % (k[0], "-cfg" + k[1] if k[1] else "", "-tile%d" % k[2] if k[2] else ""))
@pytest.mark.parametrize("case", POOL_FUSED_CASES, ids=lambda c: "n%dc%dh%dw%d_o%dk%ds%dp%dd%d" % c[:9])
def test_conv2d_with_fused_max_pool(case, kern, dev):
    """conv2d -> requantisation -> max_pool2d(2x2, stride 2) in one launch equals the oracle's three operators, for
    the automatic choice, every configuration of the wavefront kernel and every tile of the large-tile kernel."""
    n, ic, h, w, oc, k, st, pd, dl, bias = case
    cid = "poolfused-%s" % (case,)
    x = synth.tensor(cid, "x", (n, ic, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (oc, ic, k, k), -127, 127)
    b = synth.tensor(cid, "b", (oc,), -32768, 32768) if bias else None
    ch1 = [("relu",), ("cvm_right_shift", 8, 12)] if n % 2 else [("cvm_right_shift", 8, 12)]
    conv = run_chain(oracle.conv2d(x, wt, b, (st, st), (pd, pd), (dl, dl), 1), ch1)
    oh, ow = conv.shape[2:]
    eligible = hipops.conv2d_pool2_eligible(n, ic, h, w, oc, k, k, (st, st), (pd, pd), (dl, dl))
    assert eligible == (oh % 2 == 0 and ow % 2 == 0)
    xp, wp = hipops.pack_act_i8(T(x, dev)), hipops.pack_weights(T(wt, dev))
    if kern[0] != "auto":
        os.environ["CVM_HIP_CONV"] = kern[0]
    if kern[1]:
        os.environ["CVM_HIP_WAVECFG"] = kern[1]
    if kern[2]:
        os.environ["CVM_HIP_TILE"] = "%d,0" % kern[2]
    try:
        if not eligible:
            with pytest.raises(CvmHipError):
                hipops.conv2d_pool2_i8(xp, n, ic, h, w, wp, oc, k, k, T(b, dev) if bias else None, hipops.chain(*ch1),
                                       (st, st), (pd, pd), (dl, dl))
            return
        out = hipops.conv2d_pool2_i8(xp, n, ic, h, w, wp, oc, k, k, T(b, dev) if bias else None, hipops.chain(*ch1),
                                     (st, st), (pd, pd), (dl, dl))
        torch.cuda.synchronize()
    finally:
        os.environ.pop("CVM_HIP_CONV", None)
        os.environ.pop("CVM_HIP_WAVECFG", None)
        os.environ.pop("CVM_HIP_TILE", None)
    ref = oracle.max_pool2d(conv, (2, 2), (2, 2), (0, 0), False)
    eq(act_to_nchw(out, n, oc, oh // 2, ow // 2), ref, "conv + max_pool, %s" % (kern,))


def test_conv2d_with_fused_max_pool_refuses_small_channel_counts(dev):
    assert not hipops.conv2d_pool2_eligible(1, 16, 8, 8, 64, 3, 3, (1, 1), (1, 1))    # input not pixel-blocked
    assert not hipops.conv2d_pool2_eligible(1, 64, 8, 8, 16, 3, 3, (1, 1), (1, 1))    # output not pixel-blocked
    assert not hipops.conv2d_pool2_eligible(1, 64, 9, 8, 64, 3, 3, (1, 1), (1, 1))    # odd extent
    assert hipops.conv2d_pool2_eligible(1, 64, 8, 8, 64, 3, 3, (1, 1), (1, 1))


DW_MFMA_CASES = [
    # n, c, h, w, k, stride, pad, dilation
    (2, 32, 19, 17, 3, 1, 1, 1),
    (1, 96, 16, 16, 3, 2, 1, 1),       # three channel tiles, stride 2
    (1, 256, 8, 8, 5, 1, 2, 1),        # 25 taps
    (1, 40, 9, 9, 3, 1, 0, 1),         # channels padded 40 -> 64, no padding
    (3, 64, 7, 7, 3, 1, 2, 2),         # dilated
    (1, 128, 33, 31, 3, 2, 1, 1),      # ragged pixel count
    (1, 32, 6, 6, 1, 1, 0, 1),         # a single tap
    (16, 1024, 4, 4, 3, 1, 1, 1),      # many tiles, few pixels
]


@pytest.mark.parametrize("cfg", [None, "4", "5", "6"])
@pytest.mark.parametrize("case", DW_MFMA_CASES, ids=lambda c: "n%dc%dh%dw%dk%ds%dp%dd%d" % c)
def test_depthwise_conv2d_mfma_i8(case, cfg, dev):
    """Depthwise convolution as diagonal 32x32 filter blocks on the matrix cores, against the oracle's
    groups == channels convolution, for every configuration of the kernel."""
    n, c, h, w, k, st, pd, dl = case
    assert hipops.depthwise_mfma_eligible(c, k, k)
    cid = "fdwm-%s" % (case,)
    x = synth.tensor(cid, "x", (n, c, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (c, 1, k, k), -127, 127)
    b = synth.tensor(cid, "b", (c,), -3000, 3000)
    stages = [("relu",), ("cvm_right_shift", 8, 10)]
    conv = oracle.conv2d(x, wt, b, (st, st), (pd, pd), (dl, dl), c)
    ref = run_chain(conv, stages)
    xp = hipops.pack_act_i8(T(x, dev))
    wp = hipops.pack_depthwise_weights_mfma(T(wt, dev))
    if cfg is not None:
        os.environ["CVM_HIP_WAVECFG"] = cfg
    try:
        out = hipops.depthwise_conv2d_mfma_i8(xp, n, c, h, w, wp, k, k, T(b, dev), hipops.chain(*stages), True, (st, st),
                                              (pd, pd), (dl, dl))
        out32 = hipops.depthwise_conv2d_mfma_i8(xp, n, c, h, w, wp, k, k, T(b, dev), None, False, (st, st), (pd, pd), (dl, dl))
        torch.cuda.synchronize()
    finally:
        os.environ.pop("CVM_HIP_WAVECFG", None)
    eq(act_to_nchw(out, n, c, ref.shape[2], ref.shape[3]), ref, "depthwise (matrix cores) int8")
    eq(out32.cpu().numpy(), conv, "depthwise (matrix cores) int32")


def test_depthwise_mfma_rejects_unpadded_channels(dev):
    assert not hipops.depthwise_mfma_eligible(5, 3, 3)     # padded to 8, not to a multiple of 32
    assert not hipops.depthwise_mfma_eligible(32, 33, 3)   # filter side beyond the 32-bit tap masks


@pytest.mark.parametrize("case", [(2, 32, 19, 17, 3, 1, 1), (1, 96, 16, 16, 3, 2, 1), (1, 5, 9, 9, 3, 1, 0), (1, 256, 8, 8, 5, 1, 2)],
                         ids=lambda c: "n%dc%dh%dw%dk%ds%dp%d" % c)
def test_depthwise_conv2d_i8(case, dev):
    n, c, h, w, k, st, pd = case
    cid = "fdw-%s" % (case,)
    x = synth.tensor(cid, "x", (n, c, h, w), -127, 127)
    wt = synth.tensor(cid, "w", (c, 1, k, k), -127, 127)
    b = synth.tensor(cid, "b", (c,), -3000, 3000)
    stages = [("relu",), ("cvm_right_shift", 8, 10)]
    ref = run_chain(oracle.conv2d(x, wt, b, (st, st), (pd, pd), (1, 1), c), stages)
    xp = hipops.pack_act_i8(T(x, dev))
    wp = hipops.pack_depthwise_weights(T(wt, dev))
    out = hipops.depthwise_conv2d_i8(xp, n, c, h, w, wp, k, k, T(b, dev), hipops.chain(*stages), True, (st, st), (pd, pd))
    eq(act_to_nchw(out, n, c, ref.shape[2], ref.shape[3]), ref, "depthwise int8")
    out32 = hipops.depthwise_conv2d_i8(xp, n, c, h, w, wp, k, k, T(b, dev), None, False, (st, st), (pd, pd))
    torch.cuda.synchronize()
    eq(out32.cpu().numpy(), oracle.conv2d(x, wt, b, (st, st), (pd, pd), (1, 1), c), "depthwise int32")


@pytest.mark.parametrize("c", [3, 16, 70])
def test_add_i8(c, dev):
    a = synth.tensor("fadd-%d" % c, "a", (2, c, 5, 7), -127, 127)
    b = synth.tensor("fadd-%d" % c, "b", (2, c, 5, 7), -127, 127)
    stages = [("relu",), ("cvm_right_shift", 8, 1)]
    ref = run_chain(oracle.elemwise("elemwise_add", a, b), stages)
    ap, bp = hipops.pack_act_i8(T(a, dev)), hipops.pack_act_i8(T(b, dev))
    eq(act_to_nchw(hipops.add_i8(ap, bp, 2, c, 5, 7, hipops.chain(*stages), True), 2, c, 5, 7), ref, "add int8")
    out = hipops.add_i8(ap, bp, 2, c, 5, 7, None, False)
    torch.cuda.synchronize()
    eq(out.cpu().numpy(), oracle.elemwise("elemwise_add", a, b), "add int32")


@pytest.mark.parametrize("case", [(2, 64, 16, 16, 3, 2, 1, False), (1, 24, 9, 11, 2, 2, 0, False), (1, 8, 10, 10, 3, 2, 1, True)],
                         ids=lambda c: "n%dc%dh%dw%dk%ds%dp%dceil%d" % c)
def test_max_pool2d_i8(case, dev):
    n, c, h, w, k, st, pd, ceil = case
    x = synth.tensor("fpool-%s" % (case,), "x", (n, c, h, w), -128, 127)
    ref = oracle.max_pool2d(x, (k, k), (st, st), (pd, pd), ceil)
    oh, ow = ref.shape[2:]
    out = hipops.max_pool2d_i8(hipops.pack_act_i8(T(x, dev)), n, c, h, w, (k, k), (st, st), (pd, pd), oh, ow)
    eq(act_to_nchw(out, n, c, oh, ow), ref, "max_pool int8")


@pytest.mark.parametrize("c", [10, 64, 2048])
def test_sum_hw_i8(c, dev):
    x = synth.tensor("fsum-%d" % c, "x", (3, c, 7, 7), -127, 127)
    ref = oracle.reduce("sum", x, (2, 3), False, False)
    xp = hipops.pack_act_i8(T(x, dev))
    out = hipops.sum_hw_i8(xp, 3, c, 49, None, False)
    torch.cuda.synchronize()
    eq(out.cpu().numpy(), ref, "sum int32")
    stages = [("cvm_right_shift", 8, 6)]
    out8 = hipops.sum_hw_i8(xp, 3, c, 49, hipops.chain(*stages), True)
    eq(act_to_nchw(out8, 3, c, 1, 1)[:, :, 0, 0], run_chain(ref, stages), "sum int8")


def test_bad_arguments_are_refused(dev):
    x = hipops.pack_act_i8(T(np.zeros((1, 16, 4, 4), np.int32), dev))
    w = hipops.pack_weights(T(np.zeros((16, 16, 3, 3), np.int32), dev))
    from cvm_runtime_amd import CvmHipError
    with pytest.raises(CvmHipError):
        hipops.conv2d_i8(x, 1, 16, 4, 4, w, 16, 3, 3, dilation=(2, 2))      # dilated 3x3 window exceeds the 4x4 input
    bad = hipops.Chain()
    bad.count = 5
    with pytest.raises(CvmHipError):
        hipops.conv2d_i8(x, 1, 16, 4, 4, w, 16, 3, 3, chain1=bad, padding=(1, 1))


@pytest.mark.parametrize("name", ["resnet20", "resnet50", "vgg16", "ssd"])
def test_fused_executor_equals_node_by_node(name, dev):
    """The load-time planner must not change a single output value: run the same
    model with the planner on and off (CVM_HIP_FUSE=0) and compare with the oracle."""
    if name == "resnet20":
        g, heads = graphgen.resnet20_cifar(2)
    elif name == "resnet50":
        g, heads = graphgen.resnet50(2, width=16, size=64, classes=50, config_id="fuse-eq-r50")
    elif name == "vgg16":
        g, heads = graphgen.vgg16(1, size=32, width=8, fc=64, classes=20, config_id="fuse-eq-vgg")
    else:
        g, heads = graphgen.ssd_mobilenet(size=128, alpha=0.25, config_id="fuse-eq-ssd", neg_ids=True)
    js, pb = g.build(heads)
    x = synth.tensor("fuse-eq-" + name, "data", g.shape((0, 0)), -127, 127)
    outs = {}
    for mode in ("1", "0"):
        os.environ["CVM_HIP_FUSE"] = mode
        try:
            m = runtime.HipModel(js, pb)
            outs[mode] = m.inference(x.astype(np.int8).tobytes())
            tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
            m.close()
        finally:
            os.environ.pop("CVM_HIP_FUSE", None)
    assert outs["1"] == outs["0"]
    ref = og.run_graph(js, graphgen.load_params(pb), x)
    got = np.frombuffer(outs["1"], np.int32 if tsize == 4 else np.int8).astype(np.int32)
    assert np.array_equal(got, np.concatenate([r.ravel() for r in ref]))


def test_planner_folds_2x2_max_pools_into_their_convolutions(dev):
    """A VGG whose pooled layers have at least 32 channels: the planner lets those convolutions take their max-pool
    (fewer launches), CVM_HIP_POOLFUSE=0 keeps the two launches, and both equal the oracle."""
    g, heads = graphgen.vgg16(2, size=32, width=32, fc=64, classes=20, config_id="poolfuse-vgg")
    js, pb = g.build(heads)
    x = synth.tensor("poolfuse-vgg", "data", g.shape((0, 0)), -127, 127)
    outs, launches = {}, {}
    for mode in ("1", "0"):
        os.environ["CVM_HIP_POOLFUSE"] = mode
        try:
            m = runtime.HipModel(js, pb)
            outs[mode] = m.inference(x.astype(np.int8).tobytes())
            launches[mode] = m.launch_counts()[0]
            tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
            m.close()
        finally:
            os.environ.pop("CVM_HIP_POOLFUSE", None)
    assert outs["1"] == outs["0"]
    assert launches["1"] == launches["0"] - 5, launches   # all five pools of a VGG-16 follow an eligible convolution here
    ref = og.run_graph(js, graphgen.load_params(pb), x)
    got = np.frombuffer(outs["1"], np.int32 if tsize == 4 else np.int8).astype(np.int32)
    assert np.array_equal(got, np.concatenate([r.ravel() for r in ref]))


def test_planner_groups_the_heads_of_all_feature_maps(dev):
    """All detection heads of an SSD (consecutive, independent steps) share one launch; CVM_HIP_HEADGROUP=0 keeps one per
    feature map."""
    g, heads = graphgen.ssd_mobilenet(size=128, alpha=0.5, config_id="headgroup-ssd", neg_ids=True)
    js, pb = g.build(heads)
    x = synth.tensor("headgroup-ssd", "data", g.shape((0, 0)), -127, 127)
    outs, launches = {}, {}
    for mode in ("1", "0"):
        os.environ["CVM_HIP_HEADGROUP"] = mode
        try:
            m = runtime.HipModel(js, pb)
            outs[mode] = [m.inference(x.astype(np.int8).tobytes()) for _ in range(3)]
            launches[mode] = m.launch_counts()[0]
            tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
            m.close()
        finally:
            os.environ.pop("CVM_HIP_HEADGROUP", None)
    assert outs["1"][0] == outs["0"][0] and outs["1"][1] == outs["1"][0] and outs["1"][2] == outs["1"][0]
    assert launches["1"] == launches["0"] - 6, launches   # seven paired heads in one launch
    ref = og.run_graph(js, graphgen.load_params(pb), x)
    got = np.frombuffer(outs["1"][0], np.int32 if tsize == 4 else np.int8).astype(np.int32)
    assert np.array_equal(got, np.concatenate([r.ravel() for r in ref]))


def test_planner_pairs_the_two_heads_of_a_feature_map(dev):
    """The class head and the box head of each SSD feature map run as one launch; CVM_HIP_HEADPAIR=0 keeps two."""
    g, heads = graphgen.ssd_mobilenet(size=128, alpha=0.5, config_id="headpair-ssd", neg_ids=True)
    js, pb = g.build(heads)
    x = synth.tensor("headpair-ssd", "data", g.shape((0, 0)), -127, 127)
    outs, launches = {}, {}
    os.environ["CVM_HIP_HEADGROUP"] = "0"   # count the launches of the heads themselves
    for mode in ("1", "0"):
        os.environ["CVM_HIP_HEADPAIR"] = mode
        try:
            m = runtime.HipModel(js, pb)
            outs[mode] = [m.inference(x.astype(np.int8).tobytes()) for _ in range(2)]
            launches[mode] = m.launch_counts()[0]
            tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
            m.close()
        finally:
            os.environ.pop("CVM_HIP_HEADPAIR", None)
    os.environ.pop("CVM_HIP_HEADGROUP", None)
    assert outs["1"][0] == outs["0"][0] and outs["1"][1] == outs["1"][0]
    assert launches["1"] == launches["0"] - 7, launches   # seven feature maps
    ref = og.run_graph(js, graphgen.load_params(pb), x)
    got = np.frombuffer(outs["1"][0], np.int32 if tsize == 4 else np.int8).astype(np.int32)
    assert np.array_equal(got, np.concatenate([r.ravel() for r in ref]))


def test_detection_heads_written_in_place_with_other_concat_inputs(dev):
    """Two heads of different feature maps plus an ordinary tensor meet in one concatenate, batch 2.
    The heads are written into the concatenated tensor long before the concatenate node's place in
    the order, with more layers computed in between that reuse freed storage; a second concatenate
    takes a head tensor twice, which must stay with the copy kernels."""
    g = graphgen.GraphBuilder("heads-mixed")
    x = g.var("data", (2, 3, 24, 24), 8)
    f1 = g.conv_relu_q(x, 32, 3, 2, 1)                       # 12x12
    h1 = g.conv_relu_q(f1, 12, 3, 1, 1, relu=False)
    p1 = g.reshape(g.transpose(h1, (0, 2, 3, 1)), (2, 12 * 12 * 3, 4))
    f2 = g.conv_relu_q(g.conv_relu_q(f1, 64, 3, 2, 1), 64, 1)  # 6x6, storage of earlier tensors is free again here
    h2 = g.conv_relu_q(f2, 20, 1, 1, 0, relu=False)
    p2 = g.reshape(g.transpose(h2, (0, 2, 3, 1)), (2, 6 * 6 * 5, 4))
    f3 = g.conv_relu_q(f2, 32, 3, 1, 1)
    extra = g.reshape(g.conv_relu_q(f3, 8, 3, 1, 1, relu=False), (2, 6 * 6 * 2, 4))   # NCHW order: not a head
    cat = g.concat([p1, extra, p2], 1)
    h3 = g.conv_relu_q(f3, 8, 1, 1, 0, relu=False)
    p3 = g.reshape(g.transpose(h3, (0, 2, 3, 1)), (2, 6 * 6 * 2, 4))
    twice = g.concat([p3, p3], 1)
    js, pb = g.build([g.concat([cat, twice], 1)])
    xv = synth.tensor("heads-mixed", "data", (2, 3, 24, 24), -127, 127)
    outs = {}
    for mode in ("1", "0"):
        os.environ["CVM_HIP_FUSE"] = mode
        try:
            m = runtime.HipModel(js, pb)
            outs[mode] = m.inference(xv.astype(np.int8).tobytes())
            if mode == "1":
                labels = m.profile_ops()
                again = m.inference(xv.astype(np.int8).tobytes())     # graph replay gives the same bytes
            tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
            m.close()
        finally:
            os.environ.pop("CVM_HIP_FUSE", None)
    assert "conv2d+head" in labels, labels
    assert outs["1"] == outs["0"] == again
    ref = og.run_graph(js, graphgen.load_params(pb), xv)
    got = np.frombuffer(outs["1"], np.int32 if tsize == 4 else np.int8).astype(np.int32)
    assert np.array_equal(got, np.concatenate([r.ravel() for r in ref]))


def test_storage_shared_by_liveness_is_not_clobbered_by_early_writes(dev):
    """A memory-planned graph lends the storage of a dead tensor to a later one.  A fused step writes
    its chain's final int32 output at the position of the chain's first node, i.e. possibly while the
    previous owner of that storage is still alive: the planner must move such an output to storage
    of its own.  Here `t` (read by `u = abs(t)` between the convolution and the end of its chain)
    shares its storage with the chain's output."""
    import json as _json
    g = graphgen.GraphBuilder("shared-storage")
    x = g.var("data", (1, 32, 6, 6), 8)
    t = g.unary("negative", x)                       # int32 tensor, alive until u is computed
    c, _ = g.conv(x, 32, 3, 1, 1)                    # first node of the fused chain
    u = g.unary("abs", t)                            # still needs t
    q = g.clip8(g.rshift(c, 12))                     # rest of the chain; its output takes over t's storage
    (out,) = g.op("broadcast_add", [q, u], {}, [g.shape(q)])
    js, pb = g.build([out])
    d = _json.loads(js)
    sid = d["attrs"]["storage_id"][1]
    sid[g._eid(q)] = sid[g._eid(t)]
    js = _json.dumps(d)
    xv = synth.tensor("shared-storage", "data", (1, 32, 6, 6), -127, 127)
    outs = {}
    for mode in ("1", "0"):
        os.environ["CVM_HIP_FUSE"] = mode
        try:
            m = runtime.HipModel(js, pb)
            outs[mode] = m.inference(xv.astype(np.int8).tobytes())
            tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
            m.close()
        finally:
            os.environ.pop("CVM_HIP_FUSE", None)
    ref = og.run_graph(js, graphgen.load_params(pb), xv)
    want = np.concatenate([r.ravel() for r in ref])
    for mode in ("0", "1"):
        got = np.frombuffer(outs[mode], np.int32 if tsize == 4 else np.int8).astype(np.int32)
        assert np.array_equal(got, want), "planner %s" % ("on" if mode == "1" else "off")


def test_requantisation_scale_is_folded_into_the_chain(dev):
    """conv2d -> relu -> broadcast_mul(constant scalar) -> cvm_right_shift (the scale-then-shift form of a
    requantisation), the same behind a residual add, and behind the global sum: all folded into the
    producing launch, equal to node-by-node execution and to the oracle."""
    g = graphgen.GraphBuilder("scale-chain")
    x = g.var("data", (2, 3, 20, 20), 8)

    def scaled(v, m, shift, name):
        s = g.param(name, (1,), m, m, int(abs(m)).bit_length() + 1, np.int32)
        (y,) = g.op("broadcast_mul", [v, s], {}, [g.shape(v)])
        return g.clip8(g.rshift(y, shift))

    c1, _ = g.conv(x, 32, 3, 1, 1)
    a = scaled(g.relu(c1), 77, 18, "scale1")
    c2, _ = g.conv(a, 32, 3, 1, 1)
    b = scaled(g.relu(c2), 20, 19, "scale2")
    c3, _ = g.conv(b, 32, 1, 1, 0)
    r = scaled(c3, -100, 19, "scale3")                       # negative scale, no relu
    (added,) = g.op("elemwise_add", [r, a], {}, [g.shape(a)])
    z = scaled(added, 3, 2, "scale4")
    (gap,) = g.op("sum", [z], {"axis": "(2, 3)"}, [(2, 32)])
    out = scaled(gap, 5, 9, "scale5")
    d, _ = g.dense(out, 10)
    js, pb = g.build([d])
    xv = synth.tensor("scale-chain", "data", (2, 3, 20, 20), -127, 127)
    outs = {}
    for mode in ("1", "0"):
        os.environ["CVM_HIP_FUSE"] = mode
        try:
            m = runtime.HipModel(js, pb)
            outs[mode] = m.inference(xv.astype(np.int8).tobytes())
            if mode == "1":
                labels = m.profile_ops()
            tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
            m.close()
        finally:
            os.environ.pop("CVM_HIP_FUSE", None)
    assert "broadcast_mul" not in labels and "cvm_right_shift" not in labels, labels
    assert outs["1"] == outs["0"]
    ref = og.run_graph(js, graphgen.load_params(pb), xv)
    got = np.frombuffer(outs["1"], np.int32 if tsize == 4 else np.int8).astype(np.int32)
    assert np.array_equal(got, np.concatenate([r.ravel() for r in ref]))


@pytest.mark.parametrize("four_d", [False, True])
def test_dense_keeps_values_that_a_non_clipping_shift_leaves_outside_int8(four_d, dev):
    """cvm_right_shift with p + b >= 32 does not clip (elemwise.cc:133-137): precision 8, shift 24 turns
    2^31 - 1 into 128.  dense multiplies the int32 values as they are (ops.cc:53-62), so 128 * w must not
    become -128 * w on the int8 matrix-core path."""
    g = graphgen.GraphBuilder("dense-unsafe-%d" % four_d)
    shape = (3, 16, 2, 2) if four_d else (3, 64)
    x = g.var("data", shape, 32)
    s = g.rshift(x, 24, 8)
    d, _ = g.dense(g.flatten(s) if four_d else s, 24)
    js, pb = g.build([d])
    xv = synth.tensor("dense-unsafe", "data", shape, -2 ** 31, 2 ** 31 - 1)
    xv.flat[:5] = [2 ** 31 - 1, 2 ** 31 - 1, -2 ** 31, 2 ** 31 - 2 ** 23, 2 ** 31 - 2 ** 22]
    ref = og.run_graph(js, graphgen.load_params(pb), xv)
    assert oracle.cvm_right_shift(xv, 8, 24).max() == 128      # the case exists in this input
    want = np.concatenate([r.ravel() for r in ref])
    for mode in ("1", "0"):
        os.environ["CVM_HIP_FUSE"] = mode
        try:
            m = runtime.HipModel(js, pb)
            out = m.inference(xv.astype(np.int32).tobytes())
            tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
            m.close()
        finally:
            os.environ.pop("CVM_HIP_FUSE", None)
        got = np.frombuffer(out, np.int32 if tsize == 4 else np.int8).astype(np.int32)
        assert np.array_equal(got, want), "planner %s" % ("on" if mode == "1" else "off")


def test_dense_int32_kernel_blocks_of_rows(dev):
    """The exact int32 dense kernel (operands wider than 8 bits) with row counts around its row block."""
    for m, k, n in ((1, 70, 5), (8, 64, 9), (9, 130, 33), (17, 257, 12)):
        x = synth.tensor("dense32-%d" % m, "x", (m, k), -40000, 40000)
        w = synth.tensor("dense32-%d" % m, "w", (n, k), -70000, 70000)
        b = synth.tensor("dense32-%d" % m, "b", (n,), -2 ** 30, 2 ** 30)
        ref = oracle.dense(x, w, b)
        y = hipops.dense(T(x, dev), T(w, dev), T(b, dev), operand_bits=32)
        torch.cuda.synchronize()
        eq(y.cpu().numpy(), ref, "dense int32 m=%d" % m)


@pytest.mark.parametrize("case", [(8, 256, 6, 72), (5, 64, 12, 40), (16, 512, 7, 96)])
def test_dense_over_a_whole_map_through_the_flattened_copy(case, dev):
    """flatten -> dense over a 4-D tensor of 8192 or more values per image at a batch of four or more: the map is copied
    once into a tensor whose K chunks are contiguous (cvmhip_flatten_act_i8) and the layer runs as a 1x1 convolution
    over h * w * c channels.  Same bytes as with CVM_HIP_FLATDENSE=0 (the operand gathered from the map as it lies),
    as node by node, and as the oracle; the run has one launch more."""
    n, c, hw, units = case
    g = graphgen.GraphBuilder("flat-dense-%dx%dx%d" % (n, c, hw))
    x = g.var("data", (n, 3, hw, hw), 8)
    y = g.conv_relu_q(x, c, 3, 1, 1)
    y = g.conv_relu_q(y, c, 1)
    d, k = g.dense(g.flatten(y), units)
    d = g.rshift(g.relu(d), graphgen.shift_for(k))
    e, _ = g.dense(d, 10)
    js, pb = g.build([e])
    xv = synth.tensor("flat-dense", "data", (n, 3, hw, hw), -127, 127)
    ref = og.run_graph(js, graphgen.load_params(pb), xv)
    want = np.concatenate([r.ravel() for r in ref])
    launches = {}
    for flat, fuse in (("1", "1"), ("0", "1"), ("1", "0")):
        os.environ["CVM_HIP_FLATDENSE"] = flat
        os.environ["CVM_HIP_FUSE"] = fuse
        try:
            m = runtime.HipModel(js, pb)
            out = m.inference(xv.astype(np.int8).tobytes())
            tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
            launches[(flat, fuse)] = m.launch_counts()[0]
            m.close()
        finally:
            os.environ.pop("CVM_HIP_FLATDENSE", None)
            os.environ.pop("CVM_HIP_FUSE", None)
        got = np.frombuffer(out, np.int32 if tsize == 4 else np.int8).astype(np.int32)
        assert np.array_equal(got, want), "flattened copy %s, planner %s" % (flat, fuse)
    assert launches[("1", "1")] == launches[("0", "1")] + 1, launches


def test_flatten_act_i8(dev):
    """the copy itself: channel p * c + ch of image i in the result is channel ch of pixel p of image i"""
    n, c, hw = 5, 96, 11
    x = synth.tensor("flatten-act", "x", (n, c, hw, 1), -128, 127)
    yp = hipops.flatten_act_i8(hipops.pack_act_i8(T(x, dev)), n, c, hw)
    got = act_to_nchw(yp, n, hw * c, 1, 1).reshape(n, hw, c)          # (image, pixel, channel)
    eq(got, x.reshape(n, c, hw).transpose(0, 2, 1), "flatten_act_i8")
    with pytest.raises(CvmHipError):
        hipops.flatten_act_i8(hipops.pack_act_i8(T(x[:, :40], dev)), n, 40, hw)   # channels not a multiple of 32
