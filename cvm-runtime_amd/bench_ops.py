"""Bandwidth-bound operators at the shapes of the benchmark configurations:
achieved GB/s against the HBM peak, from algorithmic bytes (int32 operator
contract: 4 bytes per input and output element; the fused int8 forms move one
byte per element) over the device time of repeated launches.

Used by `bench.py --suite ops`; one result dict per operator."""
import torch

from . import hipops, synth

HBM_PEAK_GBS = 8000.0


def _timed(fn, reps):
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / reps   # microseconds per call


def _rand(shape, lo, hi, dev, dtype=torch.int32):
    return torch.randint(lo, hi + 1, shape, dtype=dtype, device=dev)


def run(reps=20):
    dev = torch.device("cuda:0")
    rows = []

    def add(name, shape_note, nbytes, fn, r=reps):
        us = _timed(fn, r)
        gbs = nbytes / us / 1e3
        rows.append({"op": name, "shape": shape_note, "algorithmic_bytes": int(nbytes), "us_per_call": us,
                     "achieved_GBps": gbs, "frac_of_hbm_peak": gbs / HBM_PEAK_GBS})

    # ---- int32 operator contract (what an un-fused node or a plug-in caller runs)
    act = (16, 256, 56, 56)                      # ResNet-50 batch 16, stage-1 output
    n_act = 16 * 256 * 56 * 56
    x = _rand(act, -30000, 30000, dev)
    y = _rand(act, -30000, 30000, dev)
    out = torch.empty_like(x)
    add("relu", "16x256x56x56 int32", 8 * n_act, lambda: hipops.relu(x, out=out))
    add("cvm_right_shift p8 b8", "16x256x56x56 int32", 8 * n_act, lambda: hipops.cvm_right_shift(x, 8, 8, out=out))
    add("cvm_clip p8", "16x256x56x56 int32", 8 * n_act, lambda: hipops.cvm_clip(x, 8, out=out))
    add("elemwise_add", "16x256x56x56 int32", 12 * n_act, lambda: hipops.elemwise("elemwise_add", x, y, out=out))
    s = _rand((1,), 3, 3, dev)
    add("broadcast_mul by scalar", "16x256x56x56 int32", 8 * n_act, lambda: hipops.broadcast("broadcast_mul", x, s))
    px = _rand((16, 64, 112, 112), -127, 127, dev)
    n_in, n_out = 16 * 64 * 112 * 112, 16 * 64 * 56 * 56
    add("max_pool2d 3x3 s2 p1", "16x64x112x112 int32", 4 * (n_in + n_out), lambda: hipops.max_pool2d(px, (3, 3), (2, 2), (1, 1)))
    vx = _rand((16, 64, 224, 224), -127, 127, dev)
    add("max_pool2d 2x2 s2", "16x64x224x224 int32 (VGG-16)", 4 * (vx.numel() + vx.numel() // 4),
        lambda: hipops.max_pool2d(vx, (2, 2), (2, 2), (0, 0)))
    del vx
    gx = _rand((16, 2048, 7, 7), -127, 127, dev)
    add("sum axis (2,3)", "16x2048x7x7 int32", 4 * (gx.numel() + 16 * 2048), lambda: hipops.reduce("sum", gx, (2, 3)))
    tx = _rand((1, 126, 64, 64), -127, 127, dev)
    add("transpose (0,2,3,1)", "1x126x64x64 int32 (SSD head)", 8 * tx.numel(), lambda: hipops.transpose(tx, (0, 2, 3, 1)))

    # ---- detection (config 5): 24 564 anchors, score threshold 10, IoU 45, top_k 400
    import numpy as np
    b = np.zeros((1, 24564, 6), np.int32)
    b[:, :, 0] = synth.tensor("bench-ops", "id", (1, 24564), 0, 20)
    b[:, :, 1] = synth.tensor("bench-ops", "score", (1, 24564), -127, 127)
    xy = np.sort(synth.tensor("bench-ops", "xy", (1, 24564, 2, 2), 0, 512), axis=2)
    b[:, :, 2:] = xy.reshape(1, 24564, 4)
    bx = torch.from_numpy(b).to(dev)
    nb = bx.numel()
    add("get_valid_counts thr 10", "1x24564x6 int32", 4 * 2 * nb + 4, lambda: hipops.get_valid_counts(bx, 10))
    vc, rows_sorted = hipops.get_valid_counts(bx, 10)
    ny = torch.empty_like(rows_sorted)

    def nms():
        hipops.non_max_suppression(rows_sorted.clone(), vc, ny, 45, False, 400)
    clone_us = _timed(lambda: rows_sorted.clone(), reps)
    add("non_max_suppression iou 45 top_k 400", "1x24564x6 int32, %d valid rows" % int(vc.item()), 4 * 2 * nb, nms)
    rows[-1]["us_per_call"] -= clone_us          # the input is mutated by the call, so each repetition works on a fresh copy
    rows[-1]["achieved_GBps"] = rows[-1]["algorithmic_bytes"] / rows[-1]["us_per_call"] / 1e3
    rows[-1]["frac_of_hbm_peak"] = rows[-1]["achieved_GBps"] / HBM_PEAK_GBS

    # the same rows without top_k: ranked by the stable radix sort (12 launches), then every valid row is a candidate of the
    # greedy walk, whose time grows with the square of their number -- a few repetitions are enough
    def nms_all():
        hipops.non_max_suppression(rows_sorted.clone(), vc, ny, 45, False, -1)
    add("non_max_suppression iou 45 without top_k", "1x24564x6 int32, %d valid rows" % int(vc.item()), 4 * 2 * nb, nms_all, r=3)

    # ---- fused int8 forms (what the graph executor runs): one byte per element
    xa = hipops.pack_act_i8(_rand(act, -127, 127, dev))
    xb = hipops.pack_act_i8(_rand(act, -127, 127, dev))
    ch = hipops.chain(("cvm_right_shift", 8, 1))
    oa = torch.zeros_like(xa)
    add("add_i8 + right_shift", "16x256x56x56 int8", 3 * n_act, lambda: hipops.add_i8(xa, xb, 16, 256, 56, 56, ch, out=oa))
    pa = hipops.pack_act_i8(_rand((16, 64, 112, 112), -127, 127, dev))
    po = hipops.max_pool2d_i8(pa, 16, 64, 112, 112, (3, 3), (2, 2), (1, 1), 56, 56)
    add("max_pool2d_i8 3x3 s2 p1", "16x64x112x112 int8", n_in + n_out,
        lambda: hipops.max_pool2d_i8(pa, 16, 64, 112, 112, (3, 3), (2, 2), (1, 1), 56, 56, out=po))
    ga = hipops.pack_act_i8(_rand((16, 2048, 7, 7), -127, 127, dev))
    gc = hipops.chain(("cvm_right_shift", 8, 5))
    go = hipops.sum_hw_i8(ga, 16, 2048, 49, gc)
    add("sum_hw_i8 + right_shift", "16x2048x7x7 int8", 16 * 2048 * 49 + 16 * 2048 * 4,
        lambda: hipops.sum_hw_i8(ga, 16, 2048, 49, gc, out=go))
    return rows
