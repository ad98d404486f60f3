#!/usr/bin/env python3
"""Headline benchmark: images/s of the int8 ResNet-50 v1 graph (224x224) on one MI355X.

A step is one pass of the graph (`CvmRuntime::Run`) over one batch that already
sits in HBM.  The line printed at the end carries the whole-job throughput, the
roofline position of the dominant kernel (the i8 MFMA implicit GEMM, timed with
HIP events on the runtime's own stream in a second pass over the same steps) and the
reference CPU runtime timed on this machine's host cores on a bounded sample.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 16]
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_I8_TOPS = 5000.0   # MI355X dense int8 MFMA peak, TOP/s
# HBM bytes per launch of the dominant kernel of a batch-16 workload, from the FETCH_SIZE and WRITE_SIZE counter
# passes summarised in the named file under profiles/ (a counter pass cannot run inside this program, so the
# figures are carried here; each is reported only for the workload and kernel it was measured on)
# The third field is the first 16 hex digits of the SHA-256 of the kernels' source file as it was when the counters were
# read: a figure is only reported while that file is unchanged, otherwise `traffic` is null (measured figures go stale).
TRAFFIC_BYTES_PER_LAUNCH = {
    ("resnet50", "k_conv_seq", 16): (530.9e6, "profiles/k_conv_seq_resnet50_b16_traffic.txt", "a1e72eef549f2e45"),
    ("vgg16", "k_conv_big", 16): (28.7e6, "profiles/k_conv_big_vgg16_b16_traffic.txt", "a1e72eef549f2e45"),
}
KERNEL_SOURCE = os.path.join(ROOT, "cvm-runtime_amd", "csrc", "conv_mfma.hip")


def kernel_source_hash():
    import hashlib
    try:
        return hashlib.sha256(open(KERNEL_SOURCE, "rb").read()).hexdigest()[:16]
    except OSError:
        return None


def dominant_conv(kt, wall_s, steps):
    """From the per-kernel event-pair totals of `steps` steps: the implicit-GEMM kernel that takes most of the step, its
    average launch duration with the cost of an event pair taken off, and the figures derived from it."""
    n_timed = sum(v["launches"] for v in kt.values())
    pair_cost_us = max(0.0, (sum(v["ms"] for v in kt.values()) * 1e3 - wall_s * 1e6) / max(n_timed, 1))
    convs = {k: v for k, v in kt.items() if k in ("k_conv_wave", "k_conv_igemm", "k_conv_seq", "k_conv_big", "k_conv_group", "k_stem_pool")}
    dom = max(convs, key=lambda k: convs[k]["ms"]) if convs else "k_conv_wave"
    conv = convs.get(dom, {"launches": 0, "ms": 0.0, "work": 0.0})
    launches = max(conv["launches"], 1)
    raw_avg_s = conv["ms"] / 1e3 / launches
    avg_s = max(raw_avg_s - pair_cost_us * 1e-6, 1e-9)
    return {"kernel": dom, "convs": convs, "conv": conv, "pair_cost_us": pair_cost_us, "raw_avg_s": raw_avg_s, "avg_s": avg_s,
            "ops_per_launch": conv["work"] / launches}


def side_workload(pkg, L, name, batch, steps, warmup, check):
    """A second benchmark configuration measured in the same process, the same way as the headline one (input resident in
    HBM, `steps` timed runs, then the same steps with an event pair around every launch): VGG-16 at batch 16 is where the
    large-tile kernel runs, so its fraction of the matrix-core peak is in the driver's line too.  With `check` the first
    image of the timed batch is compared with the CPU runtime's result for it."""
    import numpy as np
    import torch
    from cvm_runtime_amd import graphgen, runtime, synth
    g, heads = {"vgg16": graphgen.vgg16}[name](batch)
    js, pb = g.build(heads)
    x = synth.tensor("bench", "data", g.shape((0, 0)), -127, 127).astype(np.int8)
    model = runtime.HipModel(js, pb)
    counts = model.launch_counts()
    model.set_input(x.tobytes())
    model.time_run(max(warmup, 1))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    model.time_run(steps)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    L.cvmhip_kernel_timing_begin()
    model.time_run(steps)
    torch.cuda.synchronize()
    buf = ctypes.create_string_buffer(1 << 16)
    pkg.check(L.cvmhip_kernel_timing_end(buf, len(buf)))
    kt = json.loads(buf.value.decode())
    raw = model.get_output()
    tsize = runtime.CVMAPIGetOutputTypeSize(model.net)
    model.close()
    d = dominant_conv(kt, wall, steps)
    achieved = d["ops_per_launch"] / d["avg_s"] / 1e12
    out = {"workload": "cfg4 VGG-16 quantised graph, batch %d, 3x224x224 int8, random int8 weights" % batch,
           "ms_per_step": wall / steps * 1e3, "images_per_s": batch * steps / wall, "kernel_launches_per_step": counts[0],
           "kernel": d["kernel"], "launches_per_step": d["conv"]["launches"] / steps, "avg_launch_us": d["avg_s"] * 1e6,
           "algorithmic_gop_per_launch": d["ops_per_launch"] / 1e9, "achieved_tops": achieved, "frac": achieved / PEAK_I8_TOPS,
           "all_conv_dense_tops": sum(v["work"] for v in d["convs"].values()) /
                                  max(sum(v["ms"] / 1e3 - v["launches"] * d["pair_cost_us"] * 1e-6 for v in d["convs"].values()), 1e-9) / 1e12}
    if check:
        g1, h1 = {"vgg16": graphgen.vgg16}[name](1)
        js1, pb1 = g1.build(h1)
        _, want = cpu_baseline(js1, pb1, x[:1].astype(np.int32), 0.0)
        per_image = len(raw) // batch
        got = np.frombuffer(raw[:per_image], np.int32 if tsize == 4 else np.int8).astype(np.int32)
        out["parity_checked"] = bool(got.shape == want.shape and np.array_equal(got, want))
    return out


def cpu_baseline(js1, pb1, x1, budget_s=20.0):
    """Reference CPU runtime (oracle/_ref, built from the reference sources) on the first image of the timed
    batch, as a batch-1 model of the same graph; falls back to the C restatement when the reference build is
    absent.  Checker code is only timed here, never used to produce the GPU result.  Returns the baseline
    object and the int32 values the CPU runtime computed for that image (the parity check of the timed
    configuration compares the GPU's first image with them)."""
    import numpy as np
    import oracle
    import oracle.graph as og
    from cvm_runtime_amd import graphgen
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    n = 0
    if oracle.have_ref():
        L = og.ref_lib()
        net = ctypes.c_void_p()
        gj = js1.encode()
        rc = L.CVMAPILoadModel(ctypes.c_char_p(gj), len(gj), ctypes.c_char_p(pb1), len(pb1), ctypes.byref(net), 0, 0)
        assert rc == 0
        size, tsize = ctypes.c_ulonglong(), ctypes.c_ulonglong()
        L.CVMAPIGetOutputLength(net, ctypes.byref(size))
        L.CVMAPIGetOutputTypeSize(net, ctypes.byref(tsize))
        out = ctypes.create_string_buffer(size.value)
        xb = x1.astype(np.int8).tobytes()
        assert L.CVMAPIInference(net, ctypes.c_char_p(xb), len(xb), out) == 0   # warm-up, and the values to compare
        want = np.frombuffer(out.raw, np.int32 if tsize.value == 4 else np.int8).astype(np.int32)
        t0 = time.perf_counter()
        while True:
            L.CVMAPIInference(net, ctypes.c_char_p(xb), len(xb), out)
            n += 1
            dt = time.perf_counter() - t0
            if dt > budget_s or n >= 1000:
                break
        L.CVMAPIFreeModel(net)
        kind = "reference"
    else:
        params = graphgen.load_params(pb1)
        want = np.concatenate([r.ravel() for r in og.run_graph(js1, params, x1)]).astype(np.int32)
        t0 = time.perf_counter()
        while True:
            og.run_graph(js1, params, x1)
            n += 1
            dt = time.perf_counter() - t0
            if dt > budget_s or n >= 1000:
                break
        kind = "port"
    return {"value": n / dt, "unit": "images/s", "cores": cores, "kind": kind,
            "sample": "%d batch-1 CVMAPIInference calls of the same graph on the first image of the timed batch, %.1f s" % (n, dt)}, want


def layer_table(args, pkg, L, model, title):
    """One row per launch of a step, in launch order.  Durations: HIP event pairs around every launch (minus
    the cost of a pair, calibrated as in the headline run), or -- given the kernel trace of a rocprofv3 run of
    this same command -- the median over the steps of the traced duration of the launch at that position.
    Floors: algorithmic operations at 5 POP/s, algorithmic bytes at 8 TB/s, and the duration of a launch that
    does nothing (a 256-byte copy kernel, launched 50 times back to back after the steps)."""
    import csv
    import statistics
    import torch
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    model.time_run(args.steps)
    torch.cuda.synchronize()
    plain_us = (time.perf_counter() - t0) / args.steps * 1e6
    L.cvmhip_kernel_timing_begin()
    model.time_run(args.steps)
    torch.cuda.synchronize()
    buf = ctypes.create_string_buffer(1 << 24)
    pkg.check(L.cvmhip_kernel_timing_end_launches(buf, len(buf)))
    launches = json.loads(buf.value.decode())
    per_step = len(launches) // args.steps
    assert per_step * args.steps == len(launches), "launch count is not a multiple of the step count"
    step = launches[:per_step]
    pair_us = [statistics.median(launches[k * per_step + i]["ms"] * 1e3 for k in range(args.steps)) for i in range(per_step)]
    pair_cost = max(0.0, (sum(pair_us) - plain_us) / per_step)
    dur = [max(u - pair_cost, 0.0) for u in pair_us]
    source = "event pairs minus %.2f us per pair" % pair_cost
    # the launch that does nothing
    a = torch.zeros(64, dtype=torch.int32, device="cuda")
    b = torch.zeros(64, dtype=torch.int32, device="cuda")
    for _ in range(50):
        pkg.check(L.cvmhip_copy_kernel(ctypes.c_void_p(b.data_ptr()), ctypes.c_void_p(a.data_ptr()), ctypes.c_size_t(256), None))
    torch.cuda.synchronize()
    empty_us = None
    if args.trace:
        rows = sorted(csv.DictReader(open(args.trace)), key=lambda r: int(r["Start_Timestamp"]))
        base = lambda n: n.split("(")[0].split("<")[0].replace("void ", "").split("::")[-1]
        seq = []
        for r in rows:
            name, us = base(r["Kernel_Name"]), (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3
            if name == "k_slices_finish" and seq:     # second kernel of a K-sliced convolution: one launch of the table
                seq[-1] = (seq[-1][0], seq[-1][1] + us)
            else:
                seq.append((name, us))
        want = [e["kernel"] for e in step]
        alias = {"k_max_pool_i8": ("k_max_pool_i8", "k_max_pool_i8x16"), "k_conv_group": ("k_conv_group", "k_conv_group8")}
        same = lambda got, w: got == w or got in alias.get(w, ())
        hits, i = [], 0
        while i + per_step <= len(seq):
            if all(same(seq[i + j][0], want[j]) for j in range(per_step)):
                hits.append(i)
                i += per_step
            else:
                i += 1
        assert hits, "the trace holds no run of launches that matches a step"
        dur = [statistics.median(seq[h + j][1] for h in hits) for j in range(per_step)]
        source = "rocprofv3 kernel trace, median of %d steps" % len(hits)
        empties = [d for n, d in seq if n == "k_copy16"]
        if empties:
            empty_us = statistics.median(empties[-50:])
    print("# %s, batch %d, one launch per layer (layer-sequence launches switched off): %d launches per step, %.1f us per step "
          "without instrumentation" % (title, args.batch, per_step, plain_us))
    print("# durations: %s; sum %.1f us" % (source, sum(dur)))
    if empty_us is not None:
        print("# a launch that does nothing (256-byte copy kernel): %.2f us in the same trace" % empty_us)
    print("# floors: ops / 5 POP/s, bytes / 8 TB/s, the launch that does nothing; excess = duration - the largest floor")
    print("%3s %-14s %-78s %8s %8s %7s %7s %7s %7s %7s %7s" % ("#", "kernel", "launch", "GOP", "MB", "us", "mfma_us", "hbm_us", "TOP/s", "TB/s",
                                                                "excess"))
    tot_ops = tot_bytes = 0.0
    excess = []
    for i, (e, u) in enumerate(zip(step, dur)):
        is_conv = e["kernel"].startswith("k_conv") or e["kernel"] == "k_stem_pool"
        ops = e["work"] if is_conv else 0.0
        byts = e["bytes"] if is_conv else e["work"]
        tot_ops += ops
        tot_bytes += byts
        floor = max(ops / 5e15 * 1e6, byts / 8e12 * 1e6, empty_us or 0.0)
        excess.append((u - floor, i, e["kernel"], e["desc"]))
        print("%3d %-14s %-78s %8.3f %8.2f %7.2f %7.2f %7.2f %7.0f %7.2f %7.2f" % (
            i, e["kernel"], e["desc"][:78], ops / 1e9, byts / 1e6, u, ops / 5e15 * 1e6, byts / 8e12 * 1e6,
            ops / max(u, 1e-3) / 1e6, byts / max(u, 1e-3) / 1e6, u - floor))
    print("# step: %.1f GOP = %.1f us at 5 POP/s; %.1f MB = %.1f us at 8 TB/s" % (
        tot_ops / 1e9, tot_ops / 5e15 * 1e6, tot_bytes / 1e6, tot_bytes / 8e12 * 1e6))
    print("# sum of the floors %.1f us; the ten launches furthest above their floor:" % (sum(dur) - sum(x[0] for x in excess)))
    for x in sorted(excess, reverse=True)[:10]:
        print("#   %6.2f us  %3d %-14s %s" % (x[0], x[1], x[2], x[3][:78]))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--workload", choices=("resnet50", "vgg16", "resnet20", "ssd512"), default="resnet50",
                    help="resnet50 (default) is the headline configuration; the others are the remaining benchmark "
                         "configurations, measured the same way (ssd512 always runs at batch 1)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-vgg", action="store_true",
                    help="skip the VGG-16 batch-16 figures that the headline configuration reports beside its own")
    ap.add_argument("--no-batch1", action="store_true",
                    help="skip the batch-1 figures of the same graph (keeps a profiler's kernel statistics to the timed model)")
    ap.add_argument("--no-two-models", action="store_true",
                    help="skip the side measurement with two models in flight (keeps a profiler's kernel statistics to one model)")
    ap.add_argument("--suite", choices=("model", "ops"), default="model",
                    help="model: the headline line (default); ops: one JSON line per bandwidth-bound operator at the "
                         "shapes of the configurations, achieved GB/s against the 8 TB/s HBM peak")
    ap.add_argument("--layers", action="store_true",
                    help="print one row per launch of a step instead of the headline line: what the launch is, its "
                         "duration, and its floors (matrix-core peak, HBM peak, an empty launch)")
    ap.add_argument("--trace", default=None,
                    help="with --layers: kernel_trace.csv of a `rocprofv3 --kernel-trace` run of this same command; "
                         "the durations of the table are then the medians of the trace instead of event pairs")
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="also launch a plain copy kernel of known size (256 MiB read + 256 MiB written, 5 times): "
                         "under `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` its counter reading gives the scale of the counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend runs on exactly one GPU (got --gpus %d); the path shards by batch "
                 "with no exchange step, each GPU running this same program on its share" % args.gpus)

    import numpy as np
    import torch
    import __graft_entry__
    pkg = __graft_entry__.load_package()
    from cvm_runtime_amd import graphgen, runtime, synth
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    L = pkg.lib()

    if args.suite == "ops":
        from cvm_runtime_amd import bench_ops
        for row in bench_ops.run(max(args.steps, 5)):
            print(json.dumps(row))
        return

    if args.workload == "ssd512":
        args.batch = 1
    builders = {"resnet50": lambda: graphgen.resnet50(args.batch), "vgg16": lambda: graphgen.vgg16(args.batch),
                "resnet20": lambda: graphgen.resnet20_cifar(args.batch), "ssd512": graphgen.ssd_mobilenet}
    titles = {"resnet50": "cfg3 ResNet-50 v1 quantised graph, batch %d, 3x224x224 int8, random int8 weights",
              "vgg16": "cfg4 VGG-16 quantised graph, batch %d, 3x224x224 int8, random int8 weights",
              "resnet20": "cfg2 ResNet-20 v2 CIFAR quantised graph, batch %d, 3x32x32 int8, random int8 weights",
              "ssd512": "cfg5 SSD-512 MobileNet-1.0 quantised detector with get_valid_counts and NMS, batch %d, 3x512x512 int8"}
    names = {"resnet50": "ResNet-50 (224x224)", "vgg16": "VGG-16 (224x224)", "resnet20": "ResNet-20 (32x32)",
             "ssd512": "SSD-512 MobileNet-1.0"}
    g, heads = builders[args.workload]()
    js, pb = g.build(heads)
    gmac = g.macs / 1e9
    x = synth.tensor("bench", "data", g.shape((0, 0)), -127, 127).astype(np.int8)
    if args.layers:
        os.environ["CVM_HIP_SEQ"] = "0"     # the table is about single layers: one launch each
    model = runtime.HipModel(js, pb)
    launch_counts = model.launch_counts()
    model.set_input(x.tobytes())            # input resident in HBM from here on
    model.time_run(max(args.warmup, 1))
    torch.cuda.synchronize()

    if args.layers:
        layer_table(args, pkg, L, model, names[args.workload])
        model.close()
        return

    # timed region: exactly `steps` graph runs, nothing else on the stream
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dev_ms = model.time_run(args.steps)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    # the same steps again with a HIP event pair around every launch on the
    # runtime's stream: per-kernel durations for the roofline object.  The event
    # pairs slow the queue down, so this pass never feeds `value`.
    L.cvmhip_kernel_timing_begin()
    t0 = time.perf_counter()
    model.time_run(args.steps)
    torch.cuda.synchronize()
    wall_events = time.perf_counter() - t0
    buf = ctypes.create_string_buffer(1 << 16)
    pkg.check(L.cvmhip_kernel_timing_end(buf, len(buf)))
    kt = json.loads(buf.value.decode())
    raw = model.get_output()
    out_tsize = runtime.CVMAPIGetOutputTypeSize(model.net)
    out = np.frombuffer(raw + b"\0" * (-len(raw) % 4), np.int32)

    # two models of the same graph in flight (two nets on two host threads, each with its own stream, as the
    # reference's threading rules allow): how far one batch-16 model is from filling the chip.  Reported
    # beside the headline, never as it.
    two_models_rate = None
    if not args.no_two_models:
        import threading
        second = runtime.HipModel(js, pb)
        second.set_input(x.tobytes())
        second.time_run(max(args.warmup, 1))
        # (the first model too: with a second model alive it leaves its layer-sequence launch for one launch per layer,
        # and the first run after that change captures its graph anew)
        model.time_run(max(args.warmup, 1))
        torch.cuda.synchronize()
        pair = [threading.Thread(target=m.time_run, args=(args.steps,)) for m in (model, second)]
        t0 = time.perf_counter()
        for t in pair:
            t.start()
        for t in pair:
            t.join()
        torch.cuda.synchronize()
        two_models_rate = 2 * args.batch * args.steps / (time.perf_counter() - t0)
        second.close()

    # whole CVMAPIInference (host input -> H2D -> run -> D2H), reported beside the headline, never as it
    xb = x.tobytes()
    model.inference(xb)
    t0 = time.perf_counter()
    n_api = max(args.steps // 5, 3)
    for _ in range(n_api):
        model.inference(xb)
    api_s = (time.perf_counter() - t0) / n_api
    model.close()

    if args.traffic_calibration:
        a = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        b = torch.empty_like(a)
        for _ in range(5):
            pkg.check(L.cvmhip_copy_kernel(ctypes.c_void_p(b.data_ptr()), ctypes.c_void_p(a.data_ptr()),
                                           ctypes.c_size_t(a.numel()), None))
        torch.cuda.synchronize()

    # The implicit-GEMM kernels (same arithmetic, chosen per layer; k_conv_seq is a run of layers in one launch);
    # the roofline object is about the one that takes more of the step.  An event pair makes a launch look longer than it is.  Every launch
    # of a step is timed and the un-instrumented step is GPU-bound with its kernels back to back, so the
    # cost of one pair is (sum of all pair times - un-instrumented step time) / launches; it is taken off
    # every launch.  The rocprofv3 kernel trace under profiles/ measures the same durations directly.
    d = dominant_conv(kt, wall, args.steps)
    pair_cost_us, convs, dom, conv = d["pair_cost_us"], d["convs"], d["kernel"], d["conv"]
    pair_us = {"empty_us": pair_cost_us}
    ops_per_launch, raw_avg_s, avg_s = d["ops_per_launch"], d["raw_avg_s"], d["avg_s"]
    achieved = ops_per_launch / avg_s / 1e12
    all_ops = sum(v["work"] for v in convs.values())
    all_s = sum(v["ms"] / 1e3 - v["launches"] * pair_us["empty_us"] * 1e-6 for v in convs.values())
    step_s = wall / args.steps
    traffic = TRAFFIC_BYTES_PER_LAUNCH.get((args.workload, dom, args.batch), (None, None, None))
    source_hash = kernel_source_hash()
    traffic_note = None
    if traffic[0] is not None:
        if traffic[2] == source_hash:
            traffic_note = ("recorded from the FETCH_SIZE / WRITE_SIZE counter passes summarised in " + traffic[1] +
                            " (kernel source " + str(source_hash) + "), not measured by this run")
        else:
            traffic_note = ("none reported: the kernels' source (" + str(source_hash) + ") has changed since the counter passes of " +
                            traffic[1] + " (" + str(traffic[2]) + ")")
            traffic = (None, traffic[1], traffic[2])
    line = {
        "metric": "images/sec int8 %s, one MI355X, input resident in HBM" % names[args.workload],
        "value": args.batch / step_s,
        "unit": "images/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": step_s * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {"workload": titles[args.workload] % args.batch,
                   "batch": args.batch, "graph_nodes": len(g.nodes), "gmac_per_step": gmac,
                   "device_ms_per_step": dev_ms / args.steps,
                   "kernel_launches_per_step": launch_counts[0], "layer_sequence_launches": launch_counts[1],
                   "convolutions_inside_layer_sequences": launch_counts[2],
                   "ms_per_step_with_kernel_events": wall_events / args.steps * 1e3,
                   "images_per_s_through_CVMAPIInference": args.batch / api_s,
                   "images_per_s_two_models_in_flight": two_models_rate,
                   "output_checksum": int(np.bitwise_xor.reduce(out.view(np.uint32)))},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_I8_TOPS, "unit": "TOP/s",
                     "frac": achieved / PEAK_I8_TOPS,
                     "traffic": traffic[0], "traffic_unit": "bytes per launch", "traffic_source": traffic_note,
                     "kernel_source_sha256_16": source_hash,
                     "kernel": dom, "launches_per_step": conv["launches"] / args.steps,
                     "avg_launch_us": avg_s * 1e6, "avg_launch_us_with_event_pair": raw_avg_s * 1e6,
                     "event_pair_cost_us": pair_cost_us, "algorithmic_gop_per_launch": ops_per_launch / 1e9,
                     "kernel_ms_per_step": avg_s * 1e3 * conv["launches"] / args.steps,
                     "all_conv_dense_launches": {"achieved_tops": all_ops / max(all_s, 1e-9) / 1e12,
                                                 "launches_per_step": sum(v["launches"] for v in convs.values()) / args.steps,
                                                 "ms_per_step": all_s * 1e3 / args.steps},
                     "other_kernels_ms_per_step": {k: v["ms"] / args.steps for k, v in kt.items() if k != dom}},
    }
    # batch 1 of the same graph (the other half of the metric), measured the same way: input resident, `steps` runs
    b1 = {"resnet50": lambda: graphgen.resnet50(1), "vgg16": lambda: graphgen.vgg16(1),
          "resnet20": lambda: graphgen.resnet20_cifar(1), "ssd512": graphgen.ssd_mobilenet}[args.workload]
    g1, h1 = b1()
    js1, pb1 = g1.build(h1)
    if args.batch != 1 and not args.no_batch1:
        m1 = runtime.HipModel(js1, pb1)
        m1.set_input(x[:1].tobytes())
        m1.time_run(max(args.warmup, 1))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        m1.time_run(args.steps)
        torch.cuda.synchronize()
        b1_s = (time.perf_counter() - t0) / args.steps
        m1.close()
        line["config"]["images_per_s_batch1"] = 1.0 / b1_s
        line["config"]["ms_per_step_batch1"] = b1_s * 1e3
    if args.workload == "resnet50" and args.batch == 16 and not args.no_vgg:
        line["config"]["vgg16_b16"] = side_workload(pkg, L, "vgg16", 16, max(args.steps // 2, 5), args.warmup, not args.no_cpu_baseline)
        if line["config"]["vgg16_b16"].get("parity_checked") is False:
            print(json.dumps(line))
            sys.exit("bench.py: VGG-16 batch 16: the first image differs from the CPU runtime's result")
    # The CPU baseline leg runs the reference CPU runtime on the first image of the timed batch; its values also
    # check the timed configuration: the GPU's output for that image must equal them bit for bit.
    if not args.no_cpu_baseline:
        base, want = cpu_baseline(js1, pb1, x[:1].astype(np.int32), 20.0 if args.workload == "resnet50" else 5.0)
        line["cpu_baseline"] = base
        per_image = len(raw) // args.batch
        got = np.frombuffer(raw[:per_image], np.int32 if out_tsize == 4 else np.int8).astype(np.int32)
        ok = got.shape == want.shape and bool(np.array_equal(got, want))
        line["parity_checked"] = ok
        if not ok:
            print(json.dumps(line))
            sys.exit("bench.py: the output of the timed configuration differs from the CPU runtime's on the first image")
    print(json.dumps(line))


if __name__ == "__main__":
    main()
