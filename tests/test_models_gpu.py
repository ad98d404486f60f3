"""GPU parity of whole graphs through the model-level C ABI (CVMAPILoadModel /
CVMAPIInference, include/cvm_c_api.h) against the CPU oracle executing the same
graph node by node -- the method of the reference's tests/test_model.cc:94-235,
with the oracle in place of the absent /data fixtures.  Bit-exact."""
import os

import numpy as np
import pytest

import oracle
import oracle.graph as og
from cvm_runtime_amd import graphgen, runtime, synth

pytestmark = pytest.mark.gpu


def _run_both(g, heads, cid, postprocess=None):
    js, pb = g.build(heads, postprocess=postprocess)
    x = synth.tensor(cid, "data", g.shape((0, 0)), -127, 127)
    m = runtime.HipModel(js, pb)
    try:
        assert m.input_length == x.size      # int8 input: 1 byte per element
        out = m.inference(x.astype(np.int8).tobytes())
        out2 = m.inference(x.astype(np.int8).tobytes())   # storage is reused across calls
        assert out == out2
        tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
    finally:
        m.close()
    ref = og.run_graph(js, graphgen.load_params(pb), x)
    return out, tsize, ref


def _check(out, tsize, ref):
    got = np.frombuffer(out, np.int32 if tsize == 4 else np.int8).astype(np.int32)
    want = np.concatenate([r.ravel() for r in ref])
    assert got.shape == want.shape
    if not np.array_equal(got, want):
        bad = np.flatnonzero(got != want)
        raise AssertionError("%d of %d outputs differ, first at %d: got %d want %d" % (
            len(bad), want.size, bad[0], got[bad[0]], want[bad[0]]))


def test_config1_conv_shift_clip(dev):
    g, heads = graphgen.conv_op_graph()
    out, tsize, ref = _run_both(g, heads, "cfg1")
    assert tsize == 1                        # 8-bit output precision -> int8 bytes
    _check(out, tsize, ref)


@pytest.mark.parametrize("batch", [1, 64])
def test_config2_resnet20(batch, dev):
    g, heads = graphgen.resnet20_cifar(batch)
    out, tsize, ref = _run_both(g, heads, "cfg2-b%d" % batch)
    _check(out, tsize, ref)


def test_config3_resnet50_batch1_full_size(dev):
    g, heads = graphgen.resnet50(1)
    out, tsize, ref = _run_both(g, heads, "cfg3-b1")
    _check(out, tsize, ref)


def test_config3_resnet50_batch16_matches_per_image_runs(dev):
    # full-size batch 16: every image of the batch must equal the batch-1 result
    # of the same image (images are independent), and image 0 equals the oracle
    # through the batch-1 test above (same weights: same config id).
    g16, h16 = graphgen.resnet50(16)
    js16, pb = g16.build(h16)
    x = synth.tensor("cfg3-b16", "data", (16, 3, 224, 224), -127, 127).astype(np.int8)
    m16 = runtime.HipModel(js16, pb)
    out16 = np.frombuffer(m16.inference(x.tobytes()), np.int32).reshape(16, 1000)
    m16.close()
    g1, h1 = graphgen.resnet50(1)
    js1, pb1 = g1.build(h1)
    assert pb1 == pb
    m1 = runtime.HipModel(js1, pb1)
    for i in (0, 7, 15):
        o = np.frombuffer(m1.inference(x[i:i + 1].tobytes()), np.int32)
        assert np.array_equal(o, out16[i]), "image %d differs between batch 16 and batch 1" % i
    m1.close()
    ref = og.run_graph(js1, graphgen.load_params(pb1), x[3:4].astype(np.int32))
    assert np.array_equal(ref[0].ravel(), out16[3])


def test_config4_vgg16_reduced_width(dev):
    # same 13-conv / 5-pool / 3-dense structure at 1/4 width so the oracle finishes in seconds
    g, heads = graphgen.vgg16(2, size=64, width=16, fc=256, classes=100, config_id="cfg4-small")
    out, tsize, ref = _run_both(g, heads, "cfg4-small")
    _check(out, tsize, ref)


def test_config4_vgg16_full_size_batch1(dev):
    g, heads = graphgen.vgg16(1)
    out, tsize, ref = _run_both(g, heads, "cfg4-b1")
    _check(out, tsize, ref)


def test_config4_vgg16_batch16_matches_per_image_runs(dev):
    # full-size batch 16 (the large-layer regime of both convolution kernels): images are independent, so
    # every image must equal its batch-1 result; batch 1 equals the oracle through the test above
    g16, h16 = graphgen.vgg16(16)
    js16, pb = g16.build(h16)
    x = synth.tensor("cfg4-b16", "data", (16, 3, 224, 224), -127, 127).astype(np.int8)
    m16 = runtime.HipModel(js16, pb)
    out16 = np.frombuffer(m16.inference(x.tobytes()), np.int32).reshape(16, 1000)
    m16.close()
    g1, h1 = graphgen.vgg16(1)
    js1, pb1 = g1.build(h1)
    assert pb1 == pb
    m1 = runtime.HipModel(js1, pb1)
    for i in (0, 5, 15):
        o = np.frombuffer(m1.inference(x[i:i + 1].tobytes()), np.int32)
        assert np.array_equal(o, out16[i]), "image %d differs between batch 16 and batch 1" % i
    m1.close()
    # and one image of the batch straight against the oracle's graph executor (the compiled reference where it is built)
    ref = og.run_graph(js1, graphgen.load_params(pb1), x[9:10].astype(np.int32))
    assert np.array_equal(ref[0].ravel(), out16[9])


@pytest.mark.parametrize("neg_ids", [False, True])
def test_config5_ssd_mobilenet_detector(neg_ids, dev):
    g, heads = graphgen.ssd_mobilenet(neg_ids=neg_ids, config_id="cfg5-%d" % neg_ids)
    assert g.shape(heads[0]) == (1, 24564, 6)
    out, tsize, ref = _run_both(g, heads, "cfg5")
    _check(out, tsize, ref)
    kept = (ref[0][0, :, 0] >= 0).sum()
    assert 0 < kept <= 400


def test_depthwise_layers_on_the_vector_kernel_give_the_same_detections(dev):
    """The planner's two depthwise forms (matrix cores by default, vector kernel behind CVM_HIP_DW=valu)
    must both reproduce the oracle on a detector whose backbone is depthwise-separable."""
    g, heads = graphgen.ssd_mobilenet(size=128, alpha=0.5, config_id="cfg5-dw-forms", neg_ids=True)
    os.environ["CVM_HIP_DW"] = "valu"
    try:
        out, tsize, ref = _run_both(g, heads, "cfg5-dw-forms")
    finally:
        os.environ.pop("CVM_HIP_DW", None)
    _check(out, tsize, ref)
    out2, tsize2, ref2 = _run_both(g, heads, "cfg5-dw-forms")
    _check(out2, tsize2, ref2)
    assert out == out2


def _random_graph(seed, big=False):
    """A seeded random network from the building blocks the planner fuses: requantised convolutions
    (1x1 / 3x3, strided, depthwise), residual adds, pooling, channel concatenation, and one of three
    tails (global sum -> dense, flatten -> dense, detection heads).  Every tensor kept for reuse is 8-bit."""
    rng = np.random.RandomState(seed + (1000 if big else 0))
    g = graphgen.GraphBuilder("rand-%d-%d" % (seed, big))
    n = int(rng.choice([4, 16] if big else [1, 2, 3]))
    c = int(rng.choice([32, 64] if big else [3, 8, 16, 32]))
    hw = int(rng.choice([14, 28] if big else [9, 12, 16]))
    widths = [64, 128, 256, 512] if big else [16, 32, 48, 64, 96]
    x = g.var("data", (n, c, hw, hw), 8)
    pool = [x]
    for _ in range(int(rng.randint(5, 11))):
        cur = pool[-1]
        _, cc, h, w = g.shape(cur)
        kind = rng.choice(["conv", "conv", "conv", "dw", "add", "pool", "concat"])
        if kind == "conv":
            k = int(rng.choice([1, 3]))
            st = int(rng.choice([1, 1, 2])) if h >= 4 else 1
            oc = int(rng.choice(widths))
            pool.append(g.conv_relu_q(cur, oc, k, st, k // 2, relu=bool(rng.randint(2))))
        elif kind == "dw" and cc >= 8:
            st = int(rng.choice([1, 2])) if h >= 4 else 1
            pool.append(g.conv_relu_q(cur, cc, 3, st, 1, groups=cc))
        elif kind == "add":
            same = [t for t in pool[:-1] if g.shape(t) == g.shape(cur) and t is not x]
            if same:
                y = g.add(cur, same[int(rng.randint(len(same)))])
                if rng.randint(2):
                    y = g.relu(y)
                pool.append(g.rshift(y, 1))
        elif kind == "pool" and h >= 4:
            pool.append(g.max_pool(cur, 3, 2, 1) if rng.randint(2) else g.max_pool(cur, 2, 2))
        elif kind == "concat":
            same = [t for t in pool[:-1] if g.shape(t)[2:] == g.shape(cur)[2:] and g.shape(t)[0] == n and t is not x]
            if same:
                pool.append(g.concat([cur, same[int(rng.randint(len(same)))]], 1))
    cur = pool[-1]
    _, cc, h, w = g.shape(cur)
    tail = rng.choice(["sum", "flatten", "heads"])
    if tail == "flatten" and cc * h * w > 32767:   # dense precision 8 + 8 + bitlen(K) + 1 must stay within 32 bits
        tail = "sum"
    if tail == "sum":
        s_, cnt = g.global_sum(cur)
        s_ = g.rshift(s_, max(1, int(np.ceil(np.log2(cnt)))))
        y, _ = g.dense(g.flatten(s_), int(rng.choice([10, 33])))
        return g, [y]
    if tail == "flatten":
        y, _ = g.dense(g.flatten(cur), int(rng.choice([10, 33])))
        return g, [y]
    outs = []
    for src in (cur, pool[-2] if len(pool) > 2 and pool[-2] is not x else cur):
        oc = int(rng.choice([12, 24, 84]))
        y = g.conv_relu_q(src, oc, 3, 1, 1, relu=False)
        y = g.transpose(y, (0, 2, 3, 1))
        outs.append(g.reshape(y, (n, int(np.prod(g.shape(y)[1:])))))
    return g, [g.concat(outs, 1)]


@pytest.mark.parametrize("seed", range(64))
def test_random_graphs_match_the_oracle(seed, dev):
    g, heads = _random_graph(seed)
    out, tsize, ref = _run_both(g, heads, "rand-%d" % seed)
    _check(out, tsize, ref)


@pytest.mark.parametrize("seed", range(12))
def test_random_wide_graphs_match_the_oracle(seed, dev):
    """Batches of 4 and 16, up to 512 channels, 14x14 and 28x28 maps: the K-split, unsplit and large-tile
    configurations of the convolution kernel inside whole networks."""
    g, heads = _random_graph(seed, big=True)
    out, tsize, ref = _run_both(g, heads, "rand-%d-1" % seed)
    _check(out, tsize, ref)


@pytest.mark.parametrize("seed", range(16))
def test_random_graphs_node_by_node(seed, dev):
    """The same networks with the load-time fusion switched off: one registry kernel per node."""
    g, heads = _random_graph(seed)
    os.environ["CVM_HIP_FUSE"] = "0"
    try:
        out, tsize, ref = _run_both(g, heads, "rand-%d" % seed)
    finally:
        os.environ.pop("CVM_HIP_FUSE", None)
    _check(out, tsize, ref)


def test_argmax_postprocess_batch1_against_the_oracle_logits(dev):
    g, heads = graphgen.resnet20_cifar(1)
    js, pb = g.build(heads, postprocess="argmax")
    x = synth.tensor("post", "data", (1, 3, 32, 32), -127, 127)
    m = runtime.HipModel(js, pb)
    assert runtime.CVMAPIGetPreprocessMethod(m.net) == "argmax"
    assert m.output_length == 4
    out = np.frombuffer(m.inference(x.astype(np.int8).tobytes()), np.int32)
    m.close()
    logits = og.run_graph(js, graphgen.load_params(pb), x)[0].ravel()
    # the reference compares the logits as int8 (src/core/model.cc:193)
    assert out[0] == int(np.argmax(logits.astype(np.int8)))


def _golden_host():
    import json
    return json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "host_golden.json")))


@pytest.mark.parametrize("name", ["detection_int32", "two_heads_int8", "detection_narrow_heads",
                                  "detection_rows_differ", "argmax_batch4", "version_1_1_0"])
@pytest.mark.parametrize("fuse", ["1", "0"])
def test_postprocessing_models_match_the_bytes_the_reference_wrote(name, fuse, dev, capfd):
    """CVMModel::SaveTensor / GetOutputLength (src/core/model.cc:181-331): rows of several heads side by side
    in the int32 and the int8 form, heads whose row counts differ (ERROR_LOGIC), argmax over a batch with the
    reference's loop bound, and a graph of version cvm_1.1.0.  Expected sizes, status and output bytes were
    written by the compiled reference into an output buffer pre-filled with 0x5A (tests/golden/make_golden.py),
    so bytes the reference leaves untouched must stay untouched here too."""
    import ctypes
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    import make_golden
    want = _golden_host()["postprocess"][name]
    js, pb, x = make_golden.build_postprocess_model(name)
    os.environ["CVM_HIP_FUSE"] = fuse
    try:
        m = runtime.HipModel(js, pb)
    finally:
        os.environ.pop("CVM_HIP_FUSE", None)
    try:
        q = want["query"]
        assert m.input_length == q["CVMAPIGetInputLength"]
        assert m.output_length == q["CVMAPIGetOutputLength"]
        assert runtime.CVMAPIGetInputTypeSize(m.net) == q["CVMAPIGetInputTypeSize"]
        assert runtime.CVMAPIGetOutputTypeSize(m.net) == q["CVMAPIGetOutputTypeSize"]
        assert runtime.CVMAPIGetStorageSize(m.net) == q["CVMAPIGetStorageSize"]
        assert runtime.CVMAPIGetGasFromModel(m.net) == q["CVMAPIGetGasFromModel"]
        data = x.astype(np.int8).tobytes()
        for _ in range(2):                      # eager run, then the replayed graph
            out = ctypes.create_string_buffer(b"\x5a" * m.output_length, m.output_length)
            rc = runtime.lib().CVMAPIInference(m.net, ctypes.c_char_p(data), ctypes.c_int(len(data)), out)
            assert rc == want["status"], name
            if rc == 0:
                assert out.raw.hex() == want["output_hex"], name
    finally:
        m.close()
    capfd.readouterr()


def test_graph_replay_equals_eager_on_every_replay(dev):
    """After its first run a model replays a captured graph.  Every replay -- with fresh inputs, other
    GPU work and synchronisations in between -- must equal the eager, launch-by-launch result."""
    import os
    import torch
    g, heads = graphgen.resnet50(2, width=16, size=64, classes=50, config_id="replay-r50")
    js, pb = g.build(heads)
    xs = [synth.tensor("replay", "data%d" % i, (2, 3, 64, 64), -127, 127).astype(np.int8) for i in range(6)]
    os.environ["CVM_HIP_GRAPH"] = "0"
    try:
        eager = runtime.HipModel(js, pb)
        want = [eager.inference(x.tobytes()) for x in xs]
        eager.close()
    finally:
        os.environ.pop("CVM_HIP_GRAPH", None)
    m = runtime.HipModel(js, pb)
    scratch = torch.zeros(1 << 20, device=dev)
    for rnd in range(2):
        for i, x in enumerate(xs):        # run 1 is eager, run 2 captures, the rest replay
            got = m.inference(x.tobytes())
            assert got == want[i], "replay %d of round %d differs from the eager result" % (i, rnd)
            scratch.add_(1.0)             # unrelated eager work between replays
            torch.cuda.synchronize()
    m.close()
    ref = og.run_graph(js, graphgen.load_params(pb), xs[3].astype(np.int32))
    assert np.array_equal(np.frombuffer(want[3], np.int32), np.concatenate([r.ravel() for r in ref]))


def test_int8_input_is_clamped_like_the_reference(dev):
    """CvmRuntime::SetInput clamps `data` to +-(2^(p-1)-1) (graph_runtime.cc:345-352): the byte -128 runs as -127."""
    g, heads = graphgen.conv_op_graph(n=1, c=64, h=8, w=8, oc=64)
    js, pb = g.build(heads)
    x = synth.tensor("clamp", "data", (1, 64, 8, 8), -128, 127)
    x[0, :, 0, 0] = -128
    m = runtime.HipModel(js, pb)
    out = np.frombuffer(m.inference(x.astype(np.int8).tobytes()), np.int8).astype(np.int32)
    m.close()
    ref = og.run_graph(js, graphgen.load_params(pb), np.clip(x, -127, 127))
    assert np.array_equal(out, ref[0].ravel())


def test_two_nets_on_two_threads_and_many_replays(dev):
    """Distinct nets may run on different threads (the reference's threading rule): two models of
    different graphs run 40 inferences each at the same time; every result equals the one the model
    gives alone.  Also covers many replays of the captured graph of each model."""
    import threading
    ga, ha = graphgen.resnet20_cifar(4)
    gb, hb = graphgen.ssd_mobilenet(size=128, alpha=0.25, config_id="threads-ssd", neg_ids=True)
    specs = []
    for g, h, cid in ((ga, ha, "threads-a"), (gb, hb, "threads-b")):
        js, pb = g.build(h)
        x = synth.tensor(cid, "data", g.shape((0, 0)), -127, 127).astype(np.int8).tobytes()
        m = runtime.HipModel(js, pb)
        specs.append((m, x, m.inference(x)))
    errors = []

    def work(m, x, want):
        try:
            for _ in range(40):
                if m.inference(x) != want:
                    errors.append("result changed")
                    return
        except Exception as e:   # noqa: BLE001 - reported below
            errors.append(repr(e))
    threads = [threading.Thread(target=work, args=s) for s in specs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for m, _, _ in specs:
        m.close()
    assert not errors, errors
