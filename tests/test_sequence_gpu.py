"""Layer-sequence launches (a run of convolutions in one kernel, every XCD computing all layers for its share
of the images; include/cvm_hip_ops.h: cvmhip_conv_seq_*) against the CPU oracle executing the same graph node
by node, and against the same model with one launch per layer.  Bit-exact.  CVM_HIP_SEQ=1 forces the
sequences (by default a model measures both ways when it is loaded and keeps the faster), =0 switches them off."""
import os

import numpy as np
import pytest

import oracle.graph as og
from cvm_runtime_amd import graphgen, runtime, synth

pytestmark = pytest.mark.gpu


def _run(js, pb, x, seq):
    os.environ["CVM_HIP_SEQ"] = seq
    try:
        m = runtime.HipModel(js, pb)
    finally:
        os.environ.pop("CVM_HIP_SEQ", None)
    try:
        launches, sequences, layers = m.launch_counts()
        assert (sequences >= 1 and layers >= 3) if seq == "1" else (sequences == 0 and layers == 0), (launches, sequences, layers)
        outs = [m.inference(x.tobytes()) for _ in range(3)]      # eager run, captured run, replay
        tsize = runtime.CVMAPIGetOutputTypeSize(m.net)
        after = m.launch_counts()
    finally:
        m.close()
    assert outs[0] == outs[1] == outs[2], "runs of one model differ"
    assert m_counts_unchanged(seq, after), "a sequence launch gave up and the model fell back: %s" % (after,)
    return np.frombuffer(outs[0], np.int32 if tsize == 4 else np.int8).astype(np.int32)


def m_counts_unchanged(seq, after):
    return after[1] >= 1 if seq == "1" else after[1] == 0


def _check(g, heads, cid, oracle_too=True):
    js, pb = g.build(heads)
    x = synth.tensor(cid, "data", g.shape((0, 0)), -127, 127).astype(np.int8)
    with_seq = _run(js, pb, x, "1")
    without = _run(js, pb, x, "0")
    assert np.array_equal(with_seq, without), "%d of %d values differ from one launch per layer" % (
        int((with_seq != without).sum()), without.size)
    if oracle_too:
        ref = og.run_graph(js, graphgen.load_params(pb), x.astype(np.int32))
        want = np.concatenate([r.ravel() for r in ref])
        assert np.array_equal(with_seq, want), "%d of %d values differ from the oracle" % (int((with_seq != want).sum()), want.size)


def _chain(cid, n, c, hw, layers):
    """data -> a chain of requantised convolutions given as (oc, k, stride, relu, residual_from) -> global sum."""
    g = graphgen.GraphBuilder(cid)
    x = g.var("data", (n, c, hw, hw), 8)
    kept = [g.conv_relu_q(x, layers[0][0], 3, 1, 1)]          # the few-channel input layer stays outside the sequence
    for layer in layers[1:]:
        oc, k, st, relu, res = layer[:5]
        pad = layer[5] if len(layer) > 5 else k // 2
        y = g.conv_relu_q(kept[-1], oc, k, st, pad, relu=relu)
        if res is not None and g.shape(kept[res]) == g.shape(y):
            y = g.rshift(g.relu(g.add(y, kept[res])), 1)
        kept.append(y)
    s, _ = g.global_sum(kept[-1])
    return g, [g.rshift(s, 6)]


CHAINS = {
    # batch 8: one image per XCD; 7x7 and 5x5 maps give shares that are not multiples of 32 (or of 8) pixels
    "b8_1x1_3x3_residual": (8, 3, 14, [(64, 0, 0, 0, None), (64, 1, 1, True, None), (64, 3, 1, True, None), (256, 1, 1, False, None),
                                       (64, 1, 1, True, None), (64, 3, 1, True, None), (256, 1, 1, False, 3)]),
    "b8_strided_no_padding": (8, 3, 15, [(32, 0, 0, 0, None), (64, 1, 2, True, None), (96, 3, 2, True, None), (128, 1, 1, True, None),
                                         (128, 3, 1, False, None)]),
    "b16_ragged_shares_7x7": (16, 3, 7, [(128, 0, 0, 0, None), (512, 1, 1, True, None), (128, 1, 1, True, None), (128, 3, 1, True, None),
                                         (512, 1, 1, False, 1), (1000, 1, 1, True, None)]),
    "b8_deep_k": (8, 3, 5, [(64, 0, 0, 0, None), (1024, 1, 1, True, None), (256, 1, 1, True, None), (256, 3, 1, True, None),
                            (2048, 1, 1, True, None), (40, 1, 1, True, None)]),
    "b24_three_images_per_share": (24, 3, 6, [(32, 0, 0, 0, None), (32, 3, 1, True, None), (64, 1, 1, True, None), (64, 3, 2, True, None),
                                              (96, 1, 1, False, None)]),
    "b8_many_tiles_two_rounds": (8, 3, 40, [(64, 0, 0, 0, None), (256, 1, 1, True, None), (64, 1, 1, True, None), (64, 3, 1, True, None),
                                            (256, 1, 1, False, 1)]),
    # batches that do not divide over the 8 XCDs run on 1, 2 or 4 of them
    "b1_one_xcd": (1, 3, 28, [(64, 0, 0, 0, None), (256, 1, 1, True, None), (64, 1, 1, True, None), (64, 3, 1, True, None),
                              (256, 1, 1, False, 1), (128, 3, 2, True, None)]),
    "b2_two_xcds": (2, 3, 9, [(32, 0, 0, 0, None), (128, 1, 1, True, None), (128, 3, 1, True, None), (512, 1, 1, True, None),
                              (96, 1, 1, False, None)]),
    "b3_one_xcd_three_images": (3, 3, 10, [(32, 0, 0, 0, None), (64, 3, 1, True, None), (64, 1, 1, True, None), (64, 3, 2, True, None),
                                           (160, 1, 1, False, None)]),
    "b12_four_xcds": (12, 3, 8, [(64, 0, 0, 0, None), (64, 1, 1, True, None), (64, 3, 1, True, None), (256, 1, 1, False, None),
                                 (64, 1, 1, True, None)]),
}


# Runs in which a layer with 64 output channels is followed by one or two 1x1 layers over the same pixels: the wavefront
# that holds the first layer's result computes the followers from registers (cvmhip_conv_seq_link).  (name: expected
# positions, among the sequence's layers, of the heads of chains -- the few-channel input layer is not part of the sequence)
LINKED = {
    # 3x3 (padding) -> 1x1 with residual -> 1x1 back to 64, twice; the second chain has no third layer of 64 or 128 channels
    "b8_bottlenecks": (8, 3, 14, [(64, 0, 0, 0, None), (256, 1, 1, False, None), (64, 1, 1, True, None), (64, 3, 1, True, None),
                                  (256, 1, 1, False, 1), (64, 1, 1, True, None), (64, 3, 1, True, None), (256, 1, 1, False, 4),
                                  (96, 1, 1, True, None)], {2: 7, 5: 7}),
    # the third layer has 128 channels; 7x7 maps at batch 16: shares of 98 pixels that begin inside a pixel block
    "b16_third_layer_128_ragged_shares": (16, 3, 7, [(64, 0, 0, 0, None), (256, 1, 1, True, None), (64, 1, 1, True, None),
                                                     (64, 3, 1, True, None), (256, 1, 1, False, 1), (128, 1, 1, True, None),
                                                     (64, 1, 1, True, None)], {2: 7}),
    # the head is a 3x3 layer without padding and stride 2, then one with 1x1 (identity addressing); 384 and 32 channels behind
    "b8_heads_without_padding": (8, 3, 21, [(64, 0, 0, 0, None), (64, 3, 2, True, None, 0), (384, 1, 1, True, None), (64, 1, 1, True, None),
                                            (64, 1, 1, True, None), (128, 1, 1, False, None), (32, 1, 1, True, None), (64, 3, 1, True, None)],
                                 {0: 7, 3: 7}),
    # batches on one and on four XCDs
    "b3_one_xcd": (3, 3, 10, [(64, 0, 0, 0, None), (64, 3, 1, True, None), (256, 1, 1, True, None), (64, 1, 1, False, None),
                              (64, 3, 1, True, None)], {0: 7}),
    "b12_four_xcds": (12, 3, 9, [(32, 0, 0, 0, None), (64, 1, 1, True, None), (512, 1, 1, True, None), (128, 1, 1, True, None),
                                 (128, 3, 1, True, None)], {0: 7}),
}


@pytest.mark.parametrize("name", sorted(LINKED))
def test_1x1_layers_chained_behind_the_layer_that_feeds_them(name, dev):
    """The chains are found where expected (and nowhere with CVM_HIP_SEQ_CHAIN=0), and the model's output is the one of
    one launch per layer and of the oracle either way."""
    n, c, hw, layers, heads_at = LINKED[name]
    cid = "seq-link-" + name
    g, heads = _chain(cid, n, c, hw, layers)
    js, pb = g.build(heads)
    x = synth.tensor(cid, "data", g.shape((0, 0)), -127, 127).astype(np.int8)
    os.environ["CVM_HIP_SEQ"] = "1"
    try:
        m = runtime.HipModel(js, pb)
        linked = m.sequence_configs()
        m.close()
        os.environ["CVM_HIP_SEQ_CHAIN"] = "0"
        m = runtime.HipModel(js, pb)
        plain = m.sequence_configs()
        m.close()
    finally:
        os.environ.pop("CVM_HIP_SEQ", None)
        os.environ.pop("CVM_HIP_SEQ_CHAIN", None)
    assert 7 not in plain, plain
    assert [i for i, cfg in enumerate(linked) if cfg == 7] == sorted(heads_at), (linked, plain)
    with_chains = _run(js, pb, x, "1")
    os.environ["CVM_HIP_SEQ_CHAIN"] = "0"
    try:
        without_chains = _run(js, pb, x, "1")
    finally:
        os.environ.pop("CVM_HIP_SEQ_CHAIN", None)
    one_by_one = _run(js, pb, x, "0")
    assert np.array_equal(with_chains, one_by_one), "%d of %d values differ from one launch per layer" % (
        int((with_chains != one_by_one).sum()), one_by_one.size)
    assert np.array_equal(without_chains, one_by_one)
    ref = og.run_graph(js, graphgen.load_params(pb), x.astype(np.int32))
    want = np.concatenate([r.ravel() for r in ref])
    assert np.array_equal(with_chains, want), "%d of %d values differ from the oracle" % (int((with_chains != want).sum()), want.size)


@pytest.mark.parametrize("name", sorted(CHAINS))
def test_chain_of_convolutions_in_one_launch(name, dev):
    n, c, hw, layers = CHAINS[name]
    g, heads = _chain("seq-" + name, n, c, hw, layers)
    _check(g, heads, "seq-" + name)


@pytest.mark.parametrize("batch", (8, 16))
@pytest.mark.parametrize("cfg", range(7))
def test_every_configuration_of_the_tile_kernel_inside_a_sequence(cfg, batch, dev):
    """CVM_HIP_WAVECFG forces one configuration for every layer of the sequence (all three addressing modes occur).
    The model reports the configuration its table was built with: the forced one, for every layer."""
    cid = "seq-cfg%d-b%d" % (cfg, batch)
    g, heads = _chain(cid, batch, 3, 12, [(64, 0, 0, 0, None), (64, 1, 1, True, None), (128, 3, 2, True, None),
                                           (128, 1, 2, True, None), (256, 3, 1, False, 2), (256, 1, 1, True, None)])
    os.environ["CVM_HIP_WAVECFG"] = str(cfg)
    try:
        _check(g, heads, cid)
        js, pb = g.build(heads)
        os.environ["CVM_HIP_SEQ"] = "1"
        m = runtime.HipModel(js, pb)
        try:
            built = m.sequence_configs()
        finally:
            m.close()
        assert built == [cfg] * 5, built
    finally:
        os.environ.pop("CVM_HIP_WAVECFG", None)
        os.environ.pop("CVM_HIP_SEQ", None)


def test_single_layers_of_a_sequence_take_the_configuration_named_for_them(dev):
    """CVM_HIP_SEQCFG="index:config,...": the tuning hook for one layer at a time; the others keep the automatic choice."""
    n, c, hw, layers = CHAINS["b16_ragged_shares_7x7"]
    g, heads = _chain("seq-percfg", n, c, hw, layers)
    js, pb = g.build(heads)
    os.environ["CVM_HIP_SEQ"] = "1"
    try:
        m = runtime.HipModel(js, pb)
        auto = m.sequence_configs()
        m.close()
        os.environ["CVM_HIP_SEQCFG"] = "1:6,3:5"
        m = runtime.HipModel(js, pb)
        forced = m.sequence_configs()
        m.close()
    finally:
        os.environ.pop("CVM_HIP_SEQ", None)
        os.environ.pop("CVM_HIP_SEQCFG", None)
    want = list(auto)
    want[1], want[3] = 6, 5
    assert forced == want, (auto, forced)
    os.environ["CVM_HIP_SEQCFG"] = "1:6,3:5"
    try:
        _check(g, heads, "seq-percfg")
    finally:
        os.environ.pop("CVM_HIP_SEQCFG", None)


def test_a_sequence_launch_that_gives_up_is_repeated_with_one_launch_per_layer(dev):
    """CVM_HIP_SEQ_SPIN=0: every wait at a layer boundary gives up at once (all workgroups still run to the end and
    exit normally), so the launch raises its error word; the runtime must notice after the run, switch sequence
    launches off for the model and repeat the run with one launch per layer.  The bytes returned are the right ones
    every time, and the model reports no sequence launches afterwards."""
    g, heads = graphgen.resnet50(16, width=32, size=64, classes=100, config_id="seq-giveup")
    js, pb = g.build(heads)
    x = synth.tensor("seq-giveup", "data", g.shape((0, 0)), -127, 127).astype(np.int8)
    want = _run(js, pb, x, "0")
    os.environ["CVM_HIP_SEQ"] = "1"
    os.environ["CVM_HIP_SEQ_SPIN"] = "0"
    try:
        m = runtime.HipModel(js, pb)
    finally:
        os.environ.pop("CVM_HIP_SEQ", None)
        os.environ.pop("CVM_HIP_SEQ_SPIN", None)
    try:
        assert m.launch_counts()[1] >= 1
        outs = [np.frombuffer(m.inference(x.tobytes()), np.int32) for _ in range(4)]
        after = m.launch_counts()
    finally:
        m.close()
    for o in outs:
        assert np.array_equal(o, want)
    assert after[1] == 0 and after[2] == 0, after


def test_resnet50_shrunk_batch16_and_resnet20_batch64(dev):
    g, heads = graphgen.resnet50(16, width=32, size=64, classes=100, config_id="seq-r50")
    _check(g, heads, "seq-r50")
    g, heads = graphgen.resnet20_cifar(64)
    _check(g, heads, "seq-r20", oracle_too=False)     # the oracle comparison of this model is in test_models_gpu.py


def test_resnet50_full_size_batch16_equals_one_launch_per_layer(dev):
    g, heads = graphgen.resnet50(16)
    _check(g, heads, "seq-r50-full", oracle_too=False)   # image-wise oracle parity of this model: test_models_gpu.py


def test_two_models_with_sequences_on_two_threads(dev):
    """Two sequence launches must never be in flight at once; the runtime orders the runs of different models."""
    import threading
    g, heads = graphgen.resnet50(8, width=16, size=64, classes=50, config_id="seq-two")
    js, pb = g.build(heads)
    x = synth.tensor("seq-two", "data", (8, 3, 64, 64), -127, 127).astype(np.int8)
    want = _run(js, pb, x, "0")
    os.environ["CVM_HIP_SEQ"] = "1"
    try:
        models = [runtime.HipModel(js, pb) for _ in range(2)]
    finally:
        os.environ.pop("CVM_HIP_SEQ", None)
    results = [[], []]
    errors = []

    def work(i):
        try:
            for _ in range(20):
                results[i].append(models[i].inference(x.tobytes()))
        except Exception as e:   # noqa: BLE001 - reported below
            errors.append(repr(e))
    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for m in models:
        m.close()
    assert not errors, errors
    for i in range(2):
        assert len(results[i]) == 20
        for out in results[i]:
            assert np.array_equal(np.frombuffer(out, np.int32), want)


def test_while_two_models_with_sequences_are_alive_both_use_one_launch_per_layer(dev):
    """Sequence launches are for a model that has the chip to itself.  A model loaded next to one that uses them does not
    compare the two launch forms then (both would be timed as one launch per layer) but stays counted, so that neither
    of the two issues a sequence launch; when the other one is gone it makes the comparison at its next run.  Results
    are the same bytes throughout."""
    g, heads = graphgen.resnet50(8, width=16, size=64, classes=50, config_id="seq-policy")
    js, pb = g.build(heads)
    x = synth.tensor("seq-policy", "data", (8, 3, 64, 64), -127, 127).astype(np.int8)
    want = _run(js, pb, x, "0")
    os.environ["CVM_HIP_SEQ"] = "1"
    try:
        first = runtime.HipModel(js, pb)
    finally:
        os.environ.pop("CVM_HIP_SEQ", None)
    try:
        assert first.launch_counts()[1] >= 1
        second = runtime.HipModel(js, pb)          # no switch: it would measure, were it alone
        try:
            assert first.launch_counts()[1] == 0 and second.launch_counts()[1] == 0
            for m in (first, second, first, second):
                assert np.array_equal(np.frombuffer(m.inference(x.tobytes()), np.int32), want)
            assert first.launch_counts()[1] == 0 and second.launch_counts()[1] == 0
        finally:
            first.close()
            first = None
        for _ in range(3):                         # alone now: the comparison happens inside the first of these runs
            assert np.array_equal(np.frombuffer(second.inference(x.tobytes()), np.int32), want)
        second.close()
    finally:
        if first is not None:
            first.close()
