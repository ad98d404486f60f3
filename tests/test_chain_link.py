"""Host-side rules of cvmhip_conv_seq_link (include/cvm_hip_ops.h): which runs of a layer-sequence table become
chains -- 1x1 layers computed from registers by the wavefront that holds their input -- and which must not.  The
tables are built from made-up device addresses; nothing here touches a GPU."""
import ctypes

import pytest

import cvm_runtime_amd
from cvm_runtime_amd import hipops


@pytest.fixture(scope="module")
def lib():
    l = cvm_runtime_amd.lib()
    l.cvmhip_conv_seq_layer_bytes.restype = ctypes.c_size_t
    l.cvmhip_conv_seq_layer.argtypes = [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 7 + [ctypes.c_int] * 13
    l.cvmhip_conv_seq_link.argtypes = [ctypes.c_void_p, ctypes.c_int]
    l.cvmhip_conv_seq_layer_chain.argtypes = [ctypes.c_void_p, ctypes.c_int]
    l.cvmhip_conv_seq_layer_config.argtypes = [ctypes.c_void_p, ctypes.c_int]
    return l


MB = 1 << 20
X, Y1, Y2, XO, Y1O, W = 0x10000000, 0x10000000 + 64 * MB, 0x10000000 + 128 * MB, 0x10000000 + 192 * MB, 0x10000000 + 256 * MB, 0x20000000


def _table(lib, layers, n=16, hw=56):
    """layers: (input address, output address, residual address or 0, ic, oc, k, stride, pad); returns (buffer, count)"""
    entry = lib.cvmhip_conv_seq_layer_bytes()
    buf = ctypes.create_string_buffer(entry * len(layers))
    chain = hipops.Chain()
    chain.count = 0
    size = hw
    for i, (xp, out, res, ic, oc, k, st, pad) in enumerate(layers):
        rc = lib.cvmhip_conv_seq_layer(buf, i, xp, W + i * MB, None, ctypes.byref(chain), res or None, ctypes.byref(chain), out,
                                       n, ic, size, size, oc, k, k, st, st, pad, pad, 1, 1)
        assert rc == 0, (i, cvm_runtime_amd.lib().cvmhip_last_error())
        size = (size + 2 * pad - k) // st + 1
    return buf, len(layers)


def _chains(lib, buf, count):
    return [lib.cvmhip_conv_seq_layer_chain(buf, i) for i in range(count)]


def test_a_bottleneck_tail_becomes_one_chain(lib):
    """3x3 64 -> 64, 1x1 64 -> 256 with the block input as residual, 1x1 256 -> 64: the ResNet-50 run"""
    buf, n = _table(lib, [(Y1, Y2, 0, 64, 64, 3, 1, 1), (Y2, XO, X, 64, 256, 1, 1, 0), (XO, Y1O, 0, 256, 64, 1, 1, 0)])
    assert lib.cvmhip_conv_seq_link(buf, n) == 1
    assert _chains(lib, buf, n) == [2, 0, 0]
    assert lib.cvmhip_conv_seq_layer_config(buf, 0) == 7


def test_the_residual_may_be_the_output_tensor_itself(lib):
    buf, n = _table(lib, [(Y1, Y2, 0, 64, 64, 3, 1, 1), (Y2, X, X, 64, 256, 1, 1, 0), (X, Y1O, 0, 256, 128, 1, 1, 0)])
    assert lib.cvmhip_conv_seq_link(buf, n) == 1
    assert _chains(lib, buf, n) == [2, 0, 0]


@pytest.mark.parametrize("case", ["second output over the first input", "third output over the first input",
                                  "third output over the residual", "residual overlaps the output partly"])
def test_an_output_over_something_the_layer_still_reads_breaks_the_chain(lib, case):
    """While one wavefront stores its pixels, others still read the first layer's input around theirs (3x3) and the
    residual at theirs: a memory plan that reuses such a buffer is fine with a boundary between the layers and not without."""
    a, b, c = (Y1, Y2, 0, 64, 64, 3, 1, 1), (Y2, XO, X, 64, 256, 1, 1, 0), (XO, Y1O, 0, 256, 64, 1, 1, 0)
    want = [1, 0, 0]
    if case == "second output over the first input":
        b, c, want = (Y2, Y1, X, 64, 256, 1, 1, 0), (Y1, Y1O, 0, 256, 64, 1, 1, 0), [0, 0, 0]
    elif case == "third output over the first input":
        c = (XO, Y1, 0, 256, 64, 1, 1, 0)
    elif case == "third output over the residual":
        c = (XO, X, 0, 256, 64, 1, 1, 0)
    else:
        b, c, want = (Y2, X + 1024, X, 64, 256, 1, 1, 0), (X + 1024, Y1O, 0, 256, 64, 1, 1, 0), [0, 0, 0]
    buf, n = _table(lib, [a, b, c])
    lib.cvmhip_conv_seq_link(buf, n)
    assert _chains(lib, buf, n) == want


def test_what_cannot_follow(lib):
    # the follower reads another tensor; has a stride; is a 3x3; the head has 128 channels; a third layer of 256 channels
    for layers, want, hw in [
        ([(Y1, Y2, 0, 64, 64, 3, 1, 1), (X, XO, 0, 64, 256, 1, 1, 0)], [16, 0], 56),   # (no chain, but no boundary either: see below)
        ([(Y1, Y2, 0, 64, 64, 3, 1, 1), (Y2, XO, 0, 64, 256, 1, 2, 0)], [0, 0], 56),
        ([(Y1, Y2, 0, 64, 64, 3, 1, 1), (Y2, XO, 0, 64, 64, 3, 1, 1)], [0, 0], 56),
        ([(Y1, Y2, 0, 128, 128, 3, 1, 1), (Y2, XO, 0, 128, 512, 1, 1, 0)], [0, 0], 14),
        ([(Y1, Y2, 0, 64, 64, 3, 1, 1), (Y2, XO, 0, 64, 256, 1, 1, 0), (XO, Y1O, 0, 256, 256, 1, 1, 0)], [1, 0, 0], 56),
        ([(Y1, Y2, 0, 64, 64, 3, 1, 1), (Y2, XO, 0, 64, 40, 1, 1, 0)], [0, 0], 56),          # not whole 32-channel tiles
    ]:
        buf, n = _table(lib, layers, hw=hw)
        lib.cvmhip_conv_seq_link(buf, n)
        assert _chains(lib, buf, n) == want, layers


def test_layers_that_have_nothing_to_do_with_one_another_share_a_step(lib):
    """The first 1x1 layer and the shortcut projection of a ResNet block both read the block's input: no boundary between
    them (16 = no boundary behind the entry).  The 3x3 layer behind them reads the first one's output and waits."""
    buf, n = _table(lib, [(X, Y1, 0, 64, 64, 1, 1, 0), (X, XO, 0, 64, 256, 1, 1, 0), (Y1, Y2, 0, 64, 64, 3, 1, 1)])
    assert lib.cvmhip_conv_seq_link(buf, n) == 1
    assert _chains(lib, buf, n) == [16, 0, 0]
    # the second layer writes over the first one's input, or over its output: a boundary stays
    for second in [(Y2, X, 0, 64, 64, 1, 1, 0), (Y2, Y1, 0, 64, 64, 1, 1, 0), (Y2, Y1O, X + 4096, 64, 64, 1, 1, 0)]:
        buf, n = _table(lib, [(X, Y1, 0, 64, 64, 1, 1, 0), second])
        lib.cvmhip_conv_seq_link(buf, n)
        assert _chains(lib, buf, n) == ([0, 0] if second[1] != Y1O else [16, 0]), second
    # ... or reads, as residual, what the first one writes
    buf, n = _table(lib, [(X, Y1, 0, 64, 64, 1, 1, 0), (Y2, Y1O, Y1, 64, 64, 1, 1, 0)])
    lib.cvmhip_conv_seq_link(buf, n)
    assert _chains(lib, buf, n) == [0, 0]
    # a chain may be the second of the two
    buf, n = _table(lib, [(X, XO, 0, 64, 256, 1, 1, 0), (Y1, Y2, 0, 64, 64, 3, 1, 1), (Y2, Y1O, 0, 64, 128, 1, 1, 0)])
    assert lib.cvmhip_conv_seq_link(buf, n) == 2
    assert _chains(lib, buf, n) == [16, 1, 0]


def test_filters_must_fit_the_workgroups_lds(lib):
    """64 -> 64 with a 7x7 filter is 2 x 99 KiB of packed filter: more than the 128 KiB block that also has to hold the followers'"""
    buf, n = _table(lib, [(Y1, Y2, 0, 64, 64, 7, 1, 3), (Y2, XO, 0, 64, 256, 1, 1, 0)])
    lib.cvmhip_conv_seq_link(buf, n)
    assert _chains(lib, buf, n) == [0, 0]
    buf, n = _table(lib, [(Y1, Y2, 0, 64, 64, 5, 1, 2), (Y2, XO, 0, 64, 256, 1, 1, 0), (XO, Y1O, 0, 256, 128, 1, 1, 0)])
    lib.cvmhip_conv_seq_link(buf, n)   # 2 x 51 + 8 x 3 = 126 KiB with the second layer; the third one's 36 KiB no longer fit
    assert _chains(lib, buf, n) == [1, 0, 0]


def test_switched_off_and_forced_configurations(lib):
    layers = [(Y1, Y2, 0, 64, 64, 3, 1, 1), (Y2, XO, X, 64, 256, 1, 1, 0), (XO, Y1O, 0, 256, 64, 1, 1, 0)]
    try:
        lib.cvmhip_set_seq_chains(0)
        buf, n = _table(lib, layers)
        assert lib.cvmhip_conv_seq_link(buf, n) == 0 and _chains(lib, buf, n) == [0, 0, 0]
        lib.cvmhip_set_seq_chains(1)
        lib.cvmhip_set_seq_layer_config(1, 3)     # the second layer's tile configuration is forced: it stays a layer of its own
        buf, n = _table(lib, layers)
        assert lib.cvmhip_conv_seq_link(buf, n) == 0
        assert lib.cvmhip_conv_seq_layer_config(buf, 1) == 3
    finally:
        lib.cvmhip_set_seq_chains(1)
        lib.cvmhip_set_seq_layer_config(-1, -1)
