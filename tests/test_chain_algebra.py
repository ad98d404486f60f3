"""CPU-only: the requantisation chains as the kernels evaluate them (cvmhip_chain_apply_host: the prepared form, with a
clamp behind a shift stage folded into that stage's own clamp) and the epilogue with the rounding terms moved into the
bias (cvmhip_fold_requant) against the operators applied one after the other by the oracle (src/runtime/cpu/ops/
elemwise.cc:128-148 cvm_right_shift, cvm_clip, clip, relu), on boundary values of every stage and random int32."""
import ctypes

import numpy as np
import pytest

import cvm_runtime_amd
import oracle
from cvm_runtime_amd import hipops


def _ref(stages, v):
    v = v.astype(np.int32)
    for st in stages:
        if st[0] == "relu":
            v = oracle.relu(v)
        elif st[0] == "cvm_right_shift":
            v = oracle.cvm_right_shift(v, st[1], st[2])
        elif st[0] == "cvm_clip":
            v = oracle.cvm_clip(v, st[1])
        elif st[0] == "clip":
            v = oracle.clip(v, st[1], st[2])
        else:
            raise ValueError(st)
    return v


def _apply(ch, v):
    lib = cvm_runtime_amd.lib()
    v = np.ascontiguousarray(v, np.int32)
    out = np.empty_like(v)
    rc = lib.cvmhip_chain_apply_host(ctypes.byref(ch), v.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(v.size),
                                     out.ctypes.data_as(ctypes.c_void_p))
    assert rc == 0
    return out


def _values(rng, shifts):
    """int32 extremes, everything around the points where a rounding shift by b changes its result or saturates, random"""
    pts = [0, 1, -1, 127, 128, -127, -128, 2 ** 31 - 1, -2 ** 31, 2 ** 31 - 2, -2 ** 31 + 1]
    for b in shifts:
        for m in (-300, -256, -255, -129, -128, -127, -1, 0, 1, 126, 127, 128, 254, 255, 256, 300):
            c = m * (1 << b)
            half = 1 << (b - 1) if b > 0 else 0
            pts += [c, c - 1, c + 1, c + half, c + half - 1, c - half, c - half - 1, c - half + 1]
    pts = [p for p in pts if -2 ** 31 <= p < 2 ** 31]
    rnd = rng.integers(-2 ** 31, 2 ** 31, 20000, dtype=np.int64)
    small = rng.integers(-2 ** 20, 2 ** 20, 20000, dtype=np.int64)
    return np.concatenate([np.array(pts, np.int64), rnd, small]).astype(np.int32)


CHAINS = [
    [("cvm_right_shift", 8, 8), ("cvm_clip", 8), ("relu",)],
    [("cvm_right_shift", 8, 7), ("relu",), ("cvm_clip", 8)],
    [("relu",), ("cvm_right_shift", 8, 1), ("cvm_clip", 8)],
    [("cvm_right_shift", 8, 10), ("clip", 0, 100)],
    [("cvm_right_shift", 8, 6), ("clip", -5, 5)],
    [("cvm_right_shift", 8, 6), ("clip", 300, 400)],          # a clamp outside the shift's range: a constant
    [("cvm_right_shift", 16, 3), ("cvm_clip", 8)],
    [("cvm_right_shift", 30, 5), ("relu",)],                   # precision + shift >= 32: rounding shift, no saturation
    [("cvm_right_shift", 32, 1), ("cvm_clip", 8)],             # the regime whose add may wrap: must stay unmerged and exact
    [("cvm_right_shift", 8, 31), ("relu",)],                   # shift >= 31: sign only
    [("cvm_right_shift", 1, 4), ("relu",)],                    # precision 1: always zero
    [("cvm_right_shift", 8, 8), ("cvm_right_shift", 8, 2), ("relu",)],
    [("clip", -1000, 1000), ("cvm_right_shift", 8, 3), ("relu",), ("cvm_clip", 6)],
    [("relu",)],
    [],
]


@pytest.mark.parametrize("stages", CHAINS, ids=lambda s: "+".join(x[0] + "".join("_%d" % a for a in x[1:]) for x in s) or "empty")
def test_prepared_chain_equals_the_operators_one_by_one(stages):
    rng = np.random.default_rng(7)
    v = _values(rng, [st[2] for st in stages if st[0] == "cvm_right_shift"])
    got = _apply(hipops.chain(*stages), v)
    want = _ref(stages, v)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (v[bad[:5]], got[bad[:5]], want[bad[:5]])


FOLDS = [
    # (chain1, chain2 or None, terms of the dot product, bias range)
    ([("cvm_right_shift", 8, 8), ("cvm_clip", 8), ("relu",)], None, 576, 2 ** 15),
    ([("cvm_right_shift", 8, 9), ("cvm_clip", 8)], [("relu",), ("cvm_right_shift", 8, 1), ("cvm_clip", 8)], 256, 2 ** 15),
    ([("cvm_right_shift", 8, 6), ("cvm_clip", 8)], [("cvm_right_shift", 8, 2), ("relu",)], 4608, 2 ** 20),
    ([], [("relu",), ("cvm_right_shift", 8, 7), ("cvm_clip", 8)], 64, 2 ** 10),
    ([("cvm_right_shift", 8, 8), ("relu",)], [("relu",)], 64, 2 ** 10),     # nothing to move from chain2
]


@pytest.mark.parametrize("case", range(len(FOLDS)))
def test_rounding_terms_folded_into_the_bias_change_no_result(case):
    c1, c2, terms, brange = FOLDS[case]
    lib = cvm_runtime_amd.lib()
    rng = np.random.default_rng(100 + case)
    oc = 48
    bias = rng.integers(-brange, brange + 1, oc).astype(np.int32)
    bound = terms * 128 * 128
    ch1, ch2 = hipops.chain(*c1), hipops.chain(*(c2 or []))
    out1, out2 = hipops.Chain(), hipops.Chain()
    fb = np.zeros(oc, np.int32)
    folded = lib.cvmhip_fold_requant(bias.ctypes.data_as(ctypes.c_void_p), oc, ctypes.c_int64(bound), ctypes.byref(ch1),
                                     ctypes.byref(ch2), 1 if c2 is not None else 0, fb.ctypes.data_as(ctypes.c_void_p),
                                     ctypes.byref(out1), ctypes.byref(out2))
    assert folded == 1
    # accumulators over the whole proven range, dense near the saturation points of the first shift
    acc = np.concatenate([rng.integers(-bound, bound + 1, 30000), np.array([-bound, bound, 0, 1, -1]),
                          rng.integers(-2 ** 17, 2 ** 17, 30000)]).astype(np.int64)
    chn = rng.integers(0, oc, acc.size)
    res = rng.integers(-128, 128, acc.size).astype(np.int32)
    x = (acc + bias[chn]).astype(np.int32)
    want = _ref(c1, x)
    if c2 is not None:
        want = _ref(c2, (want.astype(np.int64) + res).astype(np.int32))
    y = (acc + fb[chn]).astype(np.int32)
    got = _apply(out1, y)
    if c2 is not None:
        got = _apply(out2, (got.astype(np.int64) + res).astype(np.int32))
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (acc[bad[:5]], got[bad[:5]], want[bad[:5]])
    # every stage that is left is clamp-then-shift: no add per value any more
    for ch in (out1, out2):
        for i in range(ch.count):
            assert ch.stage[i].kind == 5


def test_fold_is_refused_when_the_sum_could_wrap_or_the_chain_has_another_shape():
    lib = cvm_runtime_amd.lib()
    oc = 4
    fb = np.zeros(oc, np.int32)
    out1, out2 = hipops.Chain(), hipops.Chain()

    def fold(bias, bound, c1, c2=None):
        ch1, ch2 = hipops.chain(*c1), hipops.chain(*(c2 or []))
        b = np.asarray(bias, np.int32)
        return lib.cvmhip_fold_requant(b.ctypes.data_as(ctypes.c_void_p), oc, ctypes.c_int64(bound), ctypes.byref(ch1),
                                       ctypes.byref(ch2), 1 if c2 is not None else 0, fb.ctypes.data_as(ctypes.c_void_p),
                                       ctypes.byref(out1), ctypes.byref(out2))
    good = [("cvm_right_shift", 8, 8), ("cvm_clip", 8)]
    assert fold([0, 1, 2, 3], 10 ** 6, good) == 1
    assert fold([0, 1, 2, 2 ** 31 - 1000], 10 ** 6, good) == 0          # bias + |acc| reaches the int32 limit
    assert fold([0, 1, 2, 3], 2 ** 31 - 100, good) == 0               # |acc| + the rounding term alone reaches it
    assert fold([0, 1, 2, 3], 10 ** 6, [("relu",)]) == 0                  # nothing to fold
    assert fold([0, 1, 2, 3], 10 ** 6, [("mul", 3), ("cvm_right_shift", 8, 8)]) == 0
    assert fold([0, 1, 2, 3], 10 ** 6, [("cvm_right_shift", 8, 8), ("cvm_right_shift", 8, 2)]) == 0   # a second rounding term stays
    assert fold([0, 1, 2, 3], 10 ** 6, [("cvm_right_shift", 30, 5)]) == 0  # shift-before-add regime
