"""The entry point that allocates nothing (cvmhip_non_max_suppression_static: scratch in a fixed
array inside the library) against the existing entry point with a caller workspace, through the C
ABI.  Two calls in a row share the array, the second on a smaller input; both must equal the
workspace entry point bit for bit (output and the mutated input)."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from cvm_runtime_amd import hipops, lib, synth

pytestmark = pytest.mark.gpu


def _boxes(cid, b, n, id_lo, id_hi, extent):
    ids = synth.tensor(cid, "id", (b, n, 1), id_lo, id_hi)
    sc = synth.tensor(cid, "score", (b, n, 1), -127, 127)
    xy = synth.tensor(cid, "xy", (b, n, 4), 0, extent)
    x1 = np.minimum(xy[..., 0], xy[..., 2]); x2 = np.maximum(xy[..., 0], xy[..., 2])
    y1 = np.minimum(xy[..., 1], xy[..., 3]); y2 = np.maximum(xy[..., 1], xy[..., 3])
    return np.concatenate([ids, sc, x1[..., None], y1[..., None], x2[..., None], y2[..., None]], axis=2).astype(np.int32)


def _both(case, dev):
    b, n, id_lo, iou, topk, mos, force, extent = case
    x = _boxes("nms-static-%s" % (case,), b, n, id_lo, 20 if n > 1000 else 3, extent)
    vc, xs = oracle.get_valid_counts(x, 10)
    init = np.full_like(xs, 5)
    T = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(dev)
    x_ws, y_ws = T(xs), T(init)
    hipops.non_max_suppression(x_ws, T(vc), y_ws, iou, force, topk, max_output_size=mos)
    x_st, y_st = T(xs), T(init)
    hipops.non_max_suppression_static(x_st, T(vc), y_st, iou, force, topk, max_output_size=mos)
    torch.cuda.synchronize()
    assert torch.equal(y_st, y_ws), "output differs from the workspace entry point: %s" % (case,)
    assert torch.equal(x_st, x_ws), "mutated input differs from the workspace entry point: %s" % (case,)
    # and the oracle, so that a shared mistake cannot hide
    y_ref, x_after = oracle.non_max_suppression(xs, vc, iou, force, topk, max_output_size=mos, y_init=init)
    assert np.array_equal(y_st.cpu().numpy(), y_ref) and np.array_equal(x_st.cpu().numpy(), x_after)


def test_static_scratch_two_calls_in_a_row_second_smaller(dev):
    # b, n, id_lo, iou, topk, mos, force, extent
    _both((1, 24564, -1, 45, 400, -1, False, 512), dev)    # the detector's shape: top-k ranking, bit-matrix walk
    _both((2, 300, -1, 30, -1, -1, False, 64), dev)        # smaller, all-pairs ranking (its counters start at zero)
    _both((1, 4000, -1, 45, -1, 100, False, 256), dev)     # larger again, row-by-row walk
    _both((3, 64, -1, 10, 5, 3, True, 32), dev)


def test_static_scratch_rejects_sizes_beyond_its_capacity(dev):
    L = lib()
    cap = L.cvmhip_nms_static_capacity_bytes()
    assert cap == 2 << 20
    n = 60000
    assert L.cvmhip_nms_workspace_bytes(1, n, 6) > cap
    x = torch.zeros((1, n, 6), dtype=torch.int32, device=dev)
    y = torch.zeros_like(x)
    vc = torch.zeros((1,), dtype=torch.int32, device=dev)
    rc = L.cvmhip_non_max_suppression_static(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(vc.data_ptr()),
                                             ctypes.c_void_p(y.data_ptr()), 1, n, 6, -1, 45, -1, 2, 1, 0, 0, None)
    assert rc == 10 and b"static" in L.cvmhip_last_error()
    torch.cuda.synchronize()
    assert int(y.abs().sum()) == 0   # nothing was launched
