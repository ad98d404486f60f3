"""Thin ctypes wrappers over the operator-level C ABI (include/cvm_hip_ops.h).

Arguments and results are int32 torch tensors on the GPU (torch only supplies
the device memory and the stream).  The names and argument meaning follow the
reference's operators (`cvm.runtime.<dev>.<op>`, src/runtime/cpu/ops), so a
parity test reads like the reference's tests/test_op.cc cases.
"""
import ctypes
import os

import torch

from . import check, lib

_i32p = ctypes.POINTER(ctypes.c_int32)
_i64p = ctypes.POINTER(ctypes.c_int64)

BCAST = {"broadcast_add": 0, "broadcast_sub": 1, "broadcast_mul": 2,
         "broadcast_max": 3, "broadcast_div": 4, "broadcast_greater": 5}


def _ptr(t):
    if t is None:
        return None
    assert t.is_cuda and t.dtype == torch.int32 and t.is_contiguous(), "int32 contiguous CUDA tensor required"
    return ctypes.cast(t.data_ptr(), _i32p)


def _apply_conv_tuning():
    """The library never reads the environment on a launch; this glue turns the test hooks CVM_HIP_CONV
    (lds | wave | big), CVM_HIP_WAVECFG (index) and CVM_HIP_TILE ("wm,wn"; with big: "t,0" picks tile t = 1..3)
    into the explicit per-thread setting."""
    kind = os.environ.get("CVM_HIP_CONV", "")
    cfg = os.environ.get("CVM_HIP_WAVECFG", "")
    tile = os.environ.get("CVM_HIP_TILE", "")
    wm, wn = (int(tile[0]), int(tile[2])) if len(tile) >= 3 and tile[1] == "," else (0, 0)
    check(lib().cvmhip_set_conv_tuning({"l": 1, "w": 2, "b": 3}.get(kind[:1], 0), int(cfg) if cfg.isdigit() else -1, wm, wn))


def _stream():
    _apply_conv_tuning()
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _shape(s):
    return (ctypes.c_int64 * max(len(s), 1))(*[int(v) for v in s])


def _new(shape, like):
    return torch.empty(tuple(int(v) for v in shape), dtype=torch.int32, device=like.device)


def _workspace(nbytes, dev):
    # 256-byte aligned scratch (torch's caching allocator aligns to 512)
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=dev)


def conv_out_hw(h, w, kh, kw, sh, sw, ph, pw, dh, dw):
    return ((h + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1,
            (w + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1)


def conv2d(x, w, b=None, strides=(1, 1), padding=(0, 0), dilation=(1, 1), groups=1):
    n, ic, h, wd = x.shape
    oc, _, kh, kw = w.shape
    oh, ow = conv_out_hw(h, wd, kh, kw, strides[0], strides[1], padding[0], padding[1], dilation[0], dilation[1])
    y = _new((n, oc, oh, ow), x)
    L = lib()
    nbytes = L.cvmhip_conv2d_workspace_bytes(n, ic, h, wd, oc, kh, kw, groups)
    ws = _workspace(nbytes, x.device)
    check(L.cvmhip_conv2d(_ptr(x), _ptr(w), _ptr(b), _ptr(y), n, ic, h, wd, oc, kh, kw,
                          strides[0], strides[1], padding[0], padding[1], dilation[0], dilation[1],
                          groups, ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(ws.numel()), _stream()))
    return y


def dense(x, w, b=None, operand_bits=8):
    m, k = x.shape
    n = w.shape[0]
    y = _new((m, n), x)
    L = lib()
    ws = _workspace(L.cvmhip_dense_workspace_bytes(m, k, n), x.device)
    check(L.cvmhip_dense(_ptr(x), _ptr(w), _ptr(b), _ptr(y), m, k, n, operand_bits,
                         ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(ws.numel()), _stream()))
    return y


def _unary(fn, x, *args, out=None):
    y = torch.empty_like(x) if out is None else out
    check(fn(_ptr(x), _ptr(y), ctypes.c_int64(x.numel()), *args, _stream()))
    return y


def relu(x, out=None):
    return _unary(lib().cvmhip_relu, x, out=out)


def cvm_clip(x, precision, out=None):
    return _unary(lib().cvmhip_cvm_clip, x, int(precision), out=out)


def cvm_right_shift(x, precision, shift_bit, out=None):
    return _unary(lib().cvmhip_cvm_right_shift, x, int(precision), int(shift_bit), out=out)


def cvm_left_shift(x, precision, shift_bit, out=None):
    return _unary(lib().cvmhip_cvm_left_shift, x, int(precision), int(shift_bit), out=out)


def clip(x, a_min, a_max, out=None):
    return _unary(lib().cvmhip_clip, x, ctypes.c_int32(a_min), ctypes.c_int32(a_max), out=out)


def abs_(x, out=None):
    return _unary(lib().cvmhip_abs, x, out=out)


def negative(x, out=None):
    return _unary(lib().cvmhip_negative, x, out=out)


def cvm_precision(x, out=None):
    return _unary(lib().cvmhip_cvm_precision, x, out=out)


def elemwise(op, a, b, out=None):
    c = torch.empty_like(a) if out is None else out
    check(lib().cvmhip_elemwise(0 if op == "elemwise_add" else 1, _ptr(a), _ptr(b), _ptr(c),
                                ctypes.c_int64(a.numel()), _stream()))
    return c


def broadcast_shape(sa, sb):
    nd = max(len(sa), len(sb))
    pa = (1,) * (nd - len(sa)) + tuple(sa)
    pb = (1,) * (nd - len(sb)) + tuple(sb)
    return tuple(max(u, v) for u, v in zip(pa, pb))


def broadcast(op, a, b):
    cs = broadcast_shape(a.shape, b.shape)
    c = _new(cs, a)
    check(lib().cvmhip_broadcast(BCAST[op], _ptr(a), _shape(a.shape), a.dim(), _ptr(b), _shape(b.shape),
                                 b.dim(), _ptr(c), _shape(cs), len(cs), _stream()))
    return c


def pool_out(h, k, s, p, ceil_mode):
    if ceil_mode:
        return (h + 2 * p - k + s - 1) // s + 1
    return (h + 2 * p - k) // s + 1


def max_pool2d(x, pool_size, strides=(1, 1), padding=(0, 0), ceil_mode=False):
    n, c, h, w = x.shape
    pad = list(padding)
    if len(pad) == 1:
        pad = [pad[0], pad[0]]
    oh = pool_out(h, pool_size[0], strides[0], pad[0], ceil_mode)
    ow = pool_out(w, pool_size[1], strides[1], pad[1], ceil_mode)
    y = _new((n, c, oh, ow), x)
    check(lib().cvmhip_max_pool2d(_ptr(x), _ptr(y), n, c, h, w, oh, ow, pool_size[0], pool_size[1],
                                  strides[0], strides[1], pad[0], pad[1], _stream()))
    return y


def reduce_shape(shape, axes, keepdims, exclude):
    nd = len(shape)
    ax = sorted(a + nd if a < 0 else a for a in axes)
    if not ax:
        r = list(range(nd))
    elif exclude:
        r = [i for i in range(nd) if i not in ax]
    else:
        r = ax
    if not r:
        return tuple(shape)
    if len(r) == nd:
        return (1,) * nd if keepdims else (1,)
    if keepdims:
        return tuple(1 if i in r else s for i, s in enumerate(shape))
    return tuple(s for i, s in enumerate(shape) if i not in r)


def reduce(op, x, axes=(), keepdims=False, exclude=False):
    ys = reduce_shape(x.shape, list(axes), keepdims, exclude)
    y = _new(ys, x)
    ax = _shape(list(axes)) if len(axes) else None
    check(lib().cvmhip_reduce(0 if op == "sum" else 1, _ptr(x), _shape(x.shape), x.dim(), _ptr(y),
                              ctypes.c_int64(y.numel()), ax, len(axes), int(bool(exclude)), _stream()))
    return y


def copy(x, shape):
    y = _new(shape, x)
    check(lib().cvmhip_copy(_ptr(x), _ptr(y), ctypes.c_int64(x.numel()), _stream()))
    return y


def concatenate(xs, axis):
    nd = xs[0].dim()
    ax = axis + nd if axis < 0 else axis
    ys = list(xs[0].shape)
    ys[ax] = sum(v.shape[ax] for v in xs)
    y = _new(ys, xs[0])
    n = len(xs)
    ptrs = (_i32p * n)(*[_ptr(v) for v in xs])
    shp = [_shape(v.shape) for v in xs]
    shps = (_i64p * n)(*[ctypes.cast(s, _i64p) for s in shp])
    check(lib().cvmhip_concatenate(ptrs, shps, n, nd, axis, _ptr(y), _shape(ys), _stream()))
    return y


def transpose(x, axes=()):
    nd = x.dim()
    perm = [a + nd if a < 0 else a for a in axes] if len(axes) else list(range(nd))[::-1]
    y = _new([x.shape[p] for p in perm], x)
    check(lib().cvmhip_transpose(_ptr(x), _shape(x.shape), nd, _shape(list(axes)) if len(axes) else None,
                                 len(axes), _ptr(y), _stream()))
    return y


def strided_slice(x, begin, end, stride, out_shape):
    y = _new(out_shape, x)
    check(lib().cvmhip_strided_slice(_ptr(x), _shape(x.shape), x.dim(), _shape(begin), len(begin),
                                     _shape(stride) if len(stride) else None, len(stride),
                                     _ptr(y), _shape(out_shape), _stream()))
    return y


def slice_like(x, out_shape):
    y = _new(out_shape, x)
    check(lib().cvmhip_slice_like(_ptr(x), _shape(x.shape), x.dim(), _ptr(y), _shape(out_shape), _stream()))
    return y


def take(x, indices, axis=None):
    if axis is None:
        ys = tuple(indices.shape)
    else:
        a = axis + x.dim() if axis < 0 else axis
        ys = tuple(x.shape[:a]) + tuple(indices.shape) + tuple(x.shape[a + 1:])
    y = _new(ys, x)
    check(lib().cvmhip_take(_ptr(x), _shape(x.shape), x.dim(), _ptr(indices), _shape(indices.shape),
                            indices.dim(), _ptr(y), _shape(ys), len(ys), int(axis is not None),
                            int(axis or 0), _stream()))
    return y


def repeat(x, repeats, axis=0):
    a = axis + x.dim() if axis < 0 else axis
    ys = list(x.shape)
    ys[a] *= repeats
    y = _new(ys, x)
    check(lib().cvmhip_repeat(_ptr(x), _shape(x.shape), _ptr(y), _shape(ys), x.dim(), axis, repeats, _stream()))
    return y


def tile(x, reps):
    nd = max(x.dim(), len(reps))
    xs = (1,) * (nd - x.dim()) + tuple(x.shape)
    rp = (1,) * (nd - len(reps)) + tuple(reps)
    ys = [a * b for a, b in zip(xs, rp)]
    y = _new(ys, x)
    check(lib().cvmhip_tile(_ptr(x), _shape(x.shape), x.dim(), _ptr(y), _shape(ys), nd, _stream()))
    return y


def upsampling(x, scale):
    n, c, h, w = x.shape
    y = _new((n, c, h * scale, w * scale), x)
    check(lib().cvmhip_upsampling(_ptr(x), _ptr(y), n, c, h, w, scale, _stream()))
    return y


def where(cond, x, y, out):
    check(lib().cvmhip_where(_ptr(cond), _ptr(x), _ptr(y), _ptr(out), _shape(x.shape), x.dim(),
                             int(cond.dim() == x.dim()), _stream()))
    return out


def get_valid_counts(x, score_threshold):
    b, n, k = x.shape
    vc = _new((b,), x)
    y = torch.empty_like(x)
    L = lib()
    ws = _workspace(L.cvmhip_get_valid_counts_workspace_bytes(b, n), x.device)
    check(L.cvmhip_get_valid_counts(_ptr(x), _ptr(vc), _ptr(y), b, n, k, ctypes.c_int32(score_threshold),
                                    ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(ws.numel()), _stream()))
    return vc, y


def non_max_suppression(x, valid_count, y, iou_threshold=50, force_suppress=False, top_k=-1,
                        id_index=0, coord_start=2, score_index=1, max_output_size=-1):
    """In place on y; x is mutated exactly as the reference mutates it."""
    b, n, k = x.shape
    L = lib()
    ws = _workspace(L.cvmhip_nms_workspace_bytes(b, n, k), x.device)
    check(L.cvmhip_non_max_suppression(_ptr(x), _ptr(valid_count), _ptr(y), b, n, k, max_output_size,
                                       iou_threshold, top_k, coord_start, score_index, id_index,
                                       int(bool(force_suppress)), ctypes.c_void_p(ws.data_ptr()),
                                       ctypes.c_size_t(ws.numel()), _stream()))
    return y


def non_max_suppression_static(x, valid_count, y, iou_threshold=50, force_suppress=False, top_k=-1,
                               id_index=0, coord_start=2, score_index=1, max_output_size=-1):
    """The same operator through the entry point that allocates nothing (scratch inside the library)."""
    b, n, k = x.shape
    check(lib().cvmhip_non_max_suppression_static(_ptr(x), _ptr(valid_count), _ptr(y), b, n, k, max_output_size,
                                                  iou_threshold, top_k, coord_start, score_index, id_index,
                                                  int(bool(force_suppress)), _stream()))
    return y


# ---------------------------------------------------------------- fused int8 path
# int8 activation tensors are flat torch int8 buffers in the library's own
# layout (NHWC for up to 16 padded channels, else blocks of 32 pixels x 32
# channels in MFMA fragment order; act_offset below restates it); filters are
# opaque byte buffers made by pack_weights / pack_depthwise_weights.

class Stage(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("precision", ctypes.c_int32), ("shift_bit", ctypes.c_int32),
                ("lo", ctypes.c_int32), ("hi", ctypes.c_int32)]


class Chain(ctypes.Structure):
    _fields_ = [("count", ctypes.c_int32), ("stage", Stage * 4)]


def chain(*stages):
    """stages: ("relu",) | ("cvm_right_shift", precision, shift_bit) | ("cvm_clip", precision) | ("clip", lo, hi)
    | ("mul", m)"""
    c = Chain()
    c.count = len(stages)
    for i, st in enumerate(stages):
        if st[0] == "relu":
            c.stage[i] = Stage(1, 0, 0, 0, 0)
        elif st[0] == "cvm_right_shift":
            c.stage[i] = Stage(2, st[1], st[2], 0, 0)
        elif st[0] == "cvm_clip":
            r = (1 << (st[1] - 1)) - 1
            c.stage[i] = Stage(3, 0, 0, -r, r)
        elif st[0] == "clip":
            c.stage[i] = Stage(3, 0, 0, st[1], st[2])
        elif st[0] == "mul":
            c.stage[i] = Stage(4, 0, 0, st[1], 0)
        else:
            raise ValueError(st)
    return c


def _vp(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def pad_channels(c):
    return lib().cvmhip_pad_channels(c)


def act_offset(p, c, cp):
    """Byte offset of channel c of pixel p (numpy arrays allowed) in an int8 activation buffer."""
    if cp % 32:
        return p * cp + c
    return ((p >> 5) * (cp >> 5) + (c >> 5)) * 1024 + ((c >> 4) & 1) * 512 + (p & 31) * 16 + (c & 15)


def _act_buffer(npix, c, dev):
    return torch.zeros(lib().cvmhip_packed_act_bytes(ctypes.c_int64(npix), c), dtype=torch.int8, device=dev)


def pack_act_i8(x):
    n, c, h, w = x.shape
    xp = _act_buffer(n * h * w, c, x.device)
    check(lib().cvmhip_pack_nhwc_i8(_ptr(x), _vp(xp), n, c, h * w, _stream()))
    return xp


def flatten_act_i8(xp, n, c, hw):
    """int8 act tensor of n images x hw pixels x c channels -> act tensor of n pixels x hw * c channels (cvmhip_flatten_act_i8)"""
    yp = _act_buffer(n, hw * c, xp.device)
    check(lib().cvmhip_flatten_act_i8(_vp(xp), _vp(yp), n, c, hw, _stream()))
    return yp


def unpack_act_i8(xp, n, c, h, w):
    x = torch.empty((n, c, h, w), dtype=torch.int32, device=xp.device)
    check(lib().cvmhip_unpack_nhwc_i8(_vp(xp), _ptr(x), n, c, h * w, _stream()))
    return x


def pack_weights(w):
    oc, ic, kh, kw = w.shape
    wp = _workspace(lib().cvmhip_packed_weight_bytes(oc, ic, kh, kw), w.device)
    check(lib().cvmhip_pack_weights(_ptr(w), _vp(wp), oc, ic, kh, kw, _stream()))
    return wp


def conv2d_i8(xp, n, ic, h, w, wp, oc, kh, kw, bias=None, chain1=None, residual=None, chain2=None, out_is_i8=True,
              strides=(1, 1), padding=(0, 0), dilation=(1, 1)):
    oh, ow = conv_out_hw(h, w, kh, kw, strides[0], strides[1], padding[0], padding[1], dilation[0], dilation[1])
    if out_is_i8:
        out = _act_buffer(n * oh * ow, oc, xp.device)
    else:
        out = torch.empty((n, oc, oh, ow), dtype=torch.int32, device=xp.device)
    check(lib().cvmhip_conv2d_i8(_vp(xp), _vp(wp), _ptr(bias), ctypes.byref(chain1) if chain1 else None,
                                 _vp(residual), ctypes.byref(chain2) if chain2 else None, _vp(out), int(out_is_i8),
                                 n, ic, h, w, oc, kh, kw, strides[0], strides[1], padding[0], padding[1],
                                 dilation[0], dilation[1], _stream()))
    return out


def conv2d_pool2_eligible(n, ic, h, w, oc, kh, kw, strides=(1, 1), padding=(0, 0), dilation=(1, 1)):
    return bool(lib().cvmhip_conv2d_pool2_i8_eligible(n, ic, h, w, oc, kh, kw, strides[0], strides[1], padding[0], padding[1],
                                                      dilation[0], dilation[1]))


def conv2d_pool2_i8(xp, n, ic, h, w, wp, oc, kh, kw, bias=None, chain1=None, strides=(1, 1), padding=(0, 0), dilation=(1, 1)):
    """conv2d + chain + max_pool2d(2x2, stride 2) in one launch; returns the pooled int8 act tensor."""
    oh, ow = conv_out_hw(h, w, kh, kw, strides[0], strides[1], padding[0], padding[1], dilation[0], dilation[1])
    out = _act_buffer(n * (oh // 2) * (ow // 2), oc, xp.device)
    check(lib().cvmhip_conv2d_pool2_i8(_vp(xp), _vp(wp), _ptr(bias), ctypes.byref(chain1) if chain1 else None, _vp(out),
                                       n, ic, h, w, oc, kh, kw, strides[0], strides[1], padding[0], padding[1],
                                       dilation[0], dilation[1], _stream()))
    return out


def conv2d_i8_ws(xp, n, ic, h, w, wp, oc, kh, kw, bias=None, chain1=None, out_is_i8=True,
                 strides=(1, 1), padding=(0, 0), dilation=(1, 1)):
    """conv2d_i8 with the workspace the library asks for (K slices over the grid for small-batch dense
    layers); returns (output, workspace bytes used)."""
    L = lib()
    L.cvmhip_conv2d_i8_workspace_bytes.restype = ctypes.c_size_t
    oh, ow = conv_out_hw(h, w, kh, kw, strides[0], strides[1], padding[0], padding[1], dilation[0], dilation[1])
    need = L.cvmhip_conv2d_i8_workspace_bytes(0, n, ic, h, w, oc, kh, kw, strides[0], strides[1], padding[0], padding[1],
                                              dilation[0], dilation[1])
    ws = _workspace(need, xp.device) if need else None
    if out_is_i8:
        out = _act_buffer(n * oh * ow, oc, xp.device)
    else:
        out = torch.empty((n, oc, oh, ow), dtype=torch.int32, device=xp.device)
    check(L.cvmhip_conv2d_i8_ws(_vp(xp), _vp(wp), _ptr(bias), ctypes.byref(chain1) if chain1 else None, None, None,
                                _vp(out), int(out_is_i8), n, ic, h, w, oc, kh, kw, strides[0], strides[1],
                                padding[0], padding[1], dilation[0], dilation[1], _vp(ws), ctypes.c_size_t(need), _stream()))
    return out, need


def conv2d_i8_nhwc(xp, n, ic, h, w, wp, oc, kh, kw, out, offset, image_stride, bias=None, chain1=None,
                   strides=(1, 1), padding=(0, 0), dilation=(1, 1)):
    """The convolution's int32 result written pixel-major into the flat int32 tensor `out`:
    image i's OH*OW*OC values start at element offset + i*image_stride."""
    check(lib().cvmhip_conv2d_i8_nhwc(_vp(xp), _vp(wp), _ptr(bias), ctypes.byref(chain1) if chain1 else None,
                                      ctypes.c_void_p(out.data_ptr() + 4 * offset), ctypes.c_int64(image_stride),
                                      n, ic, h, w, oc, kh, kw, strides[0], strides[1], padding[0], padding[1],
                                      dilation[0], dilation[1], _stream()))
    return out


def conv2d_stem_pool3_eligible(n, c, h, w, oc, kh, kw, strides, padding, pool_oh, pool_ow):
    return bool(lib().cvmhip_conv2d_stem_pool3_i8_eligible(n, c, h, w, oc, kh, kw, strides[0], strides[1], padding[0], padding[1],
                                                           pool_oh, pool_ow))


def conv2d_stem_pool3_i8(x, w, bias, chain1, strides, padding, pool_oh, pool_ow):
    """Row-window convolution + chain + max_pool2d(3x3, stride 2, padding 1) in one launch; x and w are int32 NCHW / OIHW
    device tensors; returns the pooled int8 act tensor."""
    L = lib()
    n, c, h, wd = x.shape
    oc, _, kh, kw = w.shape
    L.cvmhip_stem_input_bytes.restype = ctypes.c_size_t
    L.cvmhip_packed_stem_weight_bytes.restype = ctypes.c_size_t
    xs = _workspace(L.cvmhip_stem_input_bytes(n, h, wd, kh, kw, strides[0], strides[1], padding[0], padding[1]), x.device)
    wp = _workspace(L.cvmhip_packed_stem_weight_bytes(oc, kh, kw), x.device)
    check(L.cvmhip_pack_stem_input(_ptr(x), _vp(xs), n, c, h, wd, kh, kw, strides[0], strides[1], padding[0], padding[1], _stream()))
    check(L.cvmhip_pack_stem_weights(_ptr(w), _vp(wp), oc, c, kh, kw, _stream()))
    out = _act_buffer(n * pool_oh * pool_ow, oc, x.device)
    check(L.cvmhip_conv2d_stem_pool3_i8(_vp(xs), _vp(wp), _ptr(bias), ctypes.byref(chain1) if chain1 else None, _vp(out),
                                        n, c, h, wd, oc, kh, kw, strides[0], strides[1], padding[0], padding[1],
                                        pool_oh, pool_ow, _stream()))
    return out


def pack_weights_pair(w_a, w_b):
    """Two OIHW filters over the same input packed as one (the first one's rows padded to a multiple of 32)."""
    L = lib()
    oc_a, ic, kh, kw = w_a.shape
    oc_b = w_b.shape[0]
    L.cvmhip_packed_weight_pair_bytes.restype = ctypes.c_size_t
    wp = _workspace(L.cvmhip_packed_weight_pair_bytes(oc_a, oc_b, ic, kh, kw), w_a.device)
    check(L.cvmhip_pack_weights_pair(_ptr(w_a), oc_a, _ptr(w_b), oc_b, _vp(wp), ic, kh, kw, _stream()))
    return wp


def conv2d_i8_nhwc_pair(xp, n, ic, h, w, wp, kh, kw, out_a, offset_a, stride_a, oc_a, out_b, offset_b, stride_b, oc_b,
                        bias=None, chain1=None, strides=(1, 1), padding=(0, 0), dilation=(1, 1)):
    """Two detection heads over the same tensor in one launch; see conv2d_i8_nhwc for the meaning of offset / stride."""
    check(lib().cvmhip_conv2d_i8_nhwc_pair(_vp(xp), _vp(wp), _ptr(bias), ctypes.byref(chain1) if chain1 else None,
                                           ctypes.c_void_p(out_a.data_ptr() + 4 * offset_a), ctypes.c_int64(stride_a), oc_a,
                                           ctypes.c_void_p(out_b.data_ptr() + 4 * offset_b), ctypes.c_int64(stride_b), oc_b,
                                           n, ic, h, w, kh, kw, strides[0], strides[1], padding[0], padding[1],
                                           dilation[0], dilation[1], _stream()))


class HeadGroup:
    """Independent detection-head convolutions that share one launch (cvmhip_conv_group_heads / cvmhip_conv_group_launch)."""

    def __init__(self, device):
        L = lib()
        L.cvmhip_conv_group_layer_bytes.restype = ctypes.c_size_t
        self.entry = L.cvmhip_conv_group_layer_bytes()
        self.table = bytearray()
        self.count = 0
        self.blocks = 0
        self.device = device
        self.keep = []

    def add(self, xp, n, ic, h, w, wp, kh, kw, out_a, offset_a, stride_a, oc_a, out_b=None, offset_b=0, stride_b=0, oc_b=0,
            bias=None, chain1=None, strides=(1, 1), padding=(0, 0), dilation=(1, 1)):
        self.table.extend(bytes(self.entry))
        buf = (ctypes.c_char * len(self.table)).from_buffer(self.table)
        nb = ctypes.c_int()
        _apply_conv_tuning()
        rc = lib().cvmhip_conv_group_heads(buf, self.count, self.blocks, ctypes.byref(nb), _vp(xp), _vp(wp), _ptr(bias),
                                           ctypes.byref(chain1) if chain1 else None,
                                           ctypes.c_void_p(out_a.data_ptr() + 4 * offset_a), ctypes.c_int64(stride_a), oc_a,
                                           ctypes.c_void_p(out_b.data_ptr() + 4 * offset_b) if out_b is not None else None,
                                           ctypes.c_int64(stride_b), oc_b, n, ic, h, w, kh, kw, strides[0], strides[1],
                                           padding[0], padding[1], dilation[0], dilation[1])
        del buf
        if rc != 0:
            del self.table[-self.entry:]
        check(rc)
        self.count += 1
        self.blocks += nb.value
        self.keep += [xp, wp, bias, out_a, out_b]

    def add_conv_i8(self, xp, n, ic, h, w, wp, oc, kh, kw, bias=None, chain1=None, residual=None, chain2=None,
                    strides=(1, 1), padding=(0, 0), dilation=(1, 1)):
        """An entry with int8 output (what conv2d_i8 would compute); returns the output buffer.  A table holds either such
        entries or head entries; launch with launch(i8=True)."""
        oh, ow = conv_out_hw(h, w, kh, kw, strides[0], strides[1], padding[0], padding[1], dilation[0], dilation[1])
        out = _act_buffer(n * oh * ow, oc, xp.device)
        self.table.extend(bytes(self.entry))
        buf = (ctypes.c_char * len(self.table)).from_buffer(self.table)
        nb = ctypes.c_int()
        _apply_conv_tuning()
        rc = lib().cvmhip_conv_group_conv_i8(buf, self.count, self.blocks, ctypes.byref(nb), _vp(xp), _vp(wp), _ptr(bias),
                                             ctypes.byref(chain1) if chain1 else None, _vp(residual),
                                             ctypes.byref(chain2) if chain2 else None, _vp(out), n, ic, h, w, oc, kh, kw,
                                             strides[0], strides[1], padding[0], padding[1], dilation[0], dilation[1])
        del buf
        if rc != 0:
            del self.table[-self.entry:]
        check(rc)
        self.count += 1
        self.blocks += nb.value
        self.keep += [xp, wp, bias, residual, out]
        return out

    def launch(self, i8=False):
        dev = torch.frombuffer(bytearray(self.table), dtype=torch.uint8).to(self.device)
        if i8:
            check(lib().cvmhip_conv_group_launch_i8(_vp(dev), self.count, self.blocks, ctypes.c_double(0), ctypes.c_double(0), _stream()))
            torch.cuda.synchronize()
            return
        check(lib().cvmhip_conv_group_launch(_vp(dev), self.count, self.blocks, ctypes.c_double(0), ctypes.c_double(0), _stream()))
        torch.cuda.synchronize()


def pack_depthwise_weights(w):
    c, one, kh, kw = w.shape
    wp = _workspace(lib().cvmhip_packed_depthwise_bytes(c, kh, kw), w.device)
    check(lib().cvmhip_pack_depthwise_weights(_ptr(w), _vp(wp), c, kh, kw, _stream()))
    return wp


def depthwise_mfma_eligible(c, kh, kw):
    return bool(lib().cvmhip_depthwise_mfma_eligible(c, kh, kw))


def pack_depthwise_weights_mfma(w):
    c, one, kh, kw = w.shape
    L = lib()
    L.cvmhip_packed_depthwise_mfma_bytes.restype = ctypes.c_size_t
    wp = _workspace(L.cvmhip_packed_depthwise_mfma_bytes(c, kh, kw), w.device)
    check(L.cvmhip_pack_depthwise_weights_mfma(_ptr(w), _vp(wp), c, kh, kw, _stream()))
    return wp


def depthwise_conv2d_mfma_i8(xp, n, c, h, w, wp, kh, kw, bias=None, chain1=None, out_is_i8=True,
                             strides=(1, 1), padding=(0, 0), dilation=(1, 1)):
    """depthwise_conv2d_i8 through the implicit-GEMM kernel (diagonal filter blocks); wp from
    pack_depthwise_weights_mfma."""
    oh, ow = conv_out_hw(h, w, kh, kw, strides[0], strides[1], padding[0], padding[1], dilation[0], dilation[1])
    if out_is_i8:
        out = _act_buffer(n * oh * ow, c, xp.device)
    else:
        out = torch.empty((n, c, oh, ow), dtype=torch.int32, device=xp.device)
    check(lib().cvmhip_depthwise_conv2d_mfma_i8(_vp(xp), _vp(wp), _ptr(bias), ctypes.byref(chain1) if chain1 else None,
                                                _vp(out), int(out_is_i8), n, c, h, w, kh, kw, strides[0], strides[1],
                                                padding[0], padding[1], dilation[0], dilation[1], _stream()))
    return out


def depthwise_conv2d_i8(xp, n, c, h, w, wp, kh, kw, bias=None, chain1=None, out_is_i8=True,
                        strides=(1, 1), padding=(0, 0), dilation=(1, 1)):
    oh, ow = conv_out_hw(h, w, kh, kw, strides[0], strides[1], padding[0], padding[1], dilation[0], dilation[1])
    if out_is_i8:
        out = _act_buffer(n * oh * ow, c, xp.device)
    else:
        out = torch.empty((n, c, oh, ow), dtype=torch.int32, device=xp.device)
    check(lib().cvmhip_depthwise_conv2d_i8(_vp(xp), _vp(wp), _ptr(bias), ctypes.byref(chain1) if chain1 else None,
                                           _vp(out), int(out_is_i8), n, c, h, w, kh, kw, strides[0], strides[1],
                                           padding[0], padding[1], dilation[0], dilation[1], _stream()))
    return out


def add_i8(a, b, n, c, h, w, chain1=None, out_is_i8=True, out=None):
    if out is not None:
        pass
    elif out_is_i8:
        out = torch.zeros_like(a)
    else:
        out = torch.empty((n, c, h, w), dtype=torch.int32, device=a.device)
    check(lib().cvmhip_add_i8(_vp(a), _vp(b), ctypes.byref(chain1) if chain1 else None, _vp(out), int(out_is_i8),
                              n, c, h * w, _stream()))
    return out


def max_pool2d_i8(xp, n, c, h, w, pool_size, strides, padding, oh, ow, out=None):
    if out is None:
        out = _act_buffer(n * oh * ow, c, xp.device)
    check(lib().cvmhip_max_pool2d_i8(_vp(xp), _vp(out), n, c, h, w, oh, ow, pool_size[0], pool_size[1],
                                     strides[0], strides[1], padding[0], padding[1], _stream()))
    return out


def sum_hw_i8(xp, n, c, hw, chain1=None, out_is_i8=False, out=None):
    if out is not None:
        pass
    elif out_is_i8:
        out = _act_buffer(n, c, xp.device)
    else:
        out = torch.empty((n, c), dtype=torch.int32, device=xp.device)
    check(lib().cvmhip_sum_hw_i8(_vp(xp), ctypes.byref(chain1) if chain1 else None, _vp(out), int(out_is_i8),
                                 n, c, hw, _stream()))
    return out


def conv2d_stem_i8(x, w, bias=None, chain1=None, out_is_i8=True, strides=(1, 1), padding=(0, 0)):
    """conv2d over <= 4 input channels in row-window form; x and w are int32 NCHW / OIHW device tensors."""
    L = lib()
    n, c, h, wd = x.shape
    oc, _, kh, kw = w.shape
    L.cvmhip_stem_input_bytes.restype = ctypes.c_size_t
    L.cvmhip_packed_stem_weight_bytes.restype = ctypes.c_size_t
    assert L.cvmhip_stem_eligible(c, kh, kw, 1, 1)
    xs = _workspace(L.cvmhip_stem_input_bytes(n, h, wd, kh, kw, strides[0], strides[1], padding[0], padding[1]), x.device)
    wp = _workspace(L.cvmhip_packed_stem_weight_bytes(oc, kh, kw), x.device)
    check(L.cvmhip_pack_stem_input(_ptr(x), _vp(xs), n, c, h, wd, kh, kw, strides[0], strides[1], padding[0], padding[1], _stream()))
    check(L.cvmhip_pack_stem_weights(_ptr(w), _vp(wp), oc, c, kh, kw, _stream()))
    oh, ow = conv_out_hw(h, wd, kh, kw, strides[0], strides[1], padding[0], padding[1], 1, 1)
    if out_is_i8:
        out = _act_buffer(n * oh * ow, oc, x.device)
    else:
        out = torch.empty((n, oc, oh, ow), dtype=torch.int32, device=x.device)
    check(L.cvmhip_conv2d_stem_i8(_vp(xs), _vp(wp), _ptr(bias), ctypes.byref(chain1) if chain1 else None, _vp(out),
                                  int(out_is_i8), n, c, h, wd, oc, kh, kw, strides[0], strides[1], padding[0], padding[1],
                                  _stream()))
    return out
