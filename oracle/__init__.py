"""TEST INFRASTRUCTURE ONLY: ctypes access to the CPU oracle.

`liboracle.so` is the C restatement of the reference CPU operators
(cvm_oracle.c).  `_ref/libref_driver.so` drives the *compiled reference
runtime* itself and only exists where it was built from /root/reference.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package.  The product package never does.
"""
import ctypes
import json
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_REF = None

i32p = ctypes.POINTER(ctypes.c_int32)
i64p = ctypes.POINTER(ctypes.c_int64)

BCAST = {"broadcast_add": 0, "broadcast_sub": 1, "broadcast_mul": 2,
         "broadcast_max": 3, "broadcast_div": 4, "broadcast_greater": 5}


def build():
    """Compile liboracle.so (and _ref/ when /root/reference is present)."""
    subprocess.check_call(["make", "-C", _HERE, "-j8", "all"], stdout=subprocess.DEVNULL)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
        _LIB.cvmo_iou.restype = ctypes.c_int64
    return _LIB


def have_ref():
    return os.path.exists(os.path.join(_HERE, "_ref", "libref_driver.so"))


def ref():
    global _REF
    if _REF is None:
        _REF = ctypes.CDLL(os.path.join(_HERE, "_ref", "libref_driver.so"))
    return _REF


def _a(x):
    return np.ascontiguousarray(x, dtype=np.int32)


def _p(x):
    return x.ctypes.data_as(i32p)


def _shape(s):
    arr = (ctypes.c_int64 * max(len(s), 1))(*[int(v) for v in s])
    return arr


# ----------------------------------------------------------------------------
# attribute parsing helpers (attrs are the graph JSON's string-valued dicts)
def parse_tuple(s, default=None):
    if s is None:
        return default
    s = s.strip()
    if s in ("None", ""):
        return default
    s = s.strip("()[]")
    return [int(v) for v in s.replace(" ", "").split(",") if v != ""]


def parse_bool(s, default):
    if s is None:
        return default
    return s.strip() in ("True", "true", "1")


def conv_out_hw(h, w, kh, kw, sh, sw, ph, pw, dh, dw):
    return ((h + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1,
            (w + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1)


# ----------------------------------------------------------------------------
# One function per operator: numpy in, numpy out.
def conv2d(x, w, b, strides=(1, 1), padding=(0, 0), dilation=(1, 1), groups=1):
    x, w = _a(x), _a(w)
    n, ic, h, wd = x.shape
    oc, _, kh, kw = w.shape
    oh, ow = conv_out_hw(h, wd, kh, kw, strides[0], strides[1], padding[0], padding[1],
                         dilation[0], dilation[1])
    y = np.empty((n, oc, oh, ow), np.int32)
    bb = _a(b) if b is not None else None
    rc = lib().cvmo_conv2d(_p(x), _p(w), _p(bb) if bb is not None else None, _p(y),
                           n, ic, h, wd, oc, kh, kw, strides[0], strides[1],
                           padding[0], padding[1], dilation[0], dilation[1], groups)
    assert rc == 0, rc
    return y


def dense(x, w, b):
    x, w = _a(x), _a(w)
    m, k = x.shape
    n = w.shape[0]
    y = np.empty((m, n), np.int32)
    bb = _a(b) if b is not None else None
    rc = lib().cvmo_dense(_p(x), _p(w), _p(bb) if bb is not None else None, _p(y), m, k, n)
    assert rc == 0
    return y


def _unary(fn, x, *args):
    x = _a(x)
    y = np.empty_like(x)
    rc = fn(_p(x), _p(y), ctypes.c_int64(x.size), *args)
    assert rc == 0, rc
    return y


def relu(x):
    return _unary(lib().cvmo_relu, x)


def cvm_clip(x, precision):
    return _unary(lib().cvmo_cvm_clip, x, int(precision))


def cvm_right_shift(x, precision, shift_bit):
    return _unary(lib().cvmo_cvm_right_shift, x, int(precision), int(shift_bit))


def cvm_left_shift(x, precision, shift_bit):
    return _unary(lib().cvmo_cvm_left_shift, x, int(precision), int(shift_bit))


def clip(x, a_min, a_max):
    return _unary(lib().cvmo_clip, x, ctypes.c_int32(a_min), ctypes.c_int32(a_max))


def abs_(x):
    return _unary(lib().cvmo_abs, x)


def negative(x):
    return _unary(lib().cvmo_negative, x)


def cvm_precision(x):
    return _unary(lib().cvmo_cvm_precision, x)


def elemwise(op, a, b):
    a, b = _a(a), _a(b)
    c = np.empty_like(a)
    rc = lib().cvmo_elemwise({"elemwise_add": 0, "elemwise_sub": 1}[op], _p(a), _p(b), _p(c),
                             ctypes.c_int64(a.size))
    assert rc == 0
    return c


def broadcast_shape(sa, sb):
    nd = max(len(sa), len(sb))
    pa = (1,) * (nd - len(sa)) + tuple(sa)
    pb = (1,) * (nd - len(sb)) + tuple(sb)
    return tuple(max(u, v) for u, v in zip(pa, pb))


def broadcast(op, a, b):
    a, b = _a(a), _a(b)
    cs = broadcast_shape(a.shape, b.shape)
    c = np.empty(cs, np.int32)
    rc = lib().cvmo_broadcast(BCAST[op], _p(a), _shape(a.shape), a.ndim, _p(b), _shape(b.shape),
                              b.ndim, _p(c), _shape(cs), len(cs))
    assert rc == 0
    return c


def pool_out(h, k, s, p, ceil_mode):
    if ceil_mode:
        return (h + 2 * p - k + s - 1) // s + 1
    return (h + 2 * p - k) // s + 1


def max_pool2d(x, pool_size, strides=(1, 1), padding=(0, 0), ceil_mode=False):
    x = _a(x)
    n, c, h, w = x.shape
    pad = list(padding)
    if len(pad) == 1:
        pad = [pad[0], pad[0]]
    oh = pool_out(h, pool_size[0], strides[0], pad[0], ceil_mode)
    ow = pool_out(w, pool_size[1], strides[1], pad[1], ceil_mode)
    y = np.empty((n, c, oh, ow), np.int32)
    rc = lib().cvmo_max_pool2d(_p(x), _p(y), n, c, h, w, oh, ow, pool_size[0], pool_size[1],
                               strides[0], strides[1], pad[0], pad[1])
    assert rc == 0
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
    x = _a(x)
    ys = reduce_shape(x.shape, list(axes), keepdims, exclude)
    y = np.empty(ys, np.int32)
    ax = _shape(list(axes)) if len(axes) else None
    rc = lib().cvmo_reduce(0 if op == "sum" else 1, _p(x), _shape(x.shape), x.ndim, _p(y),
                           ctypes.c_int64(y.size), ax, len(axes), int(bool(exclude)))
    assert rc == 0, rc
    return y


def concatenate(xs, axis):
    xs = [_a(v) for v in xs]
    nd = xs[0].ndim
    ax = axis + nd if axis < 0 else axis
    ys = list(xs[0].shape)
    ys[ax] = sum(v.shape[ax] for v in xs)
    y = np.empty(ys, np.int32)
    n = len(xs)
    ptrs = (i32p * n)(*[_p(v) for v in xs])
    shp = [_shape(v.shape) for v in xs]
    shps = (i64p * n)(*[ctypes.cast(s, i64p) for s in shp])
    rc = lib().cvmo_concatenate(ptrs, shps, n, nd, axis, _p(y), _shape(ys))
    assert rc == 0
    return y


def transpose(x, axes=()):
    x = _a(x)
    nd = x.ndim
    perm = [a + nd if a < 0 else a for a in axes] if len(axes) else list(range(nd))[::-1]
    ys = [x.shape[p] for p in perm]
    y = np.empty(ys, np.int32)
    rc = lib().cvmo_transpose(_p(x), _shape(x.shape), nd, _shape(list(axes)) if len(axes) else None,
                              len(axes), _p(y))
    assert rc == 0
    return y


def strided_slice_shape(shape, begin, end, stride):
    nd = len(shape)
    b = list(begin) + [0] * (nd - len(begin))
    e = list(end) + list(shape[len(end):])
    s = list(stride) + [1] * (nd - len(stride))
    out = []
    for i in range(nd):
        lo, hi = (-1, shape[i] - 1) if s[i] < 0 else (0, shape[i])
        bb = b[i] + shape[i] if b[i] < 0 else b[i]
        ee = e[i] + shape[i] if e[i] < 0 else e[i]
        bb = min(max(bb, lo), hi)
        ee = min(max(ee, lo), hi)
        out.append((abs(ee - bb) + abs(s[i]) - 1) // abs(s[i]))
    return tuple(out)


def strided_slice(x, begin, end, stride=()):
    x = _a(x)
    ys = strided_slice_shape(x.shape, begin, end, stride)
    y = np.empty(ys, np.int32)
    rc = lib().cvmo_strided_slice(_p(x), _shape(x.shape), x.ndim, _shape(begin), len(begin),
                                  _shape(stride) if len(stride) else None, len(stride),
                                  _p(y), _shape(ys))
    assert rc == 0
    return y


def slice_like(x, like_shape, axis=()):
    x = _a(x)
    ys = list(x.shape)
    if len(axis) == 0:
        for i in range(min(x.ndim, len(like_shape))):
            ys[i] = like_shape[i]
    else:
        for a in axis:
            a = a + x.ndim if a < 0 else a
            ys[a] = like_shape[a]
    y = np.empty(ys, np.int32)
    rc = lib().cvmo_slice_like(_p(x), _shape(x.shape), x.ndim, _p(y), _shape(ys))
    assert rc == 0
    return y


def take(x, indices, axis=None):
    x, indices = _a(x), _a(indices)
    if axis is None:
        ys = indices.shape
    else:
        a = axis + x.ndim if axis < 0 else axis
        ys = x.shape[:a] + indices.shape + x.shape[a + 1:]
    y = np.empty(ys, np.int32)
    rc = lib().cvmo_take(_p(x), _shape(x.shape), x.ndim, _p(indices), _shape(indices.shape),
                         indices.ndim, _p(y), _shape(ys), len(ys), int(axis is not None),
                         int(axis or 0))
    assert rc == 0
    return y


def repeat(x, repeats, axis=0):
    x = _a(x)
    a = axis + x.ndim if axis < 0 else axis
    ys = list(x.shape)
    ys[a] *= repeats
    y = np.empty(ys, np.int32)
    rc = lib().cvmo_repeat(_p(x), _shape(x.shape), _p(y), _shape(ys), x.ndim, axis, repeats)
    assert rc == 0
    return y


def tile(x, reps):
    x = _a(x)
    nd = max(x.ndim, len(reps))
    xs = (1,) * (nd - x.ndim) + x.shape
    rp = (1,) * (nd - len(reps)) + tuple(reps)
    ys = [a * b for a, b in zip(xs, rp)]
    y = np.empty(ys, np.int32)
    rc = lib().cvmo_tile(_p(x), _shape(x.shape), x.ndim, _p(y), _shape(ys), nd)
    assert rc == 0
    return y


def upsampling(x, scale):
    x = _a(x)
    n, c, h, w = x.shape
    y = np.empty((n, c, h * scale, w * scale), np.int32)
    rc = lib().cvmo_upsampling(_p(x), _p(y), n, c, h, w, scale)
    assert rc == 0
    return y


def where(cond, x, y, out_init=None):
    cond, x, y = _a(cond), _a(x), _a(y)
    out = np.zeros_like(x) if out_init is None else _a(out_init).copy()
    rc = lib().cvmo_where(_p(cond), _p(x), _p(y), _p(out), _shape(x.shape), x.ndim,
                          int(cond.ndim == x.ndim))
    assert rc == 0
    return out


def get_valid_counts(x, score_threshold):
    x = _a(x)
    b, n, k = x.shape
    vc = np.empty((b,), np.int32)
    y = np.empty_like(x)
    rc = lib().cvmo_get_valid_counts(_p(x), _p(vc), _p(y), b, n, k, ctypes.c_int32(score_threshold))
    assert rc == 0
    return vc, y


def iou(r1, r2):
    r1, r2 = _a(r1), _a(r2)
    return int(lib().cvmo_iou(_p(r1), _p(r2)))


def non_max_suppression(x, valid_count, iou_threshold=50, force_suppress=False, top_k=-1,
                        id_index=0, coord_start=2, score_index=1, max_output_size=-1,
                        y_init=None):
    """Returns (y, x_after): the reference mutates x when 0 < top_k < valid_count."""
    x = _a(x).copy()
    vc = _a(valid_count)
    b, n, k = x.shape
    y = np.zeros_like(x) if y_init is None else _a(y_init).copy()
    rc = lib().cvmo_non_max_suppression(_p(x), _p(vc), _p(y), b, n, k, max_output_size,
                                        iou_threshold, top_k, coord_start, score_index, id_index,
                                        int(bool(force_suppress)))
    assert rc == 0, rc
    return y, x


# ----------------------------------------------------------------------------
# Operator dispatch by (name, attrs) -- the same view a graph node gives.
def run_op(op, attrs, ins, out_init=None):
    """Run one operator by graph name with string-valued attrs; returns a list of outputs."""
    a = attrs
    if op == "conv2d":
        use_bias = parse_bool(a.get("use_bias"), True)
        return [conv2d(ins[0], ins[1], ins[2] if use_bias else None,
                       parse_tuple(a.get("strides"), [1, 1]), parse_tuple(a.get("padding"), [0, 0]),
                       parse_tuple(a.get("dilation"), [1, 1]), int(a.get("groups", "1")))]
    if op == "dense":
        use_bias = parse_bool(a.get("use_bias"), True)
        return [dense(ins[0], ins[1], ins[2] if use_bias else None)]
    if op == "relu":
        return [relu(ins[0])]
    if op == "cvm_clip":
        return [cvm_clip(ins[0], int(a["precision"]))]
    if op == "cvm_right_shift":
        return [cvm_right_shift(ins[0], int(a["precision"]), int(a["shift_bit"]))]
    if op == "cvm_left_shift":
        return [cvm_left_shift(ins[0], int(a["precision"]), int(a["shift_bit"]))]
    if op == "clip":
        return [clip(ins[0], int(a["a_min"]), int(a["a_max"]))]
    if op == "abs":
        return [abs_(ins[0])]
    if op == "negative":
        return [negative(ins[0])]
    if op == "cvm_precision":
        return [cvm_precision(ins[0])]
    if op in ("elemwise_add", "elemwise_sub"):
        return [elemwise(op, ins[0], ins[1])]
    if op in BCAST:
        return [broadcast(op, ins[0], ins[1])]
    if op == "max_pool2d":
        return [max_pool2d(ins[0], parse_tuple(a["pool_size"]), parse_tuple(a.get("strides"), [1, 1]),
                           parse_tuple(a.get("padding"), [0, 0]), parse_bool(a.get("ceil_mode"), False))]
    if op in ("sum", "max"):
        return [reduce(op, ins[0], parse_tuple(a.get("axis"), []), parse_bool(a.get("keepdims"), False),
                       parse_bool(a.get("exclude"), False))]
    if op == "flatten":
        x = _a(ins[0])
        return [x.reshape(x.shape[0], -1).copy()]
    if op == "reshape":
        return [_a(ins[0]).reshape(reshape_shape(ins[0].shape, parse_tuple(a["shape"]))).copy()]
    if op == "expand_dims":
        x = _a(ins[0])
        ax = int(a["axis"])
        ax = ax + x.ndim + 1 if ax < 0 else ax
        nn = int(a.get("num_newaxis", "1"))
        return [x.reshape(x.shape[:ax] + (1,) * nn + x.shape[ax:]).copy()]
    if op == "squeeze":
        x = _a(ins[0])
        ax = parse_tuple(a.get("axis"), [])
        if not ax:
            shp = tuple(s for s in x.shape if s != 1)
        else:
            ax = [v + x.ndim if v < 0 else v for v in ax]
            shp = tuple(s for i, s in enumerate(x.shape) if i not in ax)
        return [x.reshape(shp or (1,)).copy()]
    if op == "concatenate":
        return [concatenate(ins, int(a.get("axis", "1")))]
    if op == "transpose":
        return [transpose(ins[0], parse_tuple(a.get("axes"), []))]
    if op == "strided_slice":
        return [strided_slice(ins[0], parse_tuple(a["begin"]), parse_tuple(a["end"]),
                              parse_tuple(a.get("stride"), []))]
    if op == "slice_like":
        return [slice_like(ins[0], ins[1].shape, parse_tuple(a.get("axis"), []))]
    if op == "take":
        ax = a.get("axis")
        return [take(ins[0], ins[1], None if ax in (None, "None") else int(ax))]
    if op == "cvm_lut":
        return [take(ins[1], ins[0], None)]
    if op == "repeat":
        return [repeat(ins[0], int(a["repeats"]), int(a.get("axis", "0")))]
    if op == "tile":
        return [tile(ins[0], parse_tuple(a["reps"]))]
    if op == "upsampling":
        return [upsampling(ins[0], int(a["scale"]))]
    if op == "where":
        return [where(ins[0], ins[1], ins[2], out_init)]
    if op == "get_valid_counts":
        vc, y = get_valid_counts(ins[0], int(a.get("score_threshold", "0")))
        return [vc, y]
    if op == "non_max_suppression":
        y, _ = non_max_suppression(
            ins[0], ins[1], int(a.get("iou_threshold", "50")), parse_bool(a.get("force_suppress"), False),
            int(a.get("top_k", "-1")), int(a.get("id_index", "0")), int(a.get("coord_start", "2")),
            int(a.get("score_index", "1")), int(a.get("max_output_size", "-1")), out_init)
        return [y]
    raise KeyError(op)


def reshape_shape(dshape, target):
    """ReshapeInferShape, src/top/tensor/transform.cc (special values 0,-1,-2,-3,-4)."""
    dshape = list(dshape)
    out, src, infer = [], 0, -1
    i = 0
    while i < len(target):
        s = target[i]
        if s > 0:
            out.append(s); src += 1
        elif s == 0:
            out.append(dshape[src]); src += 1
        elif s == -1:
            infer = len(out); out.append(1); src += 1
        elif s == -2:
            out.extend(dshape[src:]); src = len(dshape)
        elif s == -3:
            out.append(dshape[src] * dshape[src + 1]); src += 2
        elif s == -4:
            d0 = dshape[src]; src += 1
            d1, d2 = target[i + 1], target[i + 2]; i += 2
            if d1 == -1: d1 = d0 // d2
            if d2 == -1: d2 = d0 // d1
            out.extend([d1, d2])
        i += 1
    if infer >= 0:
        out[infer] = int(np.prod(dshape)) // int(np.prod(out))
    return tuple(out)


# ----------------------------------------------------------------------------
# The compiled reference, one operator at a time.
class _RefTensor(ctypes.Structure):
    _fields_ = [("data", i32p), ("ndim", ctypes.c_int32), ("shape", ctypes.c_int64 * 6)]


def _rt(arr):
    t = _RefTensor()
    t.data = _p(arr) if arr is not None else None
    t.ndim = arr.ndim
    for i, s in enumerate(arr.shape):
        t.shape[i] = s
    return t


def ref_run_op(op, attrs, ins, outs, dev="cpu"):
    """Call cvm.runtime.<dev>.<op> of the compiled reference in place on `outs`.
    Returns (status, message)."""
    ins = [_a(v) for v in ins]
    n = len(ins) + len(outs)
    ts = (_RefTensor * n)(*([_rt(v) for v in ins] + [_rt(v) for v in outs]))
    err = ctypes.create_string_buffer(4096)
    rc = ref().ref_op_call(dev.encode(), op.encode(), json.dumps(attrs).encode(), len(ins),
                           len(outs), ts, err, 4096)
    return rc, err.value.decode(errors="replace")


def ref_infer(op, attrs, in_shapes, in_precs=None):
    """Reference FInferShape + FInferPrecision for one node (shapes only when
    `in_precs` is None).  Returns (status, out_shapes, out_precs, message)."""
    n = len(in_shapes)
    ins = (_RefTensor * max(n, 1))()
    for i, s in enumerate(in_shapes):
        ins[i].ndim = len(s)
        for d, v in enumerate(s):
            ins[i].shape[d] = v
    outs = (_RefTensor * 4)()
    ip = (ctypes.c_int * max(n, 1))(*in_precs) if in_precs is not None else None
    op_ = (ctypes.c_int * 4)()
    nout = ctypes.c_int(0)
    err = ctypes.create_string_buffer(4096)
    rc = ref().ref_op_infer(op.encode(), json.dumps(attrs).encode(), n, ins, ip, 4,
                            ctypes.byref(nout), outs, op_, err, 4096)
    shapes = [tuple(outs[i].shape[d] for d in range(outs[i].ndim)) for i in range(nout.value)]
    return rc, shapes, [op_[i] for i in range(nout.value)], err.value.decode(errors="replace")
