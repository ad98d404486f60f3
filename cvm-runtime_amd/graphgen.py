"""Synthetic CVM models: graph JSON + parameter blob in the reference's formats.

The reference ships no models (its tests read /data/... on the authors'
machines), so the benchmark configurations are generated here: random int8
weights from named splitmix64 streams, per-layer right shifts chosen from the
layer's fan-in so activations stay spread over 8 bits, graph JSON with the keys
`GraphCompile` emits (src/compiler/graph_compile.cc:92-215) and that
CvmRuntime::Load reads (src/runtime/graph_runtime.h:204-436), parameters in the
`CVMSaveParamsDict` layout (src/runtime/param_dict.cc:40-55,
include/cvm/runtime/ndarray.h:430-483).
"""
import json
import math
import struct

import numpy as np

from . import synth

LIST_MAGIC = 0xF7E58D4F05049CB7
ARRAY_MAGIC = 0xDD5E40F096B4A13F

# operators whose output may share its input's storage (graph_runtime.cc:150-157)
_INPLACE = {"relu", "cvm_clip", "cvm_right_shift", "cvm_left_shift", "clip", "flatten", "reshape",
            "expand_dims", "squeeze", "elemwise_add"}


def save_params(params):
    """params: list of (name, ndarray int8|int32) -> bytes."""
    out = [struct.pack("<QQ", LIST_MAGIC, 0), struct.pack("<Q", len(params))]
    for name, _ in params:
        b = name.encode()
        out.append(struct.pack("<Q", len(b)) + b)
    out.append(struct.pack("<Q", len(params)))
    for _, arr in params:
        arr = np.ascontiguousarray(arr)
        bits = 8 if arr.dtype == np.int8 else 32
        assert arr.dtype in (np.int8, np.int32)
        out.append(struct.pack("<QQ", ARRAY_MAGIC, 0))
        out.append(struct.pack("<iii", 1, 0, arr.ndim))         # DLContext{kDLCPU, 0}, ndim
        out.append(struct.pack("<BBH", 0, bits, 1))             # DLDataType{kDLInt, bits, lanes}
        out.append(struct.pack("<%dq" % arr.ndim, *arr.shape))
        out.append(struct.pack("<q", arr.nbytes))
        out.append(arr.tobytes())
    return b"".join(out)


def load_params(blob):
    """Inverse of save_params (used by the oracle-side graph executor and tests)."""
    off = 0

    def rd(fmt):
        nonlocal off
        v = struct.unpack_from(fmt, blob, off)
        off += struct.calcsize(fmt)
        return v
    magic, _ = rd("<QQ")
    assert magic == LIST_MAGIC
    (n,) = rd("<Q")
    names = []
    for _ in range(n):
        (ln,) = rd("<Q")
        names.append(blob[off:off + ln].decode())
        off += ln
    (n2,) = rd("<Q")
    assert n2 == n
    out = {}
    for name in names:
        magic, _ = rd("<QQ")
        assert magic == ARRAY_MAGIC
        _, _, ndim = rd("<iii")
        _, bits, _ = rd("<BBH")
        shape = rd("<%dq" % ndim)
        (nbytes,) = rd("<q")
        dt = np.int8 if bits == 8 else np.int32
        out[name] = np.frombuffer(blob, dt, nbytes // (bits // 8), off).reshape(shape).astype(np.int32)
        off += nbytes
    return out


def conv_out(h, k, s, p, d=1):
    return (h + 2 * p - (d * (k - 1) + 1)) // s + 1


def shift_for(fan_in, sigma_in=40.0, sigma_w=73.3, target=40.0):
    """Right shift that maps an accumulator of `fan_in` random products to ~target spread."""
    sigma = math.sqrt(fan_in) * sigma_in * sigma_w
    return max(1, int(round(math.log2(sigma / target))))


class GraphBuilder:
    """Accumulates nodes in topological order and emits graph JSON + params."""

    def __init__(self, config_id):
        self.cid = config_id
        self.nodes = []        # dicts: op, name, inputs, attrs(str dict), func
        self.shapes = []       # per entry
        self.precs = []        # per entry (-1 for operator outputs)
        self.row_ptr = [0]
        self.params = []       # (name, ndarray)
        self.consumers = {}    # entry id -> count
        self.macs = 0          # conv/dense multiply-accumulates per forward pass
        self._n = 0

    # ---- low-level
    def _eid(self, e):
        return self.row_ptr[e[0]] + e[1]

    def _add(self, node, out_shapes, out_precs):
        nid = len(self.nodes)
        self.nodes.append(node)
        for s, p in zip(out_shapes, out_precs):
            self.shapes.append([int(v) for v in s])
            self.precs.append(p)
        self.row_ptr.append(len(self.shapes))
        return [(nid, i) for i in range(len(out_shapes))]

    def _plan_storage(self, heads):
        """One storage id per entry, except that an operator from the reference's
        in-place list writes over its first input when nothing else reads it."""
        readers = dict(self.consumers)
        for e in heads:
            readers[self._eid(e)] = readers.get(self._eid(e), 0) + 1
        sids, nxt = [], 0
        for nid, node in enumerate(self.nodes):
            for i in range(self.row_ptr[nid + 1] - self.row_ptr[nid]):
                sid = None
                if node["op"] != "null" and i == 0 and node["attrs"]["func_name"] in _INPLACE:
                    src = self._eid(tuple(node["inputs"][0][:2]))
                    src_is_var = self.nodes[node["inputs"][0][0]]["op"] == "null"
                    same = int(np.prod(self.shapes[src])) == int(np.prod(self.shapes[self.row_ptr[nid]]))
                    if readers.get(src, 0) == 1 and not src_is_var and same:
                        sid = sids[src]
                if sid is None:
                    sid, nxt = nxt, nxt + 1
                sids.append(sid)
        return sids

    def shape(self, e):
        return tuple(self.shapes[self._eid(e)])

    def var(self, name, shape, precision, values=None):
        node = {"op": "null", "name": name, "inputs": []}
        (e,) = self._add(node, [shape], [precision])
        if values is not None:
            self.params.append((name, values))
        return e

    def param(self, name, shape, lo, hi, precision, dtype=np.int8):
        vals = synth.tensor(self.cid, name, shape, lo, hi).astype(dtype)
        return self.var(name, shape, precision, vals)

    def op(self, func, inputs, attrs, out_shapes, name=None):
        self._n += 1
        name = name or "%s%d" % (func, self._n)
        for e in inputs:
            self.consumers[self._eid(e)] = self.consumers.get(self._eid(e), 0) + 1
        node = {"op": "cvm_op", "name": name, "inputs": [[e[0], e[1], 0] for e in inputs],
                "attrs": {"func_name": func, "num_inputs": str(len(inputs)), "num_outputs": str(len(out_shapes)),
                          "flatten_data": "0"},
                "op_attrs": {k: str(v) for k, v in attrs.items()}}
        return self._add(node, out_shapes, [-1] * len(out_shapes))

    # ---- layers
    def conv(self, x, oc, k, stride=1, pad=0, groups=1, bias=True, dilation=1, name=None):
        n, ic, h, w = self.shape(x)
        self._n += 1
        name = name or "conv%d" % self._n
        icg = ic // groups
        wt = self.param(name + "_weight", (oc, icg, k, k), -127, 127, 8)
        ins = [x, wt]
        if bias:
            ins.append(self.param(name + "_bias", (oc,), -32768, 32768, 17, np.int32))
        oh, ow = conv_out(h, k, stride, pad, dilation), conv_out(w, k, stride, pad, dilation)
        attrs = {"channels": oc, "kernel_size": "[%d, %d]" % (k, k), "strides": "(%d, %d)" % (stride, stride),
                 "padding": "(%d, %d)" % (pad, pad), "dilation": "(%d, %d)" % (dilation, dilation),
                 "groups": groups, "use_bias": "True" if bias else "False"}
        self.macs += n * oc * oh * ow * icg * k * k
        (y,) = self.op("conv2d", ins, attrs, [(n, oc, oh, ow)], name)
        return y, icg * k * k

    def dense(self, x, units, bias=True, name=None):
        m, k = self.shape(x)
        self._n += 1
        name = name or "dense%d" % self._n
        wt = self.param(name + "_weight", (units, k), -127, 127, 8)
        ins = [x, wt]
        if bias:
            ins.append(self.param(name + "_bias", (units,), -32768, 32768, 17, np.int32))
        self.macs += m * units * k
        (y,) = self.op("dense", ins, {"units": units, "use_bias": "True" if bias else "False"}, [(m, units)], name)
        return y, k

    def unary(self, func, x, **attrs):
        (y,) = self.op(func, [x], attrs, [self.shape(x)])
        return y

    def relu(self, x):
        return self.unary("relu", x)

    def rshift(self, x, shift_bit, precision=8):
        return self.unary("cvm_right_shift", x, precision=precision, shift_bit=shift_bit)

    def clip8(self, x):
        return self.unary("cvm_clip", x, precision=8)

    def add(self, a, b):
        (y,) = self.op("elemwise_add", [a, b], {}, [self.shape(a)])
        return y

    def max_pool(self, x, k, stride, pad=0):
        n, c, h, w = self.shape(x)
        oh, ow = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
        (y,) = self.op("max_pool2d", [x], {"pool_size": "[%d, %d]" % (k, k), "strides": "(%d, %d)" % (stride, stride),
                                           "padding": "(%d, %d)" % (pad, pad)}, [(n, c, oh, ow)])
        return y

    def global_sum(self, x):
        n, c, h, w = self.shape(x)
        (y,) = self.op("sum", [x], {"axis": "(2, 3)"}, [(n, c)])
        return y, h * w

    def flatten(self, x):
        s = self.shape(x)
        (y,) = self.op("flatten", [x], {}, [(s[0], int(np.prod(s[1:])))])
        return y

    def reshape(self, x, shape):
        (y,) = self.op("reshape", [x], {"shape": "(%s)" % ", ".join(str(v) for v in shape)}, [shape])
        return y

    def transpose(self, x, axes):
        s = self.shape(x)
        (y,) = self.op("transpose", [x], {"axes": "(%s)" % ", ".join(str(v) for v in axes)}, [[s[a] for a in axes]])
        return y

    def concat(self, xs, axis):
        s = list(self.shape(xs[0]))
        s[axis] = sum(self.shape(v)[axis] for v in xs)
        (y,) = self.op("concatenate", xs, {"axis": axis}, [s])
        return y

    def conv_relu_q(self, x, oc, k, stride=1, pad=0, groups=1, relu=True):
        """conv (+bias) -> [relu] -> cvm_right_shift to 8 bits: the requantised layer MRT emits."""
        y, fan_in = self.conv(x, oc, k, stride, pad, groups)
        if relu:
            y = self.relu(y)
        return self.rshift(y, shift_for(fan_in))

    # ---- output
    def build(self, heads, postprocess=None, version="cvm_1.0.0"):
        g = {
            "nodes": [{k: v for k, v in n.items() if k != "op_attrs"} for n in self.nodes],
            "arg_nodes": [i for i, n in enumerate(self.nodes) if n["op"] == "null"],
            "node_row_ptr": self.row_ptr,
            "heads": [[e[0], e[1], 0] for e in heads],
            "attrs": {
                "storage_id": ["list_int", self._plan_storage(heads)],
                "shape": ["list_shape", self.shapes],
                "dltype": ["list_str", ["int32"] * len(self.shapes)],
                "precision": ["list_int", self.precs],
                "op_attrs": ["list_str", [json.dumps(n.get("op_attrs", {})) for n in self.nodes]],
            },
            "version": version,
        }
        if postprocess:
            g["postprocess"] = postprocess
        return json.dumps(g), save_params(self.params)


# ---------------------------------------------------------------------------- models
def conv_op_graph(n=1, c=64, h=56, w=56, oc=64):
    """BASELINE config 1: conv2d 3x3 s1 p1 + bias -> cvm_right_shift(8) -> cvm_clip(8)."""
    g = GraphBuilder("cfg1-conv")
    x = g.var("data", (n, c, h, w), 8)
    y, _ = g.conv(x, oc, 3, 1, 1, name="conv")
    y = g.clip8(g.rshift(y, 8))
    return g, [y]


def resnet20_cifar(batch=1):
    """BASELINE config 2: 3 stages x 3 basic blocks (16/32/64), global sum, dense 10."""
    g = GraphBuilder("cfg2-resnet20")
    x = g.var("data", (batch, 3, 32, 32), 8)
    x = g.conv_relu_q(x, 16, 3, 1, 1)
    for stage, ch in enumerate((16, 32, 64)):
        for blk in range(3):
            stride = 2 if (stage > 0 and blk == 0) else 1
            y = g.conv_relu_q(x, ch, 3, stride, 1)
            y = g.conv_relu_q(y, ch, 3, 1, 1, relu=False)
            sc = g.conv_relu_q(x, ch, 1, stride, 0, relu=False) if stride == 2 else x
            x = g.rshift(g.relu(g.add(y, sc)), 1)
    s, cnt = g.global_sum(x)
    s = g.rshift(s, max(1, int(round(math.log2(cnt * 30 / 40.0)))))
    y, _ = g.dense(g.flatten(s), 10)
    return g, [y]


def resnet50(batch=1, width=64, blocks=(3, 4, 6, 3), size=224, classes=1000, config_id="cfg3-resnet50"):
    """BASELINE config 3: 7x7/2 stem, 3x3/2 max-pool, bottleneck stages, global sum, dense.
    `width`/`blocks`/`size` shrink the model for quick tests (same structure)."""
    g = GraphBuilder(config_id)
    x = g.var("data", (batch, 3, size, size), 8)
    x = g.conv_relu_q(x, width, 7, 2, 3)
    x = g.max_pool(x, 3, 2, 1)
    for stage, nblk in enumerate(blocks):
        mid = width * (2 ** stage)
        out = mid * 4
        for blk in range(nblk):
            stride = 2 if (stage > 0 and blk == 0) else 1
            y = g.conv_relu_q(x, mid, 1)
            y = g.conv_relu_q(y, mid, 3, stride, 1)
            y = g.conv_relu_q(y, out, 1, relu=False)
            sc = g.conv_relu_q(x, out, 1, stride, 0, relu=False) if blk == 0 else x
            x = g.rshift(g.relu(g.add(y, sc)), 1)
    s, cnt = g.global_sum(x)
    s = g.rshift(s, max(1, int(round(math.log2(cnt * 30 / 40.0)))))
    y, _ = g.dense(g.flatten(s), classes)
    return g, [y]


def vgg16(batch=1, size=224, width=64, fc=4096, classes=1000, config_id="cfg4-vgg16"):
    """BASELINE config 4: thirteen 3x3 convs, five 2x2 max-pools, three dense layers."""
    g = GraphBuilder(config_id)
    x = g.var("data", (batch, 3, size, size), 8)
    for mult, reps in ((1, 2), (2, 2), (4, 3), (8, 3), (8, 3)):
        for _ in range(reps):
            x = g.conv_relu_q(x, width * mult, 3, 1, 1)
        x = g.max_pool(x, 2, 2)
    x = g.flatten(x)
    for _ in range(2):
        y, k = g.dense(x, fc)
        x = g.rshift(g.relu(y), shift_for(k))
    y, _ = g.dense(x, classes)
    return g, [y]


def ssd_mobilenet(size=512, classes=21, alpha=1.0, config_id="cfg5-ssd512", neg_ids=False):
    """BASELINE config 5: MobileNet-1.0 depthwise-separable backbone, multibox heads over
    7 feature maps (24564 anchors at 512x512), get_valid_counts(10), NMS(iou 45, top-k 400)."""
    g = GraphBuilder(config_id)
    x = g.var("data", (1, 3, size, size), 8)

    def ch(c):
        return max(8, int(c * alpha))
    x = g.conv_relu_q(x, ch(32), 3, 2, 1)
    feats = []
    cfg = [(64, 1), (128, 2), (128, 1), (256, 2), (256, 1), (512, 2)] + [(512, 1)] * 5 + [(1024, 2), (1024, 1)]
    for i, (c, s) in enumerate(cfg):
        ic = g.shape(x)[1]
        x = g.conv_relu_q(x, ic, 3, s, 1, groups=ic)      # depthwise
        x = g.conv_relu_q(x, ch(c), 1)                    # pointwise
        if i in (4, 10, 12):
            feats.append(x)
    for c in (512, 256, 256, 128):
        x = g.conv_relu_q(x, ch(c) // 2, 1)
        x = g.conv_relu_q(x, ch(c), 3, 2, 1)
        feats.append(x)
    anchors_per = [4, 6, 6, 6, 6, 4, 4]
    cls_parts, loc_parts = [], []
    for f, a in zip(feats, anchors_per):
        n, c, h, w = g.shape(f)
        cl = g.conv_relu_q(f, a * classes, 3, 1, 1, relu=False)
        lo = g.conv_relu_q(f, a * 4, 3, 1, 1, relu=False)
        cls_parts.append(g.reshape(g.transpose(cl, (0, 2, 3, 1)), (1, h * w * a, classes)))
        loc_parts.append(g.reshape(g.transpose(lo, (0, 2, 3, 1)), (1, h * w * a, 4)))
    cls = g.concat(cls_parts, 1)
    loc = g.concat(loc_parts, 1)
    na = g.shape(cls)[1]
    (score,) = g.op("max", [cls], {"axis": "(2,)", "keepdims": "True"}, [(1, na, 1)])
    # anchor boxes (x1<x2, y1<y2 inside the image) shifted by the predicted offsets
    xy = np.sort(synth.tensor(config_id, "anchors", (1, na, 2, 2), 0, size), axis=2).reshape(1, na, 4)
    anchors = g.var("anchors", (1, na, 4), 11, xy.astype(np.int32))
    (boxes,) = g.op("broadcast_add", [anchors, g.rshift(loc, 3, 6)], {}, [(1, na, 4)])
    ids = g.var("anchor_ids", (1, na, 1), 6,
                synth.tensor(config_id, "anchor_ids", (1, na, 1), -1 if neg_ids else 0, classes - 1))
    rows = g.concat([ids, score, boxes], 2)
    vc, compact = g.op("get_valid_counts", [rows], {"score_threshold": 10}, [(1,), (1, na, 6)])
    (det,) = g.op("non_max_suppression", [compact, vc], {"iou_threshold": 45, "top_k": 400}, [(1, na, 6)])
    return g, [det]
