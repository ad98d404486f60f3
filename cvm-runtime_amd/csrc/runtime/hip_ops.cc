// cvm.runtime.hip.<op>: one registry entry per operator, each unpacking the
// node's tensors and attributes and calling the operator-level C ABI
// (include/cvm_hip_ops.h).  This is the counterpart of the reference's
// src/runtime/cuda/ops/ops_cuda.cc for the HIP device.
#include <memory>
#include <mutex>

#include "../../../include/cvm_hip_ops.h"
#include "graph_runtime.h"

namespace cvmrt {
namespace {

void Check(int rc, const char* what) {
  if (rc == CVMHIP_OK) return;
  if (rc < CVMHIP_ERR_RUNTIME) CVM_VERIFY(false) << what << ": " << cvmhip_last_error();
  CVM_CHECK(false) << what << ": " << cvmhip_last_error();
}

struct DeviceBuffer {
  void* ptr = nullptr;
  ~DeviceBuffer() { if (ptr) cvmhip_free(ptr); }
};

struct ConvDims {
  int n, ic, h, w, oc, kh, kw, sh, sw, ph, pw, dh, dw, groups;
};

ConvDims GetConvDims(const OpCall& c) {
  const OpAttrs& a = *c.attrs;
  const Shape &x = c.in[0].shape, &w = c.in[1].shape;
  ConvDims d;
  d.n = (int)x[0]; d.ic = (int)x[1]; d.h = (int)x[2]; d.w = (int)x[3];
  d.oc = (int)w[0]; d.kh = (int)w[2]; d.kw = (int)w[3];
  d.sh = (int)a.t("strides")[0]; d.sw = (int)a.t("strides")[1];
  d.ph = (int)a.t("padding")[0]; d.pw = (int)a.t("padding")[1];
  d.dh = (int)a.t("dilation")[0]; d.dw = (int)a.t("dilation")[1];
  d.groups = (int)a.i("groups");
  CVM_VERIFY(w.size() == 4 && w[0] == a.i("channels") && w[1] == x[1] / d.groups && w[2] == a.t("kernel_size")[0] &&
             w[3] == a.t("kernel_size")[1])
      << "conv2d " << a.node_name << ": filter shape " << shape_str(w) << " does not match the data and attributes";
  return d;
}

// conv2d: [x, w, (b), y].  A constant filter is packed once in prepare().
OpKernel ConvKernel() {
  OpKernel k;
  k.workspace_bytes = [](const OpCall& c) {
    const ConvDims d = GetConvDims(c);
    return cvmhip_conv2d_workspace_bytes(d.n, d.ic, d.h, d.w, d.oc, d.kh, d.kw, d.groups);
  };
  k.prepare = [](OpCall& c) {
    const ConvDims d = GetConvDims(c);
    if (d.groups != 1 || !c.in[1].is_param) return;
    auto buf = std::make_shared<DeviceBuffer>();
    Check(cvmhip_alloc(&buf->ptr, cvmhip_packed_weight_bytes(d.oc, d.ic, d.kh, d.kw)), "conv2d filter buffer");
    Check(cvmhip_pack_weights(c.in[1].data, buf->ptr, d.oc, d.ic, d.kh, d.kw, c.stream), "conv2d filter pack");
    c.state = buf;
  };
  k.run = [](OpCall& c) {
    const ConvDims d = GetConvDims(c);
    const int32_t* bias = c.in.size() == 3 ? c.in[2].data : nullptr;
    if (c.state) {
      Check(cvmhip_conv2d_packed(c.in[0].data, static_cast<DeviceBuffer*>(c.state.get())->ptr, bias, c.out[0].data,
                                 d.n, d.ic, d.h, d.w, d.oc, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.dh, d.dw,
                                 c.workspace, c.workspace_bytes, c.stream), "conv2d");
    } else {
      Check(cvmhip_conv2d(c.in[0].data, c.in[1].data, bias, c.out[0].data, d.n, d.ic, d.h, d.w, d.oc, d.kh, d.kw,
                          d.sh, d.sw, d.ph, d.pw, d.dh, d.dw, d.groups, c.workspace, c.workspace_bytes, c.stream), "conv2d");
    }
  };
  return k;
}

// dense: [x, w, (b), y].  The reference multiplies the int32 values as they are (ops.cc:53-62; only conv2d
// narrows), and a declared precision of 8 bits does not bound a tensor: cvm_right_shift with p + b >= 32
// does not clip (elemwise.cc:133-137) and can emit 128.  A node that runs on its own therefore always
// takes the exact int32 kernel; the int8 matrix-core form is chosen by the fused planner, and only for
// operands whose value range it has proven.
OpKernel DenseKernel() {
  OpKernel k;
  k.run = [](OpCall& c) {
    const int m = (int)c.in[0].shape[0], kk = (int)c.in[0].shape[1], n = (int)c.in[1].shape[0];
    const int32_t* bias = c.in.size() == 3 ? c.in[2].data : nullptr;
    Check(cvmhip_dense(c.in[0].data, c.in[1].data, bias, c.out[0].data, m, kk, n, 32, nullptr, 0, c.stream), "dense");
  };
  return k;
}

template <typename F>
OpKernel Simple(F f) {
  OpKernel k;
  k.run = f;
  return k;
}

const int64_t* Dims(const Shape& s) { return s.data(); }

void RegisterAll() {
  OpRegistry& r = OpRegistry::Global();
  auto reg = [&](const char* op, OpKernel k) { r.Register(std::string("cvm.runtime.hip.") + op, std::move(k)); };

  reg("conv2d", ConvKernel());
  reg("dense", DenseKernel());
  reg("relu", Simple([](OpCall& c) { Check(cvmhip_relu(c.in[0].data, c.out[0].data, c.in[0].size(), c.stream), "relu"); }));
  reg("abs", Simple([](OpCall& c) { Check(cvmhip_abs(c.in[0].data, c.out[0].data, c.in[0].size(), c.stream), "abs"); }));
  reg("negative", Simple([](OpCall& c) { Check(cvmhip_negative(c.in[0].data, c.out[0].data, c.in[0].size(), c.stream), "negative"); }));
  reg("cvm_precision", Simple([](OpCall& c) {
        Check(cvmhip_cvm_precision(c.in[0].data, c.out[0].data, c.in[0].size(), c.stream), "cvm_precision");
      }));
  reg("clip", Simple([](OpCall& c) {
        Check(cvmhip_clip(c.in[0].data, c.out[0].data, c.in[0].size(), (int32_t)c.attrs->i("a_min"),
                          (int32_t)c.attrs->i("a_max"), c.stream), "clip");
      }));
  reg("cvm_clip", Simple([](OpCall& c) {
        Check(cvmhip_cvm_clip(c.in[0].data, c.out[0].data, c.in[0].size(), (int)c.attrs->i("precision"), c.stream), "cvm_clip");
      }));
  reg("cvm_right_shift", Simple([](OpCall& c) {
        Check(cvmhip_cvm_right_shift(c.in[0].data, c.out[0].data, c.in[0].size(), (int)c.attrs->i("precision"),
                                     (int)c.attrs->i("shift_bit"), c.stream), "cvm_right_shift");
      }));
  reg("cvm_left_shift", Simple([](OpCall& c) {
        Check(cvmhip_cvm_left_shift(c.in[0].data, c.out[0].data, c.in[0].size(), (int)c.attrs->i("precision"),
                                    (int)c.attrs->i("shift_bit"), c.stream), "cvm_left_shift");
      }));
  reg("elemwise_add", Simple([](OpCall& c) {
        Check(cvmhip_elemwise(CVMHIP_ADD, c.in[0].data, c.in[1].data, c.out[0].data, c.in[0].size(), c.stream), "elemwise_add");
      }));
  reg("elemwise_sub", Simple([](OpCall& c) {
        Check(cvmhip_elemwise(CVMHIP_SUB, c.in[0].data, c.in[1].data, c.out[0].data, c.in[0].size(), c.stream), "elemwise_sub");
      }));
  static const struct { const char* name; int op; } kBroadcast[] = {
      {"broadcast_add", CVMHIP_ADD}, {"broadcast_sub", CVMHIP_SUB}, {"broadcast_mul", CVMHIP_MUL},
      {"broadcast_max", CVMHIP_MAX}, {"broadcast_div", CVMHIP_DIV}, {"broadcast_greater", CVMHIP_GREATER}};
  for (const auto& b : kBroadcast) {
    const int op = b.op;
    reg(b.name, Simple([op](OpCall& c) {
          Check(cvmhip_broadcast(op, c.in[0].data, Dims(c.in[0].shape), (int)c.in[0].shape.size(), c.in[1].data,
                                 Dims(c.in[1].shape), (int)c.in[1].shape.size(), c.out[0].data, Dims(c.out[0].shape),
                                 (int)c.out[0].shape.size(), c.stream), "broadcast");
        }));
  }
  reg("max_pool2d", Simple([](OpCall& c) {
        const OpAttrs& a = *c.attrs;
        const Shape &x = c.in[0].shape, &y = c.out[0].shape, &pad = a.t("padding");
        const int ph = (int)pad[0], pw = pad.size() == 2 ? (int)pad[1] : (int)pad[0];
        Check(cvmhip_max_pool2d(c.in[0].data, c.out[0].data, (int)x[0], (int)x[1], (int)x[2], (int)x[3], (int)y[2],
                                (int)y[3], (int)a.t("pool_size")[0], (int)a.t("pool_size")[1], (int)a.t("strides")[0],
                                (int)a.t("strides")[1], ph, pw, c.stream), "max_pool2d");
      }));
  for (const char* name : {"sum", "max"}) {
    const int op = std::string(name) == "sum" ? CVMHIP_SUM : CVMHIP_RMAX;
    reg(name, Simple([op](OpCall& c) {
          const Shape& ax = c.attrs->t("axis");
          Check(cvmhip_reduce(op, c.in[0].data, Dims(c.in[0].shape), (int)c.in[0].shape.size(), c.out[0].data,
                              c.out[0].size(), ax.empty() ? nullptr : ax.data(), (int)ax.size(),
                              c.attrs->b("exclude") ? 1 : 0, c.stream), "reduce");
        }));
  }
  for (const char* name : {"flatten", "reshape", "expand_dims", "squeeze"}) {
    reg(name, Simple([](OpCall& c) { Check(cvmhip_copy(c.in[0].data, c.out[0].data, c.in[0].size(), c.stream), "copy"); }));
  }
  reg("concatenate", Simple([](OpCall& c) {
        std::vector<const int32_t*> ptrs;
        std::vector<const int64_t*> shapes;
        for (const DevTensor& t : c.in) { ptrs.push_back(t.data); shapes.push_back(t.shape.data()); }
        Check(cvmhip_concatenate(ptrs.data(), shapes.data(), (int)c.in.size(), (int)c.in[0].shape.size(),
                                 (int)c.attrs->i("axis"), c.out[0].data, Dims(c.out[0].shape), c.stream), "concatenate");
      }));
  reg("transpose", Simple([](OpCall& c) {
        const Shape& ax = c.attrs->t("axes");
        Check(cvmhip_transpose(c.in[0].data, Dims(c.in[0].shape), (int)c.in[0].shape.size(), ax.empty() ? nullptr : ax.data(),
                               (int)ax.size(), c.out[0].data, c.stream), "transpose");
      }));
  reg("strided_slice", Simple([](OpCall& c) {
        const Shape &b = c.attrs->t("begin"), &s = c.attrs->t("stride");
        Check(cvmhip_strided_slice(c.in[0].data, Dims(c.in[0].shape), (int)c.in[0].shape.size(), b.empty() ? nullptr : b.data(),
                                   (int)b.size(), s.empty() ? nullptr : s.data(), (int)s.size(), c.out[0].data,
                                   Dims(c.out[0].shape), c.stream), "strided_slice");
      }));
  reg("slice_like", Simple([](OpCall& c) {
        Check(cvmhip_slice_like(c.in[0].data, Dims(c.in[0].shape), (int)c.in[0].shape.size(), c.out[0].data,
                                Dims(c.out[0].shape), c.stream), "slice_like");
      }));
  reg("take", Simple([](OpCall& c) {
        Check(cvmhip_take(c.in[0].data, Dims(c.in[0].shape), (int)c.in[0].shape.size(), c.in[1].data, Dims(c.in[1].shape),
                          (int)c.in[1].shape.size(), c.out[0].data, Dims(c.out[0].shape), (int)c.out[0].shape.size(),
                          c.attrs->has("axis") ? 1 : 0, (int)c.attrs->i("axis"), c.stream), "take");
      }));
  // cvm_lut(indices, table) = take(table, indices) on the flattened table (ops.cc:949-956)
  reg("cvm_lut", Simple([](OpCall& c) {
        Check(cvmhip_take(c.in[1].data, Dims(c.in[1].shape), (int)c.in[1].shape.size(), c.in[0].data, Dims(c.in[0].shape),
                          (int)c.in[0].shape.size(), c.out[0].data, Dims(c.out[0].shape), (int)c.out[0].shape.size(), 0, 0,
                          c.stream), "cvm_lut");
      }));
  reg("repeat", Simple([](OpCall& c) {
        Check(cvmhip_repeat(c.in[0].data, Dims(c.in[0].shape), c.out[0].data, Dims(c.out[0].shape), (int)c.in[0].shape.size(),
                            (int)c.attrs->i("axis"), (int)c.attrs->i("repeats"), c.stream), "repeat");
      }));
  reg("tile", Simple([](OpCall& c) {
        Check(cvmhip_tile(c.in[0].data, Dims(c.in[0].shape), (int)c.in[0].shape.size(), c.out[0].data, Dims(c.out[0].shape),
                          (int)c.out[0].shape.size(), c.stream), "tile");
      }));
  reg("upsampling", Simple([](OpCall& c) {
        const Shape& x = c.in[0].shape;
        Check(cvmhip_upsampling(c.in[0].data, c.out[0].data, (int)x[0], (int)x[1], (int)x[2], (int)x[3],
                                (int)c.attrs->i("scale"), c.stream), "upsampling");
      }));
  reg("where", Simple([](OpCall& c) {
        Check(cvmhip_where(c.in[0].data, c.in[1].data, c.in[2].data, c.out[0].data, Dims(c.out[0].shape),
                           (int)c.out[0].shape.size(), c.in[0].shape.size() == c.in[1].shape.size() ? 1 : 0, c.stream), "where");
      }));
  {
    OpKernel k;
    k.workspace_bytes = [](const OpCall& c) {
      return cvmhip_get_valid_counts_workspace_bytes((int)c.in[0].shape[0], (int)c.in[0].shape[1]);
    };
    k.run = [](OpCall& c) {
      const Shape& x = c.in[0].shape;
      Check(cvmhip_get_valid_counts(c.in[0].data, c.out[0].data, c.out[1].data, (int)x[0], (int)x[1], (int)x[2],
                                    (int32_t)c.attrs->i("score_threshold"), c.workspace, c.workspace_bytes, c.stream),
            "get_valid_counts");
    };
    reg("get_valid_counts", k);
  }
  {
    OpKernel k;
    k.workspace_bytes = [](const OpCall& c) {
      return cvmhip_nms_workspace_bytes((int)c.in[0].shape[0], (int)c.in[0].shape[1], (int)c.in[0].shape[2]);
    };
    k.run = [](OpCall& c) {
      const Shape& x = c.in[0].shape;
      const OpAttrs& a = *c.attrs;
      Check(cvmhip_non_max_suppression(c.in[0].data, c.in[1].data, c.out[0].data, (int)x[0], (int)x[1], (int)x[2],
                                       (int)a.i("max_output_size"), (int)a.i("iou_threshold"), (int)a.i("top_k"),
                                       (int)a.i("coord_start"), (int)a.i("score_index"), (int)a.i("id_index"),
                                       a.b("force_suppress") ? 1 : 0, c.workspace, c.workspace_bytes, c.stream),
            "non_max_suppression");
    };
    reg("non_max_suppression", k);
  }
}

}  // namespace

void RegisterHipKernels() {
  static std::once_flag once;
  std::call_once(once, RegisterAll);
}

}  // namespace cvmrt
