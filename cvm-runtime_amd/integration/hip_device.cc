// HIP as a device of the reference runtime: the file a maintainer of cvm-runtime adds to its tree (e.g. as
// src/runtime/hip/hip_device.cc, linked with libcvm_runtime_hip.so) to run its own graph runtime on MI355X.
// It registers one packed function per operator under "cvm.runtime.hip.<op>" -- the 37 names the graph
// runtime looks up (src/runtime/graph_runtime.cc:660-664, include/cvm/runtime/registry.h:129-131) -- and the
// device API "device_api.hip" (include/cvm/runtime/device_api.h:43-108).  Every wrapper does what the
// "cvm.runtime.cpu.<op>" body it stands in for does with its arguments (inputs, then outputs, then the
// node's attributes; src/runtime/cpu/ops/*.cc) and hands plain pointers and sizes to include/cvm_hip_ops.h.
//
// This file compiles only against the reference's headers:
//   g++ -std=c++11 -fsyntax-only -I<cvm-runtime>/include -I<this repository>/include hip_device.cc
// All tensors are int32 on the device; scratch comes from args.ext_space (the FOpExtraSpace of the operator
// must return cvmhip_*_workspace_bytes()/4 int32 elements for this device).
#include <cvm/dlpack.h>
#include <cvm/node.h>
#include <cvm/op.h>
#include <cvm/runtime/device_api.h>
#include <cvm/runtime/packed_func.h>
#include <cvm/runtime/registry.h>
#include <cvm/top/nn.h>
#include <cvm/top/tensor.h>

#include <string>
#include <vector>

#include "cvm_hip_ops.h"

namespace cvm {
namespace runtime {
namespace {

// CVMHIP_ERR_ARG is what the reference reports with VERIFY (ERROR_LOGIC), anything else non-zero with CHECK
// (ERROR_RUNTIME); include/cvm/errors.h:15-36
inline void HipCall(int rc) {
  if (rc == CVMHIP_ERR_ARG) VERIFY(false) << cvmhip_last_error();
  CHECK(rc == CVMHIP_OK) << cvmhip_last_error();
}

inline int32_t* I32(DLTensor* t) { return static_cast<int32_t*>(t->data); }
inline int64_t Count(const DLTensor* t) {
  int64_t n = 1;
  for (int i = 0; i < t->ndim; ++i) n *= t->shape[i];
  return n;
}
template <typename P>
inline const P& Param(CVMArgs& args) {
  void* attr = args[args.num_args - 1];
  return cvm::get<P>(static_cast<cvm::NodeAttrs*>(attr)->parsed);
}
inline void* Scratch(CVMArgs& args) { return args.ext_space ? args.ext_space->data : nullptr; }
inline size_t ScratchBytes(CVMArgs& args) {
  return args.ext_space && args.ext_space->ndim > 0 ? static_cast<size_t>(args.ext_space->shape[0]) * 4 : 0;
}
// a tuple attribute as the int64 array the C ABI takes
template <typename T>
inline std::vector<int64_t> Dims(const T& t) {
  std::vector<int64_t> v;
  for (auto it = t.begin(); it != t.end(); ++it) v.push_back(static_cast<int64_t>(*it));
  return v;
}
inline const int64_t* PtrOrNull(const std::vector<int64_t>& v) { return v.empty() ? nullptr : v.data(); }

// unary operators without attributes: (x, y, attrs)
template <int (*F)(const int32_t*, int32_t*, int64_t, void*)>
void Unary(CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  HipCall(F(I32(x), I32(y), Count(x), nullptr));
}
// flatten / reshape / expand_dims / squeeze: a copy unless in place (ops.cc:567 ff.)
void CopyOp(CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  if (x->data == y->data) return;
  HipCall(cvmhip_copy(I32(x), I32(y), Count(x), nullptr));
}
template <int OP>
void Elemwise(CVMArgs args, CVMRetValue*) {   // elemwise.cc:8-45
  DLTensor* a = args[0];
  DLTensor* b = args[1];
  DLTensor* c = args[2];
  HipCall(cvmhip_elemwise(OP, I32(a), I32(b), I32(c), Count(a), nullptr));
}
template <int OP>
void Broadcast(CVMArgs args, CVMRetValue*) {   // broadcast.cc:6-125
  DLTensor* a = args[0];
  DLTensor* b = args[1];
  DLTensor* c = args[2];
  HipCall(cvmhip_broadcast(OP, I32(a), a->shape, a->ndim, I32(b), b->shape, b->ndim, I32(c), c->shape, c->ndim, nullptr));
}
template <int OP>
void Reduce(CVMArgs args, CVMRetValue*) {   // reduce.cc:6-140
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  const auto& p = Param<cvm::top::ReduceParam>(args);
  const std::vector<int64_t> axis = Dims(p.axis);
  HipCall(cvmhip_reduce(OP, I32(x), x->shape, x->ndim, I32(y), Count(y), PtrOrNull(axis), static_cast<int>(axis.size()),
                        p.exclude ? 1 : 0, nullptr));
}

}  // namespace

// ---- convolution and dense (ops.cc:368-456, ops.cc:34-75)
CVM_REGISTER_GLOBAL("cvm.runtime.hip.conv2d").set_body([](CVMArgs args, CVMRetValue*) {
  const bool has_bias = args.num_args == 5;
  DLTensor* x = args[0];
  DLTensor* w = args[1];
  DLTensor* b = has_bias ? static_cast<DLTensor*>(args[2]) : nullptr;
  DLTensor* y = has_bias ? args[3] : args[2];
  const auto& p = Param<cvm::top::Conv2DParam>(args);
  HipCall(cvmhip_conv2d(I32(x), I32(w), b ? I32(b) : nullptr, I32(y), static_cast<int>(x->shape[0]),
                        static_cast<int>(x->shape[1]), static_cast<int>(x->shape[2]), static_cast<int>(x->shape[3]),
                        static_cast<int>(w->shape[0]), static_cast<int>(w->shape[2]), static_cast<int>(w->shape[3]),
                        static_cast<int>(p.strides[0]), static_cast<int>(p.strides[1]), static_cast<int>(p.padding[0]),
                        static_cast<int>(p.padding[1]), static_cast<int>(p.dilation[0]), static_cast<int>(p.dilation[1]),
                        p.groups, Scratch(args), ScratchBytes(args), nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.dense").set_body([](CVMArgs args, CVMRetValue*) {
  const bool has_bias = args.num_args == 5;
  DLTensor* x = args[0];
  DLTensor* w = args[1];
  DLTensor* b = has_bias ? static_cast<DLTensor*>(args[2]) : nullptr;
  DLTensor* y = has_bias ? args[3] : args[2];
  // operand_bits 32: exact for any operands.  A caller that has verified the graph (DenseInferPrecision,
  // src/top/nn/nn.cc:22-44, bounds both operands by 8 bits) may pass 8 to reach the matrix cores.
  HipCall(cvmhip_dense(I32(x), I32(w), b ? I32(b) : nullptr, I32(y), static_cast<int>(x->shape[0]),
                       static_cast<int>(x->shape[1]), static_cast<int>(w->shape[0]), 32, Scratch(args), ScratchBytes(args),
                       nullptr));
});

// ---- unary elementwise (ops.cc:12-26,525-553,632-642, elemwise.cc:47-193)
CVM_REGISTER_GLOBAL("cvm.runtime.hip.relu").set_body(Unary<cvmhip_relu>);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.abs").set_body(Unary<cvmhip_abs>);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.negative").set_body(Unary<cvmhip_negative>);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.cvm_precision").set_body(Unary<cvmhip_cvm_precision>);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.clip").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  const auto& p = Param<cvm::top::ClipParam>(args);
  HipCall(cvmhip_clip(I32(x), I32(y), Count(x), p.a_min, p.a_max, nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.cvm_clip").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  const auto& p = Param<cvm::top::CVMClipParam>(args);
  HipCall(cvmhip_cvm_clip(I32(x), I32(y), Count(x), p.precision, nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.cvm_right_shift").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  const auto& p = Param<cvm::top::CVMRightShiftParam>(args);
  HipCall(cvmhip_cvm_right_shift(I32(x), I32(y), Count(x), p.precision, p.shift_bit, nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.cvm_left_shift").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  const auto& p = Param<cvm::top::CVMLeftShiftParam>(args);
  HipCall(cvmhip_cvm_left_shift(I32(x), I32(y), Count(x), p.precision, p.shift_bit, nullptr));
});

// ---- binary and broadcasting
CVM_REGISTER_GLOBAL("cvm.runtime.hip.elemwise_add").set_body(Elemwise<CVMHIP_ADD>);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.elemwise_sub").set_body(Elemwise<CVMHIP_SUB>);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.broadcast_add").set_body(Broadcast<CVMHIP_ADD>);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.broadcast_sub").set_body(Broadcast<CVMHIP_SUB>);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.broadcast_mul").set_body(Broadcast<CVMHIP_MUL>);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.broadcast_max").set_body(Broadcast<CVMHIP_MAX>);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.broadcast_div").set_body(Broadcast<CVMHIP_DIV>);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.broadcast_greater").set_body(Broadcast<CVMHIP_GREATER>);

// ---- pooling and reductions (ops.cc:466-523, reduce.cc)
CVM_REGISTER_GLOBAL("cvm.runtime.hip.max_pool2d").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  const auto& p = Param<cvm::top::MaxPool2DParam>(args);
  const int pad_h = static_cast<int>(p.padding[0]);
  const int pad_w = p.padding.ndim() == 2 ? static_cast<int>(p.padding[1]) : pad_h;   // ops.cc:478-481
  HipCall(cvmhip_max_pool2d(I32(x), I32(y), static_cast<int>(x->shape[0]), static_cast<int>(x->shape[1]),
                            static_cast<int>(x->shape[2]), static_cast<int>(x->shape[3]), static_cast<int>(y->shape[2]),
                            static_cast<int>(y->shape[3]), static_cast<int>(p.pool_size[0]), static_cast<int>(p.pool_size[1]),
                            static_cast<int>(p.strides[0]), static_cast<int>(p.strides[1]), pad_h, pad_w, nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.sum").set_body(Reduce<CVMHIP_SUM>);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.max").set_body(Reduce<CVMHIP_RMAX>);

// ---- shape-only operators
CVM_REGISTER_GLOBAL("cvm.runtime.hip.flatten").set_body(CopyOp);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.reshape").set_body(CopyOp);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.expand_dims").set_body(CopyOp);
CVM_REGISTER_GLOBAL("cvm.runtime.hip.squeeze").set_body(CopyOp);

// ---- index-remap copies (ops.cc:567-989,1049-1075)
CVM_REGISTER_GLOBAL("cvm.runtime.hip.concatenate").set_body([](CVMArgs args, CVMRetValue*) {
  const int ninputs = args.num_args - 2;   // inputs, then the output, then the attributes
  DLTensor* y = args[ninputs];
  const auto& p = Param<cvm::top::ConcatenateParam>(args);
  std::vector<const int32_t*> ptrs;
  std::vector<const int64_t*> shapes;
  for (int i = 0; i < ninputs; ++i) {
    DLTensor* t = args[i];
    ptrs.push_back(I32(t));
    shapes.push_back(t->shape);
  }
  int axis = p.axis;
  if (axis < 0) axis += y->ndim;
  HipCall(cvmhip_concatenate(ptrs.data(), shapes.data(), ninputs, y->ndim, axis, I32(y), y->shape, nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.transpose").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  const std::vector<int64_t> axes = Dims(Param<cvm::top::TransposeParam>(args).axes);
  HipCall(cvmhip_transpose(I32(x), x->shape, x->ndim, PtrOrNull(axes), static_cast<int>(axes.size()), I32(y), nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.strided_slice").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  const auto& p = Param<cvm::top::StridedSliceParam>(args);
  const std::vector<int64_t> begin = Dims(p.begin), stride = Dims(p.stride);
  HipCall(cvmhip_strided_slice(I32(x), x->shape, x->ndim, PtrOrNull(begin), static_cast<int>(begin.size()),
                               PtrOrNull(stride), static_cast<int>(stride.size()), I32(y), y->shape, nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.slice_like").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];   // args[1] only lends its shape, which the output already has
  DLTensor* y = args[2];
  HipCall(cvmhip_slice_like(I32(x), x->shape, x->ndim, I32(y), y->shape, nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.take").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* idx = args[1];
  DLTensor* y = args[2];
  const auto& p = Param<cvm::top::TakeParam>(args);
  const bool has_axis = p.axis.has_value();
  HipCall(cvmhip_take(I32(x), x->shape, x->ndim, I32(idx), idx->shape, idx->ndim, I32(y), y->shape, y->ndim,
                      has_axis ? 1 : 0, has_axis ? p.axis.value() : 0, nullptr));
});
// cvm_lut(indices, table) = take(table, indices) on the flattened table (ops.cc:949-956)
CVM_REGISTER_GLOBAL("cvm.runtime.hip.cvm_lut").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* idx = args[0];
  DLTensor* table = args[1];
  DLTensor* y = args[2];
  HipCall(cvmhip_take(I32(table), table->shape, table->ndim, I32(idx), idx->shape, idx->ndim, I32(y), y->shape, y->ndim, 0, 0,
                      nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.repeat").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  const auto& p = Param<cvm::top::RepeatParam>(args);
  HipCall(cvmhip_repeat(I32(x), x->shape, I32(y), y->shape, x->ndim, p.axis, p.repeats, nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.tile").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  HipCall(cvmhip_tile(I32(x), x->shape, x->ndim, I32(y), y->shape, y->ndim, nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.upsampling").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* y = args[1];
  const auto& p = Param<cvm::top::UpSamplingParam>(args);
  HipCall(cvmhip_upsampling(I32(x), I32(y), static_cast<int>(x->shape[0]), static_cast<int>(x->shape[1]),
                            static_cast<int>(x->shape[2]), static_cast<int>(x->shape[3]), p.scale, nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.where").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* cond = args[0];
  DLTensor* x = args[1];
  DLTensor* y = args[2];
  DLTensor* out = args[3];
  HipCall(cvmhip_where(I32(cond), I32(x), I32(y), I32(out), out->shape, out->ndim, cond->ndim == x->ndim ? 1 : 0, nullptr));
});

// ---- detection post-processing (nms.cc:42-140)
CVM_REGISTER_GLOBAL("cvm.runtime.hip.get_valid_counts").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* valid_count = args[1];
  DLTensor* y = args[2];
  const auto& p = Param<cvm::top::GetValidCountsParam>(args);
  HipCall(cvmhip_get_valid_counts(I32(x), I32(valid_count), I32(y), static_cast<int>(x->shape[0]),
                                  static_cast<int>(x->shape[1]), static_cast<int>(x->shape[2]), p.score_threshold,
                                  Scratch(args), ScratchBytes(args), nullptr));
});
CVM_REGISTER_GLOBAL("cvm.runtime.hip.non_max_suppression").set_body([](CVMArgs args, CVMRetValue*) {
  DLTensor* x = args[0];
  DLTensor* valid_count = args[1];
  DLTensor* y = args[2];
  const auto& p = Param<cvm::top::NonMaximumSuppressionParam>(args);
  HipCall(cvmhip_non_max_suppression(I32(x), I32(valid_count), I32(y), static_cast<int>(x->shape[0]),
                                     static_cast<int>(x->shape[1]), static_cast<int>(x->shape[2]), p.max_output_size,
                                     p.iou_threshold, p.top_k, p.coord_start, p.score_index, p.id_index,
                                     p.force_suppress ? 1 : 0, Scratch(args), ScratchBytes(args), nullptr));
});

// ---- scratch memory.  The reference sizes an operator's ext_space with the operator's FOpExtraSpace attribute
// (include/cvm/op_attr_types.h; called with the node's attributes, input shapes, precisions and the context in
// src/runtime/graph_runtime.cc), in int32 elements.  For this device the sizes are this library's: the bodies of
// FOpExtraSpace for conv2d, dense, get_valid_counts and non_max_suppression (src/top/nn/*.cc) return
// HIPOpExtraSpace(attrs, shapes) when ctx.device_type is the HIP device.  Operators it does not name need none.
int64_t HIPOpExtraSpace(const cvm::NodeAttrs& attrs, const std::vector<TShape>& in_shapes) {
  const std::string& op = attrs.op->name;
  size_t bytes = 0;
  if (op == "conv2d" && in_shapes.size() >= 2 && in_shapes[0].ndim() == 4 && in_shapes[1].ndim() == 4) {
    const auto& p = cvm::get<cvm::top::Conv2DParam>(attrs.parsed);
    const TShape &x = in_shapes[0], &w = in_shapes[1];
    bytes = cvmhip_conv2d_workspace_bytes(static_cast<int>(x[0]), static_cast<int>(x[1]), static_cast<int>(x[2]),
                                          static_cast<int>(x[3]), static_cast<int>(w[0]), static_cast<int>(w[2]),
                                          static_cast<int>(w[3]), p.groups);
  } else if (op == "dense" && in_shapes.size() >= 2 && in_shapes[0].ndim() == 2 && in_shapes[1].ndim() == 2) {
    bytes = cvmhip_dense_workspace_bytes(static_cast<int>(in_shapes[0][0]), static_cast<int>(in_shapes[0][1]),
                                         static_cast<int>(in_shapes[1][0]));
  } else if (op == "get_valid_counts" && in_shapes.size() >= 1 && in_shapes[0].ndim() == 3) {
    bytes = cvmhip_get_valid_counts_workspace_bytes(static_cast<int>(in_shapes[0][0]), static_cast<int>(in_shapes[0][1]));
  } else if (op == "non_max_suppression" && in_shapes.size() >= 1 && in_shapes[0].ndim() == 3) {
    bytes = cvmhip_nms_workspace_bytes(static_cast<int>(in_shapes[0][0]), static_cast<int>(in_shapes[0][1]),
                                       static_cast<int>(in_shapes[0][2]));
  }
  return static_cast<int64_t>((bytes + 3) / 4);
}

// ---- the device: memory and copies (cpu_device_api.cc:18-78 is the CPU counterpart).  The new device type takes
// the next free value of DLDeviceType (include/cvm/dlpack.h:18-25).
constexpr int kDLHIP = 5;

class HIPDeviceAPI final : public DeviceAPI {
 public:
  void SetDevice(CVMContext ctx) final { HipCall(cvmhip_set_device(ctx.device_id)); }
  void GetAttr(CVMContext ctx, DeviceAttrKind kind, CVMRetValue* rv) final {
    if (kind == kExist) {
      int count = 0;
      *rv = (cvmhip_device_count(&count) == CVMHIP_OK && ctx.device_id < count) ? 1 : 0;
    } else if (kind == kWarpSize) {
      *rv = 64;
    } else if (kind == kMultiProcessorCount) {
      *rv = 256;
    }
  }
  void* AllocDataSpace(CVMContext ctx, size_t nbytes, size_t, CVMType) final {
    HipCall(cvmhip_set_device(ctx.device_id));
    void* p = nullptr;
    HipCall(cvmhip_alloc(&p, nbytes));   // hipMalloc: 256-byte aligned, above kAllocAlignment
    return p;
  }
  void FreeDataSpace(CVMContext ctx, void* ptr) final {
    HipCall(cvmhip_set_device(ctx.device_id));
    HipCall(cvmhip_free(ptr));
  }
  void CopyDataFromTo(const void* from, size_t from_offset, void* to, size_t to_offset, size_t num_bytes, CVMContext ctx_from,
                      CVMContext ctx_to, CVMType, CVMStreamHandle stream) final {
    const char* src = static_cast<const char*>(from) + from_offset;
    char* dst = static_cast<char*>(to) + to_offset;
    if (ctx_from.device_type == kDLCPU) {
      HipCall(cvmhip_set_device(ctx_to.device_id));
      HipCall(cvmhip_copy_h2d(dst, src, num_bytes, stream));
    } else if (ctx_to.device_type == kDLCPU) {
      HipCall(cvmhip_set_device(ctx_from.device_id));
      HipCall(cvmhip_copy_d2h(dst, src, num_bytes, stream));
    } else {
      HipCall(cvmhip_set_device(ctx_from.device_id));
      HipCall(cvmhip_copy_d2d(dst, src, num_bytes, stream));
    }
    HipCall(cvmhip_stream_sync(stream));   // the runtime reads the destination right after the call
  }
};

CVM_REGISTER_GLOBAL("device_api.hip").set_body([](CVMArgs, CVMRetValue* rv) {
  static HIPDeviceAPI inst;
  *rv = static_cast<void*>(&inst);
});

}  // namespace runtime
}  // namespace cvm
