// Test infrastructure only (never linked into the product library).
//
// Executes the operator plug-in a maintainer of the reference would add (cvm-runtime_amd/integration/hip_device.cc,
// compiled into this same shared object) the way the reference's own graph runtime would: it looks the packed
// function up in the reference's registry under "cvm.runtime.hip.<op>" (include/cvm/runtime/registry.h:129-131,
// src/runtime/graph_runtime.cc:660-664), allocates the tensors through the registered "device_api.hip"
// (include/cvm/runtime/device_api.h), passes inputs, outputs and the parsed NodeAttrs in the reference's argument
// convention (include/cvm/runtime/packed_func.h:294-314) with an ext_space tensor sized by HIPOpExtraSpace, and
// copies the results back.  Built by oracle/Makefile against the reference's headers and its compiled runtime
// (oracle/_ref/libcvm_runtime_ref.so) and against cvm-runtime_amd/libcvm_runtime_hip.so.
#include <cvm/c_api.h>
#include <cvm/node.h>
#include <cvm/op.h>
#include <cvm/op_attr_types.h>
#include <cvm/tuple.h>
#include <cvm/runtime/c_runtime_api.h>
#include <cvm/runtime/device_api.h>
#include <cvm/runtime/packed_func.h>
#include <cvm/runtime/registry.h>
#include <utils/json.h>

#include <cstring>
#include <sstream>
#include <string>
#include <vector>

namespace cvm {
namespace runtime {
int64_t HIPOpExtraSpace(const cvm::NodeAttrs& attrs, const std::vector<cvm::TShape>& in_shapes);
}
}

extern "C" {

struct PluginTensor {
  int32_t* data;       // host values: inputs are read, outputs are read (initial contents) and written
  int32_t ndim;
  int64_t shape[6];
};

static int plugin_fail(char* err, int errlen, const char* msg, int code) {
  if (err && errlen > 0) {
    std::strncpy(err, msg, errlen - 1);
    err[errlen - 1] = 0;
  }
  return code;
}

// Calls cvm.runtime.hip.<op>(in..., out..., attrs) on device copies of the tensors.  With copy_inputs_back the inputs are
// copied back as well (non_max_suppression overwrites part of its input).  0 ok, 1 logic error, 2 runtime error.
int hip_plugin_op_call(const char* op, const char* attr_json, int n_in, int n_out, PluginTensor* t, int copy_inputs_back,
                       char* err, int errlen) {
  using namespace cvm::runtime;
  const int kDLHIP = 5;   // the device type hip_device.cc gives the device
  std::vector<void*> dev;
  DeviceAPI* api = nullptr;
  CVMContext hip_ctx, cpu_ctx;
  hip_ctx.device_type = static_cast<DLDeviceType>(kDLHIP);
  hip_ctx.device_id = 0;
  cpu_ctx.device_type = kDLCPU;
  cpu_ctx.device_id = 0;
  CVMType i32;
  i32.code = kDLInt;
  i32.bits = 32;
  i32.lanes = 1;
  int status = 0;
  std::string message;
  try {
    const PackedFunc* get_api = Registry::Get("device_api.hip");
    if (!get_api) return plugin_fail(err, errlen, "device_api.hip is not registered", 2);
    void* handle = (*get_api)();
    api = static_cast<DeviceAPI*>(handle);
    api->SetDevice(hip_ctx);

    cvm::NodeAttrs attrs;
    attrs.name = op;
    attrs.op = cvm::Op::Get(op);
    std::istringstream is(attr_json);
    utils::JSONReader reader(&is);
    reader.Read(&attrs.dict);
    if (attrs.op->attr_parser) attrs.op->attr_parser(&attrs);

    const int n = n_in + n_out;
    std::vector<DLTensor> dl(n);
    std::vector<CVMValue> values(n + 1);
    std::vector<int> tcodes(n + 1);
    std::vector<size_t> bytes(n);
    std::vector<cvm::TShape> in_shapes;
    for (int i = 0; i < n; ++i) {
      int64_t count = 1;
      for (int d = 0; d < t[i].ndim; ++d) count *= t[i].shape[d];
      bytes[i] = static_cast<size_t>(count) * 4;
      void* p = api->AllocDataSpace(hip_ctx, bytes[i] ? bytes[i] : 4, 256, i32);
      dev.push_back(p);
      if (bytes[i]) api->CopyDataFromTo(t[i].data, 0, p, 0, bytes[i], cpu_ctx, hip_ctx, i32, nullptr);
      dl[i].data = p;
      dl[i].ctx = hip_ctx;
      dl[i].ndim = t[i].ndim;
      dl[i].dtype = i32;
      dl[i].shape = t[i].shape;
      dl[i].strides = nullptr;
      dl[i].byte_offset = 0;
      values[i].v_handle = &dl[i];
      tcodes[i] = kArrayHandle;
      if (i < n_in) in_shapes.push_back(cvm::TShape(t[i].shape, t[i].shape + t[i].ndim));
    }
    values[n].v_handle = &attrs;
    tcodes[n] = kHandle;

    // scratch, as the graph runtime hands it over: a one-dimensional int32 tensor
    int64_t ext_elems = HIPOpExtraSpace(attrs, in_shapes);
    DLTensor ext;
    int64_t ext_shape[1] = {ext_elems};
    void* ext_dev = nullptr;
    if (ext_elems > 0) {
      ext_dev = api->AllocDataSpace(hip_ctx, static_cast<size_t>(ext_elems) * 4, 256, i32);
      dev.push_back(ext_dev);
    }
    ext.data = ext_dev;
    ext.ctx = hip_ctx;
    ext.ndim = 1;
    ext.dtype = i32;
    ext.shape = ext_shape;
    ext.strides = nullptr;
    ext.byte_offset = 0;

    const std::string name = std::string("cvm.runtime.hip.") + op;
    const PackedFunc* f = Registry::Get(name);
    if (f == nullptr) {
      status = 2;
      message = "function undefined: " + name;
    } else {
      CVMRetValue rv;
      CVMArgs args(values.data(), tcodes.data(), n + 1, ext_elems > 0 ? &ext : nullptr);
      f->CallPacked(args, &rv);
      for (int i = copy_inputs_back ? 0 : n_in; i < n; ++i)
        if (bytes[i]) api->CopyDataFromTo(dev[i], 0, t[i].data, 0, bytes[i], hip_ctx, cpu_ctx, i32, nullptr);
    }
  } catch (const std::runtime_error& e) {
    status = 2;
    message = e.what();
  } catch (const std::logic_error& e) {
    status = 1;
    message = e.what();
  } catch (const std::exception& e) {
    status = 2;
    message = e.what();
  }
  if (api)
    for (void* p : dev) {
      try { api->FreeDataSpace(hip_ctx, p); } catch (...) {}
    }
  if (status) return plugin_fail(err, errlen, message.c_str(), status);
  return 0;
}

}  // extern "C"
