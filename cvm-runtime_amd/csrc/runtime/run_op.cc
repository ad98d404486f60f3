// CVMHIPRunOp: one registered operator on host tensors -- the single-operator
// call that the reference's tests/test_op.cc:479-660 makes for every case
// directory (parse attr.txt, FInferShape, allocate, copy in, look the packed
// function up as cvm.runtime.<dev>.<op>, call it with the extra space, copy
// out).  Everything a node of a loaded graph would get is built here for one
// node: parsed attributes, inferred output shapes, device tensors, scratch.
#include <cstring>
#include <string>
#include <vector>

#include "../../../include/cvm_c_api.h"
#include "../../../include/cvm_hip_ext.h"
#include "../../../include/cvm_hip_ops.h"
#include "graph_runtime.h"

namespace {

using cvmrt::Shape;

void DevCheck(int rc, const char* what) {
  if (rc == CVMHIP_OK) return;
  if (rc < CVMHIP_ERR_RUNTIME) CVM_VERIFY(false) << what << ": " << cvmhip_last_error();
  CVM_CHECK(false) << what << ": " << cvmhip_last_error();
}

// device allocations of one call, released on every way out
struct Arena {
  std::vector<void*> ptrs;
  void* stream = nullptr;
  void* Alloc(size_t bytes) {
    void* p = nullptr;
    DevCheck(cvmhip_alloc(&p, bytes < 256 ? 256 : bytes), "allocate tensor");
    ptrs.push_back(p);
    return p;
  }
  ~Arena() {
    if (stream) {
      cvmhip_stream_sync(stream);
      cvmhip_stream_destroy(stream);
    }
    for (void* p : ptrs) cvmhip_free(p);
  }
};

// smallest signed width that holds every value (what a graph would declare for the tensor)
int PrecisionOf(const int32_t* v, int64_t n) {
  int64_t hi = 0;
  for (int64_t i = 0; i < n; ++i) {
    const int64_t a = v[i] < 0 ? -static_cast<int64_t>(v[i]) : v[i];
    if (a > hi) hi = a;
  }
  int bits = 1;
  while ((int64_t{1} << (bits - 1)) - 1 < hi && bits < 32) ++bits;
  return bits;
}

}  // namespace

extern "C" int CVMHIPRunOp(const char* op, const char* attr_json, int n_in, const long long* in_shapes,
                           const int* in_ndims, const int* const* in_data, int max_out, int* n_out,
                           long long* out_shapes, int* out_ndims, int* const* out_data,
                           const long long* out_capacity, int* failed_stage, char* err, int errlen) {
  int stage = 0;
  auto fail = [&](const char* msg, int code) {
    if (err && errlen > 0) {
      std::strncpy(err, msg, errlen - 1);
      err[errlen - 1] = 0;
    }
    if (failed_stage) *failed_stage = stage;
    return code;
  };
  try {
    CVM_CHECK(op && attr_json && n_in >= 0 && n_out && out_shapes && out_ndims && max_out >= 1) << "CVMHIPRunOp arguments";
    CVM_CHECK(n_in == 0 || (in_shapes && in_ndims && in_data)) << "CVMHIPRunOp inputs";
    const cvmrt::OpSchema* schema = cvmrt::FindOp(op);
    if (!schema) return fail("operator is not registered", ERROR_RUNTIME);
    cvmrt::Json dict = cvmrt::Json::Parse(attr_json);
    CVM_CHECK(dict.is_object()) << "attributes must be a JSON object of strings";
    cvmrt::AttrDict ad;
    for (const auto& kv : dict.obj) {
      CVM_CHECK(kv.second.is_string()) << "attribute " << kv.first << " is not a string";
      ad.emplace_back(kv.first, kv.second.s);
    }
    const cvmrt::OpAttrs attrs = cvmrt::ParseAttrs(*schema, op, ad);
    CVM_VERIFY(cvmrt::NumInputs(*schema, attrs, n_in) == n_in) << "inputs length invalid";
    std::vector<Shape> in;
    for (int i = 0; i < n_in; ++i) {
      CVM_CHECK(in_ndims[i] >= 0 && in_ndims[i] <= 6) << "at most 6 dimensions";
      in.emplace_back(in_shapes + 6 * i, in_shapes + 6 * i + in_ndims[i]);
    }
    const std::vector<Shape> out = schema->infer_shape(attrs, in);
    CVM_CHECK(static_cast<int>(out.size()) <= max_out) << "operator has " << out.size() << " outputs";
    *n_out = static_cast<int>(out.size());
    for (size_t i = 0; i < out.size(); ++i) {
      CVM_CHECK(out[i].size() <= 6) << "at most 6 dimensions";
      out_ndims[i] = static_cast<int>(out[i].size());
      for (size_t d = 0; d < out[i].size(); ++d) out_shapes[6 * i + d] = out[i][d];
    }

    stage = 1;  // shapes are known from here on; what follows needs the device
    if (!out_data) return SUCCEED;
    CVM_CHECK(out_capacity != nullptr) << "CVMHIPRunOp output capacities";
    for (size_t i = 0; i < out.size(); ++i)
      CVM_CHECK(out_data[i] && out_capacity[i] >= cvmrt::shape_size(out[i]))
          << "output " << i << " needs " << cvmrt::shape_size(out[i]) << " elements";
    cvmrt::RegisterHipKernels();
    cvmhip_set_conv_tuning(0, -1, 0, 0);   // automatic kernel choice, whatever this thread forced before
    const std::string fname = std::string("cvm.runtime.hip.") + op;
    const cvmrt::OpKernel* kernel = cvmrt::OpRegistry::Global().Get(fname);
    CVM_VERIFY(kernel != nullptr) << "function undefined " << fname;

    Arena arena;
    DevCheck(cvmhip_stream_create(&arena.stream), "create stream");
    cvmrt::OpCall call;
    call.op = op;
    call.attrs = &attrs;
    call.stream = arena.stream;
    for (int i = 0; i < n_in; ++i) {
      cvmrt::DevTensor t;
      t.shape = in[i];
      const int64_t n = t.size();
      t.data = static_cast<int32_t*>(arena.Alloc(static_cast<size_t>(n) * 4));
      t.precision = PrecisionOf(in_data[i], n);
      if (n) DevCheck(cvmhip_copy_h2d(t.data, in_data[i], static_cast<size_t>(n) * 4, arena.stream), "copy input");
      call.in.push_back(t);
    }
    for (size_t i = 0; i < out.size(); ++i) {
      cvmrt::DevTensor t;
      t.shape = out[i];
      const int64_t n = t.size();
      t.data = static_cast<int32_t*>(arena.Alloc(static_cast<size_t>(n) * 4));
      // an output starts with the caller's bytes: some operators leave part of it untouched
      if (n) DevCheck(cvmhip_copy_h2d(t.data, out_data[i], static_cast<size_t>(n) * 4, arena.stream), "seed output");
      call.out.push_back(t);
    }
    if (kernel->workspace_bytes) {
      call.workspace_bytes = kernel->workspace_bytes(call);
      if (call.workspace_bytes) call.workspace = arena.Alloc(call.workspace_bytes);
    }
    if (kernel->prepare) kernel->prepare(call);
    kernel->run(call);
    for (size_t i = 0; i < out.size(); ++i) {
      const int64_t n = call.out[i].size();
      if (n) DevCheck(cvmhip_copy_d2h(out_data[i], call.out[i].data, static_cast<size_t>(n) * 4, arena.stream), "copy output");
    }
    DevCheck(cvmhip_stream_sync(arena.stream), "synchronise");
    call.state.reset();
  } catch (const std::runtime_error& e) {
    return fail(e.what(), ERROR_RUNTIME);
  } catch (const std::logic_error& e) {
    return fail(e.what(), ERROR_LOGIC);
  } catch (const std::exception& e) {
    return fail(e.what(), ERROR_RUNTIME);
  }
  return SUCCEED;
}
