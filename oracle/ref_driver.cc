// Test infrastructure only (never linked into the product library).
//
// A thin driver over the *compiled reference runtime* (oracle/_ref/
// libcvm_runtime_ref.so, built from /root/reference sources in place).  It
// exposes two plain-C entry points so Python tests can (1) call a single
// reference operator `cvm.runtime.<dev>.<op>` the way the reference's own
// tests/test_op.cc:92-150 does, and (2) run the reference's shape / precision
// inference for one node (src/runtime/infer_attr.cc:31-91,161-217).
//
// This file contains no reference code; it only includes the reference's
// public headers where they lie and calls through its registry.
#include <cvm/c_api.h>
#include <cvm/op.h>
#include <cvm/node.h>
#include <cvm/op_attr_types.h>
#include <cvm/runtime/registry.h>
#include <cvm/runtime/packed_func.h>
#include <cvm/runtime/c_runtime_api.h>
#include <utils/json.h>

#include <cstring>
#include <sstream>
#include <string>
#include <vector>

extern "C" {

struct RefTensor {
  int32_t* data;
  int32_t ndim;
  int64_t shape[6];
};

static int fail(char* err, int errlen, const char* msg, int code) {
  if (err && errlen > 0) {
    std::strncpy(err, msg, errlen - 1);
    err[errlen - 1] = 0;
  }
  return code;
}

static void make_attrs(const char* op, const char* attr_json, cvm::NodeAttrs* attrs) {
  attrs->name = op;
  attrs->op = cvm::Op::Get(op);
  std::istringstream is(attr_json);
  utils::JSONReader reader(&is);
  reader.Read(&attrs->dict);
  if (attrs->op->attr_parser) attrs->op->attr_parser(attrs);
}

// Calls cvm.runtime.<dev>.<op>(in..., out..., attrs).  0 ok, 1 logic error,
// 2 runtime error (same mapping as include/cvm/errors.h:15-36).
int ref_op_call(const char* dev, const char* op, const char* attr_json,
                int n_in, int n_out, RefTensor* t, char* err, int errlen) {
  try {
    cvm::NodeAttrs attrs;
    make_attrs(op, attr_json, &attrs);
    int n = n_in + n_out;
    std::vector<DLTensor> dl(n);
    std::vector<CVMValue> values(n + 1);
    std::vector<int> tcodes(n + 1);
    for (int i = 0; i < n; ++i) {
      dl[i].data = t[i].data;
      dl[i].ctx.device_type = kDLCPU;
      dl[i].ctx.device_id = 0;
      dl[i].ndim = t[i].ndim;
      dl[i].dtype.code = kDLInt;
      dl[i].dtype.bits = 32;
      dl[i].dtype.lanes = 1;
      dl[i].shape = t[i].shape;
      dl[i].strides = nullptr;
      dl[i].byte_offset = 0;
      values[i].v_handle = &dl[i];
      tcodes[i] = kArrayHandle;
    }
    values[n].v_handle = &attrs;
    tcodes[n] = kHandle;
    std::string name = std::string("cvm.runtime.") + dev + "." + op;
    auto* f = cvm::runtime::Registry::Get(name);
    if (f == nullptr) return fail(err, errlen, "function undefined", 2);
    cvm::runtime::CVMRetValue rv;
    cvm::runtime::CVMArgs args(values.data(), tcodes.data(), n + 1, nullptr);
    f->CallPacked(args, &rv);
  } catch (const std::runtime_error& e) {
    return fail(err, errlen, e.what(), 2);
  } catch (const std::logic_error& e) {
    return fail(err, errlen, e.what(), 1);
  } catch (const std::exception& e) {
    return fail(err, errlen, e.what(), 2);
  }
  return 0;
}

// Runs attr parsing + FInferShape + FInferPrecision for one node.
// in: shapes + precisions of inputs; out: shapes (filled) + precisions (filled).
// *n_out receives the operator's output count.  Same status codes as above.
// in_prec == NULL: attribute parsing and FInferShape only.
int ref_op_infer(const char* op, const char* attr_json, int n_in,
                 const RefTensor* in, const int* in_prec, int max_out,
                 int* n_out, RefTensor* out, int* out_prec, char* err,
                 int errlen) {
  try {
    cvm::NodeAttrs attrs;
    make_attrs(op, attr_json, &attrs);
    uint32_t nout = attrs.op->get_num_outputs ? attrs.op->get_num_outputs(attrs)
                                              : attrs.op->num_outputs;
    if ((int)nout > max_out) return fail(err, errlen, "too many outputs", 2);
    *n_out = (int)nout;
    static auto& fshape = cvm::Op::GetAttr<cvm::FInferShape>("FInferShape");
    static auto& fprec = cvm::Op::GetAttr<cvm::FInferPrecision>("FInferPrecision");
    std::vector<cvm::TShape> ishape(n_in), oshape(nout);
    for (int i = 0; i < n_in; ++i)
      ishape[i] = cvm::TShape(in[i].shape, in[i].shape + in[i].ndim);
    auto fs = fshape.get(attrs.op, nullptr);
    if (fs == nullptr) return fail(err, errlen, "no FInferShape", 2);
    if (!fs(attrs, &ishape, &oshape)) return fail(err, errlen, "infer shape failed", 2);
    std::vector<cvm::TShape> shapes(ishape);
    for (uint32_t i = 0; i < nout; ++i) {
      out[i].ndim = oshape[i].ndim();
      for (int d = 0; d < (int)oshape[i].ndim() && d < 6; ++d) out[i].shape[d] = oshape[i][d];
      shapes.push_back(oshape[i]);
    }
    if (in_prec == nullptr) return 0;  // shapes only, as tests/test_op.cc:522-556 does before it runs a case
    std::vector<int> ip(in_prec, in_prec + n_in), opv(nout, -1);
    auto fp = fprec.get(attrs.op, nullptr);
    if (fp == nullptr) return fail(err, errlen, "no FInferPrecision", 2);
    if (!fp(attrs, &shapes, &ip, &opv)) return fail(err, errlen, "infer precision failed", 2);
    for (uint32_t i = 0; i < nout; ++i) out_prec[i] = opv[i];
  } catch (const std::runtime_error& e) {
    return fail(err, errlen, e.what(), 2);
  } catch (const std::logic_error& e) {
    return fail(err, errlen, e.what(), 1);
  } catch (const std::exception& e) {
    return fail(err, errlen, e.what(), 2);
  }
  return 0;
}

}  // extern "C"
