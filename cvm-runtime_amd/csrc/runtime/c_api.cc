// The model-level C ABI (include/cvm_c_api.h) and the backend's extensions
// (include/cvm_hip_ext.h).  Exceptions stop here and become status codes, with
// the message printed as "ERROR: ..." (include/cvm/errors.h:15-36).
#include <cstdio>
#include <cstring>
#include <sstream>

#include "../../../include/cvm_c_api.h"
#include "../../../include/cvm_hip_ext.h"
#include "../../../include/cvm_hip_ops.h"
#include "model.h"

using cvmrt::HipModel;

#define API_BEGIN() try {
#define API_END()                                                           \
  }                                                                         \
  catch (const std::runtime_error& e) { std::printf("ERROR: %s\n", e.what()); return ERROR_RUNTIME; } \
  catch (const std::logic_error& e) { std::printf("ERROR: %s\n", e.what()); return ERROR_LOGIC; }     \
  catch (const std::exception& e) { std::printf("ERROR: %s\n", e.what()); return ERROR_RUNTIME; }     \
  return SUCCEED;

#define NOT_NULL(x) CVM_CHECK((x) != nullptr)

extern "C" {

int CVMAPILoadModel(const char* graph_json, int graph_strlen, const char* param_bytes, int param_strlen,
                    void** net, int device_type, int device_id) {
  API_BEGIN();
  NOT_NULL(graph_json);
  NOT_NULL(param_bytes);
  NOT_NULL(net);
  CVM_CHECK(graph_strlen >= 0 && param_strlen >= 0);
  const std::string graph(graph_json, graph_strlen);
  const std::string params(param_bytes, param_strlen);
  CVM_CHECK(device_type >= 0 && device_type <= 3)
      << "Invalid device type: " << device_type << ", only supported 0(CPU), 1(GPU), 2(FORMAL), 3(HIP)\n";
  CVM_CHECK(device_type == 1 || device_type == 3)
      << "device type " << device_type << " is not built into this library (the gfx950 backend serves 1 and 3)";
  HipModel* model = nullptr;
  try {
    model = new HipModel(graph, device_id);
    model->LoadParams(params);
  } catch (...) {
    delete model;
    throw;
  }
  *net = model;
  API_END();
}

int CVMAPIFreeModel(void* net) {
  API_BEGIN();
  if (net) delete static_cast<HipModel*>(net);
  API_END();
}

int CVMAPIInference(void* net, char* input_data, int input_len, char* output_data) {
  API_BEGIN();
  NOT_NULL(net);
  NOT_NULL(input_data);
  NOT_NULL(output_data);
  HipModel* model = static_cast<HipModel*>(net);
  model->SetInput(input_data, input_len);
  model->Run();
  model->GetOutput(output_data);
  API_END();
}

int CVMAPIGetVersion(void* net, char* version) {
  API_BEGIN();
  NOT_NULL(net);
  NOT_NULL(version);
  std::strcpy(version, static_cast<HipModel*>(net)->GetVersion().c_str());
  API_END();
}

int CVMAPIGetPreprocessMethod(void* net, char* method) {
  API_BEGIN();
  NOT_NULL(net);
  NOT_NULL(method);
  std::strcpy(method, static_cast<HipModel*>(net)->GetPostprocessMethod().c_str());
  API_END();
}

#define SIZE_GETTER(NAME, EXPR)                                   \
  int NAME(void* net, unsigned long long* size) {                 \
    API_BEGIN();                                                  \
    NOT_NULL(net);                                                \
    NOT_NULL(size);                                               \
    HipModel* model = static_cast<HipModel*>(net);                \
    *size = static_cast<unsigned long long>(EXPR);                \
    API_END();                                                    \
  }

SIZE_GETTER(CVMAPIGetInputLength, model->GetInputLength())
SIZE_GETTER(CVMAPIGetOutputLength, model->GetOutputLength())
SIZE_GETTER(CVMAPIGetInputTypeSize, model->GetSizeOfInputType())
SIZE_GETTER(CVMAPIGetOutputTypeSize, model->GetSizeOfOutputType())
SIZE_GETTER(CVMAPIGetStorageSize, model->GetStorageSize())
SIZE_GETTER(CVMAPIGetGasFromModel, model->GetOps())

int CVMAPIGetGasFromGraphFile(const char* graph_json, unsigned long long* gas) {
  API_BEGIN();
  NOT_NULL(graph_json);
  NOT_NULL(gas);
  cvmrt::HipGraphRuntime rt(std::string(graph_json), 0, false);
  *gas = static_cast<unsigned long long>(rt.GetOps());
  API_END();
}

// ---------------------------------------------------------------- extensions
int CVMHIPSetInput(void* net, const char* input_data, int input_len) {
  API_BEGIN();
  NOT_NULL(net);
  NOT_NULL(input_data);
  static_cast<HipModel*>(net)->SetInput(input_data, input_len);
  API_END();
}

int CVMHIPRun(void* net) {
  API_BEGIN();
  NOT_NULL(net);
  static_cast<HipModel*>(net)->Run();
  static_cast<HipModel*>(net)->runtime()->SyncStream();
  API_END();
}

int CVMHIPGetOutput(void* net, char* output_data) {
  API_BEGIN();
  NOT_NULL(net);
  NOT_NULL(output_data);
  static_cast<HipModel*>(net)->GetOutput(output_data);
  API_END();
}

int CVMHIPTimeRun(void* net, int iterations, float* elapsed_ms) {
  API_BEGIN();
  NOT_NULL(net);
  NOT_NULL(elapsed_ms);
  CVM_CHECK(iterations >= 1);
  *elapsed_ms = static_cast<HipModel*>(net)->runtime()->TimeRuns(iterations);
  API_END();
}

int CVMHIPLaunchCounts(void* net, int* launches_per_run, int* sequence_launches, int* layers_in_sequences) {
  API_BEGIN();
  NOT_NULL(net);
  static_cast<HipModel*>(net)->runtime()->LaunchCounts(launches_per_run, sequence_launches, layers_in_sequences);
  API_END();
}

int CVMHIPSequenceConfigs(void* net, int* configs, int capacity, int* count) {
  API_BEGIN();
  NOT_NULL(net);
  NOT_NULL(count);
  const std::vector<int> v = static_cast<HipModel*>(net)->runtime()->SequenceConfigs();
  *count = static_cast<int>(v.size());
  for (int i = 0; configs && i < capacity && i < *count; ++i) configs[i] = v[i];
  API_END();
}

int CVMHIPProfileOps(void* net, char* json_out, int capacity) {
  API_BEGIN();
  NOT_NULL(net);
  NOT_NULL(json_out);
  auto times = static_cast<HipModel*>(net)->runtime()->ProfileRun();
  std::ostringstream os;
  os << "{";
  bool first = true;
  for (const auto& kv : times) {
    os << (first ? "" : ", ") << "\"" << kv.first << "\": " << kv.second;
    first = false;
  }
  os << "}";
  const std::string s = os.str();
  CVM_CHECK(static_cast<int>(s.size()) < capacity) << "profile buffer too small";
  std::strcpy(json_out, s.c_str());
  API_END();
}

int CVMHIPInferNode(const char* op, const char* attr_json, int n_in, const long long* in_shapes, const int* in_ndims,
                    const int* in_precs, int* n_out, long long* out_shapes, int* out_ndims, int* out_precs, char* err,
                    int errlen) {
  auto fail = [&](const char* msg, int code) {
    if (err && errlen > 0) {
      std::strncpy(err, msg, errlen - 1);
      err[errlen - 1] = 0;
    }
    return code;
  };
  try {
    const cvmrt::OpSchema* schema = cvmrt::FindOp(op);
    if (!schema) return fail("operator is not registered", ERROR_RUNTIME);
    cvmrt::Json dict = cvmrt::Json::Parse(attr_json);
    CVM_CHECK(dict.is_object());
    cvmrt::AttrDict ad;
    for (const auto& kv : dict.obj) {
      CVM_CHECK(kv.second.is_string());
      ad.emplace_back(kv.first, kv.second.s);
    }
    cvmrt::OpAttrs attrs = cvmrt::ParseAttrs(*schema, op, ad);
    CVM_VERIFY(cvmrt::NumInputs(*schema, attrs, n_in) == n_in) << "inputs length invalid";
    std::vector<cvmrt::Shape> in;
    for (int i = 0; i < n_in; ++i) in.emplace_back(in_shapes + 6 * i, in_shapes + 6 * i + in_ndims[i]);
    std::vector<cvmrt::Shape> out = schema->infer_shape(attrs, in);
    std::vector<cvmrt::Shape> all(in);
    all.insert(all.end(), out.begin(), out.end());
    std::vector<int> ip(in_precs, in_precs + n_in);
    std::vector<int> op_prec = schema->infer_prec(attrs, all, ip);
    *n_out = static_cast<int>(out.size());
    for (size_t i = 0; i < out.size(); ++i) {
      out_ndims[i] = static_cast<int>(out[i].size());
      for (size_t d = 0; d < out[i].size() && d < 6; ++d) out_shapes[6 * i + d] = out[i][d];
      out_precs[i] = op_prec[i];
    }
  } catch (const std::runtime_error& e) {
    return fail(e.what(), ERROR_RUNTIME);
  } catch (const std::logic_error& e) {
    return fail(e.what(), ERROR_LOGIC);
  } catch (const std::exception& e) {
    return fail(e.what(), ERROR_RUNTIME);
  }
  return SUCCEED;
}

int CVMHIPListOps(char* out, int capacity) {
  API_BEGIN();
  NOT_NULL(out);
  cvmrt::RegisterHipKernels();
  std::string s;
  for (const std::string& n : cvmrt::OpRegistry::Global().ListNames()) s += n + "\n";
  CVM_CHECK(static_cast<int>(s.size()) < capacity);
  std::strcpy(out, s.c_str());
  API_END();
}

}  // extern "C"
