// CVMModel for the HIP device: the host-side wrapper between the C API and the
// graph runtime (reference: include/cvm/model.h:21-66, src/core/model.cc).
// It widens int8 input bytes to the int32 storage type and turns the output
// tensors into the caller's byte layout (argmax / detection rows / int32 / int8).
#ifndef CVM_RT_MODEL_H_
#define CVM_RT_MODEL_H_

#include <memory>
#include <string>
#include <vector>

#include "graph_runtime.h"

namespace cvmrt {

class HipModel {
 public:
  HipModel(const std::string& graph, int device_id);
  void LoadParams(const std::string& params);
  int GetInputLength() const;
  int GetOutputLength() const;
  int GetSizeOfInputType() const { return input_bytes_; }
  int GetSizeOfOutputType() const { return output_bytes_; }
  int64_t GetStorageSize() const { return rt_->GetStorageSize(); }
  int64_t GetOps() const { return rt_->GetOps(); }
  std::string GetVersion() const { return version_; }
  std::string GetPostprocessMethod() const { return postprocess_; }

  void SetInput(const void* input, int size);  // PlanInput + set_input
  void Run() { rt_->Run(); }
  void GetOutput(char* mem);                   // get_output + SaveTensor
  HipGraphRuntime* runtime() { return rt_.get(); }

 private:
  void SaveTensor(const std::vector<const int32_t*>& outputs, char* mem) const;
  std::unique_ptr<HipGraphRuntime> rt_;
  int64_t in_size_ = 0;
  std::vector<int64_t> out_size_;
  std::vector<Shape> out_shape_;
  Shape in_shape_;
  int out_num_ = 0;
  int input_bytes_ = 1, output_bytes_ = 1;
  std::string version_, postprocess_;
};

}  // namespace cvmrt
#endif
