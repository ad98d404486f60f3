#include "model.h"

#include <cstring>

namespace cvmrt {

// model.cc:24-112
HipModel::HipModel(const std::string& graph, int device_id) {
  rt_.reset(new HipGraphRuntime(graph, device_id, true));
  rt_->GetStorageSize();  // enforces the storage limit at load time
  out_num_ = rt_->NumOutputs();
  postprocess_ = rt_->postprocess_method();
  input_bytes_ = rt_->GetInputPrecision() > 8 ? 4 : 1;
  output_bytes_ = rt_->GetOutputPrecision() > 8 ? 4 : 1;
  if (postprocess_ == "argmax" || postprocess_ == "detection") output_bytes_ = 4;
  version_ = rt_->version();
  in_shape_ = rt_->InputShape();
  in_size_ = shape_size(in_shape_);
  for (int k = 0; k < out_num_; ++k) {
    out_shape_.push_back(rt_->OutputShape(k));
    out_size_.push_back(shape_size(out_shape_.back()));
  }
}

void HipModel::LoadParams(const std::string& params) {
  CVM_VERIFY(params.size() != 0U);
  rt_->LoadParams(params);
}

// model.cc:293-331
int HipModel::GetInputLength() const { return static_cast<int>(in_size_) * input_bytes_; }

int HipModel::GetOutputLength() const {
  int ret = 0;
  if (postprocess_ == "argmax") {
    for (int k = 0; k < out_num_; ++k) {
      const uint32_t last_dim = static_cast<uint32_t>(out_shape_[k].back());
      ret += static_cast<uint32_t>(out_size_[k]) / last_dim;
    }
  } else if (postprocess_ == "detection") {
    const Shape& s0 = out_shape_[0];
    const int rows = s0.size() >= 2 ? static_cast<int>(s0[s0.size() - 2]) : 0;
    for (int k = 0; k < out_num_; ++k) ret += static_cast<uint32_t>(out_shape_[k].back());
    ret *= rows;
  } else {
    for (int k = 0; k < out_num_; ++k) ret += static_cast<int>(out_size_[k]);
  }
  return ret * output_bytes_;
}

// model.cc:154-169 + 284-291
void HipModel::SetInput(const void* input, int size) {
  CVM_VERIFY(GetInputLength() == size);
  if (input_bytes_ == 4) {
    rt_->SetData(static_cast<const int32_t*>(input), in_shape_);
  } else {
    rt_->SetDataI8(static_cast<const int8_t*>(input), in_shape_);   // widened on the device
  }
}

void HipModel::GetOutput(char* mem) {
  SaveTensor(rt_->FetchOutputs(), mem);   // all heads in pinned host memory, one synchronisation
}

// model.cc:181-263, restated including its loop bounds
void HipModel::SaveTensor(const std::vector<const int32_t*>& outputs, char* mem) const {
  if (postprocess_ == "argmax") {
    int32_t* cp = reinterpret_cast<int32_t*>(mem);
    for (int k = 0; k < out_num_; ++k) {
      const uint32_t last_dim = static_cast<uint32_t>(out_shape_[k].back());
      const uint32_t rows = static_cast<uint32_t>(out_size_[k]) / last_dim;
      const int32_t* data = outputs[k];
      // the row cursor advances by last_dim while bounded by the row count
      for (size_t i = 0; i < rows; i += last_dim) {
        uint32_t max_id = 0;
        for (size_t j = i; j < i + last_dim; ++j)
          if (static_cast<int8_t>(data[j]) > static_cast<int8_t>(data[i + max_id])) max_id = static_cast<uint32_t>(j - i);
        *cp++ = static_cast<int32_t>(max_id);
      }
    }
  } else if (postprocess_ == "detection" || outputs.size() > 1) {
    bool can_concat = outputs.size() != 1;
    std::vector<uint64_t> xs(outputs.size()), ys(outputs.size());
    if (can_concat) {
      for (size_t k = 0; k < outputs.size(); ++k) {
        ys[k] = static_cast<uint64_t>(out_shape_[k].back());
        xs[k] = static_cast<uint64_t>(out_size_[k]) / ys[k];
      }
      for (size_t k = 1; k < outputs.size(); ++k)
        if (xs[k] != xs[0]) { can_concat = false; break; }
    }
    CVM_VERIFY(can_concat) << "detection model output cannot concat";
    if (output_bytes_ == 4) {
      int32_t* cp = reinterpret_cast<int32_t*>(mem);
      const int32_t nx = static_cast<int32_t>(xs[0]);
      for (int x = 0; x < nx; ++x)
        for (size_t k = 0; k < outputs.size(); ++k) {
          const int32_t* row = outputs[k] + static_cast<size_t>(x) * ys[k];
          for (size_t i = 0; i < ys[k]; ++i) *cp++ = row[i];
        }
    } else {
      char* cp = mem;
      for (size_t x = 0; x < xs[0]; ++x)
        for (size_t k = 0; k < outputs.size(); ++k) {
          const int32_t* row = outputs[k] + x * ys[k];
          for (size_t i = 0; i < ys[k]; ++i) *cp++ = static_cast<int8_t>(row[i]);
        }
    }
  } else if (output_bytes_ == 4) {
    int32_t* ref = reinterpret_cast<int32_t*>(mem);
    for (size_t k = 0; k < outputs.size(); ++k) {
      std::memcpy(ref, outputs[k], sizeof(int32_t) * static_cast<size_t>(out_size_[k]));
      ref += out_size_[k];
    }
  } else {
    for (size_t k = 0; k < outputs.size(); ++k)
      for (int64_t i = 0; i < out_size_[k]; ++i) *mem++ = static_cast<int8_t>(outputs[k][i]);
  }
}

}  // namespace cvmrt
