// Minimal JSON document reader (objects keep key order; numbers are kept as
// int64 when integral).  Enough for CVM graph files; parse errors throw
// std::runtime_error like the reference's JSONReader CHECKs.
#ifndef CVM_RT_JSON_H_
#define CVM_RT_JSON_H_

#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "base.h"

namespace cvmrt {

struct Json {
  enum Kind { kNull, kBool, kInt, kDouble, kString, kArray, kObject };
  Kind kind = kNull;
  bool b = false;
  int64_t i = 0;
  double d = 0;
  std::string s;
  std::vector<Json> arr;
  std::vector<std::pair<std::string, Json>> obj;

  bool is_object() const { return kind == kObject; }
  bool is_array() const { return kind == kArray; }
  bool is_string() const { return kind == kString; }
  bool is_int() const { return kind == kInt; }

  static Json Parse(const std::string& text);
};

}  // namespace cvmrt
#endif
