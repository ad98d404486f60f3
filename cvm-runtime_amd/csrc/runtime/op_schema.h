// Device-independent operator schemas: attribute parsing, input/output counts,
// shape inference and precision inference for every operator the runtime can
// execute.  They restate the rules of the reference's src/top/** so that a
// graph is accepted or rejected (and with the same error class) exactly as the
// reference's CvmRuntime::Init does (src/runtime/infer_attr.cc).
#ifndef CVM_RT_OP_SCHEMA_H_
#define CVM_RT_OP_SCHEMA_H_

#include <functional>
#include <map>
#include <string>
#include <utility>
#include <vector>

#include "base.h"

namespace cvmrt {

typedef std::vector<std::pair<std::string, std::string>> AttrDict;

enum FieldType { F_INT, F_BOOL, F_TUPLE, F_STR, F_OPT_INT };

struct Field {
  const char* name;
  FieldType type;
  bool required;
  const char* def;  // default, in the attribute string syntax
};

// Parsed attributes of one node.
struct OpAttrs {
  std::string op;
  std::string node_name;
  std::map<std::string, int64_t> ints;
  std::map<std::string, bool> bools;
  std::map<std::string, Shape> tuples;
  std::map<std::string, std::string> strs;
  std::map<std::string, bool> has_opt;  // F_OPT_INT: whether a value is present

  int64_t i(const char* k) const { return ints.at(k); }
  bool b(const char* k) const { return bools.at(k); }
  const Shape& t(const char* k) const { return tuples.at(k); }
  const std::string& s(const char* k) const { return strs.at(k); }
  bool has(const char* k) const { return has_opt.at(k); }
};

struct OpSchema {
  std::string name;
  std::vector<Field> fields;
  int num_inputs;   // -1: variadic (takes the node's input count), -2: 2 or 3 by use_bias
  int num_outputs;
  // in: input shapes; returns output shapes.  Throws on violation.
  std::function<std::vector<Shape>(const OpAttrs&, const std::vector<Shape>&)> infer_shape;
  // shapes: inputs then outputs; returns output precisions.
  std::function<std::vector<int>(const OpAttrs&, const std::vector<Shape>&, const std::vector<int>&)> infer_prec;
};

// nullptr when the operator is unknown.
const OpSchema* FindOp(const std::string& name);
std::vector<std::string> ListOps();

// Parses `dict` against the schema (unknown key, missing required key or a
// malformed value -> std::runtime_error, as utils::ParamError is).
OpAttrs ParseAttrs(const OpSchema& schema, const std::string& node_name, const AttrDict& dict);

int NumInputs(const OpSchema& schema, const OpAttrs& attrs, size_t graph_inputs);

int GetReduceSumBit(int64_t size);
int GetNumberPrecision(int64_t n);

}  // namespace cvmrt
#endif
