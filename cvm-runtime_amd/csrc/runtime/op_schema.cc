#include "op_schema.h"

#include <algorithm>
#include <cctype>
#include <cstdlib>
#include <set>
#include <sstream>

namespace cvmrt {

// ---------------------------------------------------------------- attribute values
namespace {

[[noreturn]] void ParamFail(const Field& f, const std::string& value, const OpAttrs& a) {
  // utils::ParamError derives from std::runtime_error in the reference
  CVM_FATAL() << "Invalid Parameter format for " << f.name << " value='" << value << "', in operator " << a.op
              << "(name=\"" << a.node_name << "\")";
  std::abort();
}

bool ParseInt(const std::string& v, int64_t* out) {
  const char* s = v.c_str();
  while (std::isspace(static_cast<unsigned char>(*s))) ++s;
  char* end = nullptr;
  errno = 0;
  long long r = std::strtoll(s, &end, 10);
  if (end == s || errno != 0) return false;
  while (*end) {
    if (!std::isspace(static_cast<unsigned char>(*end))) return false;
    ++end;
  }
  if (r < INT32_MIN || r > INT32_MAX) return false;  // every integer attribute is a 32-bit field
  *out = r;
  return true;
}

// "(1, 2)", "[1, 2]", "(3,)", "()", or a bare integer "3" (include/cvm/tuple.h:221-280)
bool ParseTuple(const std::string& v, Shape* out) {
  out->clear();
  size_t p = 0;
  while (p < v.size()) {
    char ch = v[p];
    if (std::isdigit(static_cast<unsigned char>(ch)) || ch == '-') {
      char* end = nullptr;
      long long r = std::strtoll(v.c_str() + p, &end, 10);
      if (end == v.c_str() + p) return false;
      out->push_back(r);
      return true;
    }
    ++p;
    if (ch == '(' || ch == '[') break;
    if (!std::isspace(static_cast<unsigned char>(ch))) return false;
  }
  if (p >= v.size()) return false;
  while (p < v.size() && std::isspace(static_cast<unsigned char>(v[p]))) ++p;
  if (p < v.size() && (v[p] == ')' || v[p] == ']')) return true;
  while (true) {
    char* end = nullptr;
    const char* s = v.c_str() + p;
    long long r = std::strtoll(s, &end, 10);
    if (end == s) return false;
    out->push_back(r);
    p = static_cast<size_t>(end - v.c_str());
    while (p < v.size() && std::isspace(static_cast<unsigned char>(v[p]))) ++p;
    if (p < v.size() && v[p] == 'L') ++p;
    if (p >= v.size()) return false;
    if (v[p] == ',') {
      ++p;
      while (p < v.size() && std::isspace(static_cast<unsigned char>(v[p]))) ++p;
      if (p < v.size() && (v[p] == ')' || v[p] == ']')) return true;
    } else if (v[p] == ')' || v[p] == ']') {
      return true;
    } else {
      return false;
    }
  }
}

void SetField(const Field& f, const std::string& value, OpAttrs* a) {
  switch (f.type) {
    case F_INT: {
      int64_t r;
      if (!ParseInt(value, &r)) ParamFail(f, value, *a);
      a->ints[f.name] = r;
      break;
    }
    case F_OPT_INT: {
      if (value == "None") { a->has_opt[f.name] = false; a->ints[f.name] = 0; break; }
      int64_t r;
      if (!ParseInt(value, &r)) ParamFail(f, value, *a);
      a->ints[f.name] = r;
      a->has_opt[f.name] = true;
      break;
    }
    case F_BOOL: {
      std::string lc(value);
      std::transform(lc.begin(), lc.end(), lc.begin(), ::tolower);
      if (lc == "true" || lc == "1") a->bools[f.name] = true;
      else if (lc == "false" || lc == "0") a->bools[f.name] = false;
      else ParamFail(f, value, *a);
      break;
    }
    case F_TUPLE: {
      Shape t;
      if (!ParseTuple(value, &t)) ParamFail(f, value, *a);
      a->tuples[f.name] = t;
      break;
    }
    case F_STR:
      a->strs[f.name] = value;
      break;
  }
}

}  // namespace

OpAttrs ParseAttrs(const OpSchema& schema, const std::string& node_name, const AttrDict& dict) {
  OpAttrs a;
  a.op = schema.name;
  a.node_name = node_name;
  std::set<std::string> seen;
  for (const auto& kv : dict) {
    const Field* f = nullptr;
    for (const auto& cand : schema.fields)
      if (kv.first == cand.name) f = &cand;
    if (f == nullptr) {
      // "__hidden__" keys are tolerated (kAllowHidden, include/utils/parameter.h:411-417)
      const std::string& k = kv.first;
      if (k.size() > 4 && k.compare(0, 2, "__") == 0 && k.compare(k.size() - 2, 2, "__") == 0) continue;
      if (schema.fields.empty()) {
        CVM_VERIFY(false) << "operator " << schema.name << " name=" << node_name << " should not have attributes";
      }
      CVM_FATAL() << "Cannot find argument '" << k << "', in operator " << schema.name << "(name=\"" << node_name << "\")";
    }
    SetField(*f, kv.second, &a);
    seen.insert(kv.first);
  }
  for (const auto& f : schema.fields) {
    if (seen.count(f.name)) continue;
    if (f.required)
      CVM_FATAL() << "Required parameter " << f.name << " of operator " << schema.name << " is not presented, name=\""
                  << node_name << "\"";
    SetField(f, f.def, &a);
  }
  if (schema.name == "dense") {
    if (a.i("units") < 1) CVM_FATAL() << "value " << a.i("units") << " for Parameter units should be greater equal to 1";
  }
  if (schema.name == "expand_dims") {
    if (a.i("num_newaxis") < 1) CVM_FATAL() << "value for Parameter num_newaxis should be greater equal to 1";
  }
  if (schema.name == "conv2d") {
    static const char* kTypes[] = {"same", "float16", "float32", "float64", "uint8", "uint16", "uint32",
                                   "uint64", "int8", "int16", "int32", "int64"};
    bool ok = false;
    for (const char* t : kTypes) ok = ok || a.s("out_dtype") == t;
    if (!ok) CVM_FATAL() << "Invalid Input: '" << a.s("out_dtype") << "' for out_dtype";
  }
  if (schema.name == "sum" || schema.name == "max") {
    // AxesParamParser sorts the raw axis values (src/top/tensor/reduce.cc:96-102)
    Shape& ax = a.tuples["axis"];
    std::sort(ax.begin(), ax.end());
  }
  return a;
}

int NumInputs(const OpSchema& schema, const OpAttrs& attrs, size_t graph_inputs) {
  if (schema.num_inputs == -1) return static_cast<int>(graph_inputs);
  if (schema.num_inputs == -2) return attrs.b("use_bias") ? 3 : 2;
  return schema.num_inputs;
}

int GetReduceSumBit(int64_t size) {
  int prec = 0;
  while (size != 0) { ++prec; size >>= 1; }
  return prec;
}

int GetNumberPrecision(int64_t n) {
  int prec = 0;
  n = n + 1;
  while (n != 0) { ++prec; n >>= 1; }
  return prec + 1;
}

// ---------------------------------------------------------------- inference helpers
namespace {

const int kAttrMin = 0, kAttrMax = 4096;  // src/top/op_common.h:23-24

void VerifyAttrRange(int64_t val, const char* name, int64_t lo = kAttrMin, int64_t hi = kAttrMax) {
  CVM_VERIFY(lo <= val && val <= hi) << "attribute " << name << " value: " << val << " out of range [" << lo << ", " << hi << "]";
}

// an input whose shape the operator dictates (CVM_ASSIGN_INPUT_SHAPE -> LOG(FATAL) on mismatch)
void ExpectInput(const OpAttrs& a, const std::vector<Shape>& in, size_t index, const Shape& want) {
  if (in[index] != want)
    CVM_FATAL() << "Operator " << a.op << "(name=" << a.node_name << ") expects input " << index << "'s shape to be "
                << shape_str(want) << ", but got " << shape_str(in[index]) << ".";
}

void InPrecCheck(const OpAttrs& a, const std::vector<int>& ip) {
  for (size_t i = 0; i < ip.size(); ++i)
    CVM_VERIFY(ip[i] != -1) << "operator " << a.node_name << "'s inputs(" << i << ") has not been infered precision";
}

std::vector<int> SamePrec(const OpAttrs& a, const std::vector<Shape>&, const std::vector<int>& ip) {
  InPrecCheck(a, ip);
  return {ip.at(0)};
}

std::vector<int> PlusPrec(const OpAttrs& a, const std::vector<Shape>&, const std::vector<int>& ip) {
  InPrecCheck(a, ip);
  CVM_VERIFY(ip.size() == 2U);
  return {std::max(ip[0], ip[1]) + 1};
}

std::vector<int> MulPrec(const OpAttrs& a, const std::vector<Shape>&, const std::vector<int>& ip) {
  InPrecCheck(a, ip);
  CVM_VERIFY(ip.size() == 2U);
  return {ip[0] + ip[1]};
}

std::vector<int> MaxInPrec(const OpAttrs& a, const std::vector<Shape>&, const std::vector<int>& ip) {
  InPrecCheck(a, ip);
  CVM_VERIFY(ip.size() > 0U);
  return {*std::max_element(ip.begin(), ip.end())};
}

std::vector<Shape> SameShape1(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 1U) << " in operator " << a.node_name;
  return {in[0]};
}

std::vector<Shape> SameShape2(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 2U) << " in operator " << a.node_name;
  CVM_VERIFY(in[0] == in[1]) << "Incompatible attr in node " << a.node_name << ": expected " << shape_str(in[0])
                             << ", got " << shape_str(in[1]);
  return {in[0]};
}

std::vector<Shape> BroadcastShape(const OpAttrs&, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 2U);
  const Shape& l = in[0];
  const Shape& r = in[1];
  if (l == r) return {l};
  const size_t nd = std::max(l.size(), r.size());
  Shape out(nd);
  const size_t bl = nd - l.size(), br = nd - r.size();
  for (size_t i = 0; i < nd; ++i) {
    const int64_t lv = i >= bl ? l[i - bl] : 1, rv = i >= br ? r[i - br] : 1;
    if (lv != rv) {
      CVM_VERIFY(lv == 1 || rv == 1) << "operands could not be broadcast together with shapes " << shape_str(l) << " "
                                     << shape_str(r);
      out[i] = std::max(lv, rv);
    } else {
      out[i] = lv;
    }
  }
  return {out};
}

std::vector<Shape> ConvShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(a.s("layout") == "NCHW") << "Conv2D only supported layout: NCHW vs. " << a.s("layout");
  CVM_VERIFY(a.s("kernel_layout") == "OIHW") << "Conv2D only supported kernel layout: OIHW vs. " << a.s("kernel_layout");
  CVM_VERIFY(a.s("out_layout") == "__undef__" || a.s("out_layout") == "NCHW");
  const bool use_bias = a.b("use_bias");
  CVM_VERIFY(in.size() == (use_bias ? 3U : 2U)) << "Input:[data, weight" << (use_bias ? ", bias]" : "]");
  const Shape& d = in[0];
  CVM_VERIFY(d.size() == 4U) << "Input data should be 4D";
  const Shape &ks = a.t("kernel_size"), &pad = a.t("padding"), &st = a.t("strides"), &dil = a.t("dilation");
  CVM_VERIFY(ks.size() == 2U);
  CVM_VERIFY(pad.size() == 2U);
  VerifyAttrRange(pad[0], "Conv2D.padding[0]");
  VerifyAttrRange(pad[1], "Conv2D.padding[1]");
  CVM_VERIFY(st.size() == 2U) << "incorrect stride size";
  VerifyAttrRange(st[0], "Conv2D.strides[0]", 1);
  VerifyAttrRange(st[1], "Conv2D.strides[1]", 1);
  CVM_VERIFY(dil.size() == 2U) << "incorrect dilate size";
  VerifyAttrRange(dil[0], "Conv2D.dilation[0]", 1);
  VerifyAttrRange(dil[1], "Conv2D.dilation[1]", 1);
  const int64_t groups = a.i("groups"), channels = a.i("channels");
  CVM_VERIFY(groups > 0 && d[1] % groups == 0 && channels % groups == 0)
      << "Conv2D only supported groups (1 or in_channels " << channels << ") vs. " << groups;
  // the filter shape is only assigned when unknown (src/top/nn/convolution.cc:75-77), never
  // compared; the kernel wrapper rejects a mismatching filter when the node runs
  if (use_bias) ExpectInput(a, in, 2, Shape{channels});
  const int64_t ky = 1 + (ks[0] - 1) * dil[0], kx = 1 + (ks[1] - 1) * dil[1];
  Shape o{d[0], channels, (d[2] + pad[0] * 2 - ky) / st[0] + 1, (d[3] + pad[1] * 2 - kx) / st[1] + 1};
  CVM_VERIFY(ky <= d[2] + 2 * pad[0]) << "kernel size exceed input";
  CVM_VERIFY(kx <= d[3] + 2 * pad[1]) << "kernel size exceed input";
  return {o};
}

std::vector<int> ConvPrec(const OpAttrs& a, const std::vector<Shape>& shapes, const std::vector<int>& ip) {
  InPrecCheck(a, ip);
  CVM_VERIFY(ip.at(0) <= 8) << "Conv2D " << a.node_name << " input must be INT8 vs. INT" << ip[0];
  CVM_VERIFY(ip.at(1) <= 8) << "Conv2D " << a.node_name << " weight must be INT8 vs. INT" << ip[1];
  const Shape& w = shapes.at(1);
  CVM_VERIFY(w.size() == 4U);
  int oprec = ip[0] + ip[1] + GetReduceSumBit(shape_size(w) / w[0]);
  if (a.b("use_bias")) oprec = std::max(oprec, ip.at(2)) + 1;
  return {oprec};
}

std::vector<Shape> DenseShape(const OpAttrs& a, const std::vector<Shape>& in) {
  const bool use_bias = a.b("use_bias");
  CVM_VERIFY(in.size() == (use_bias ? 3U : 2U)) << "Input:[data, weight" << (use_bias ? ", bias]" : "]");
  CVM_VERIFY(in[0].size() == 2U) << "dense require 2-D data";
  CVM_VERIFY(in[1].size() == 2U) << "dense require 2-D weight";
  const int64_t units = a.i("units");
  ExpectInput(a, in, 1, Shape{units, in[0][1]});
  if (use_bias) ExpectInput(a, in, 2, Shape{units});
  return {Shape{in[0][0], units}};
}

std::vector<int> DensePrec(const OpAttrs& a, const std::vector<Shape>& shapes, const std::vector<int>& ip) {
  CVM_VERIFY(ip.at(0) <= 8) << "Dense " << a.node_name << " input must be INT8 vs. INT" << ip[0];
  CVM_VERIFY(ip.at(1) <= 8) << "Dense " << a.node_name << " weight must be INT8 vs. INT" << ip[1];
  int oprec = ip[0] + ip[1] + GetReduceSumBit(shapes.at(0)[1]);
  if (a.b("use_bias")) oprec = std::max(oprec, ip.at(2)) + 1;
  return {oprec};
}

std::vector<Shape> PoolShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 1U);
  const Shape& d = in[0];
  CVM_VERIFY(d.size() == 4U) << "Pool2D only support input = 4-D: NCHW";
  CVM_VERIFY(a.s("layout") == "NCHW") << "Pool2D only supported NCHW layout vs. " << a.s("layout");
  const Shape &pad = a.t("padding"), &ps = a.t("pool_size"), &st = a.t("strides");
  CVM_VERIFY(pad.size() == 1U || pad.size() == 2U) << "Pool2D only supported 1-D or 2-D padding";
  VerifyAttrRange(pad[0], "MaxPool2D.padding[0]");
  int64_t pad_h = pad[0] * 2, pad_w = pad[0] * 2;
  if (pad.size() == 2) {
    pad_w = pad[1] * 2;
    VerifyAttrRange(pad[1], "MaxPool2D.padding[1]");
  }
  CVM_VERIFY(ps.size() == 2U);
  CVM_VERIFY(st.size() == 2U);
  VerifyAttrRange(st[0], "MaxPool2D.strides[0]", 1);
  VerifyAttrRange(st[1], "MaxPool2D.strides[1]", 1);
  VerifyAttrRange(ps[0], "MaxPool2D.pool_size[0]", 0, d[2] + pad_h);
  VerifyAttrRange(ps[1], "MaxPool2D.pool_size[1]", 0, d[3] + pad_w);
  const int64_t tp0 = pad[0], tp1 = pad.size() == 2 ? pad[1] : pad[0];
  CVM_VERIFY(tp0 < ps[0]);
  CVM_VERIFY(tp1 < ps[1]);
  Shape o = d;
  if (!a.b("ceil_mode")) {
    o[2] = (d[2] + pad_h - ps[0]) / st[0] + 1;
    o[3] = (d[3] + pad_w - ps[1]) / st[1] + 1;
  } else {
    o[2] = (d[2] + pad_h - ps[0] + st[0] - 1) / st[0] + 1;
    const int32_t min_o_h = static_cast<int32_t>((o[2] - 1) * st[0] - pad[0]);
    CVM_VERIFY(min_o_h < d[2]);
    o[3] = (d[3] + pad_w - ps[1] + st[1] - 1) / st[1] + 1;
    const int32_t min_o_w = static_cast<int32_t>((o[3] - 1) * st[1] - tp1);
    CVM_VERIFY(min_o_w < d[3]);
  }
  return {o};
}

Shape ReduceAxes(int64_t indim, const Shape& axis, bool exclude) {
  if (axis.empty()) {
    Shape r(indim);
    for (int64_t i = 0; i < indim; ++i) r[i] = i;
    return r;
  }
  Shape in_axis = axis;
  for (auto& i : in_axis) {
    i = i < 0 ? i + indim : i;
    VerifyAttrRange(i, "reduce.axis", 0, indim - 1);
  }
  std::sort(in_axis.begin(), in_axis.end());
  for (size_t i = 0; i + 1 < in_axis.size(); ++i) CVM_VERIFY(in_axis[i] != in_axis[i + 1]);
  if (!exclude) return in_axis;
  Shape r;
  for (int64_t i = 0; i < indim; ++i)
    if (!std::binary_search(in_axis.begin(), in_axis.end(), i)) r.push_back(i);
  return r;
}

std::vector<Shape> ReduceShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 1U);
  const Shape& ishape = in[0];
  const int64_t indim = static_cast<int64_t>(ishape.size());
  const Shape r = ReduceAxes(indim, a.t("axis"), a.b("exclude"));
  const bool keepdims = a.b("keepdims");
  if (r.empty()) return {ishape};
  if (static_cast<int64_t>(r.size()) == indim) return {Shape(keepdims ? indim : 1, 1)};
  Shape o;
  for (int64_t i = 0; i < indim; ++i) {
    const bool reduced = std::binary_search(r.begin(), r.end(), i);
    if (keepdims) o.push_back(reduced ? 1 : ishape[i]);
    else if (!reduced) o.push_back(ishape[i]);
  }
  return {o};
}

std::vector<int> SumPrec(const OpAttrs& a, const std::vector<Shape>& shapes, const std::vector<int>& ip) {
  InPrecCheck(a, ip);
  const int64_t suml = shape_size(shapes.at(0)) / shape_size(shapes.at(1));
  return {ip.at(0) + GetReduceSumBit(suml)};
}

std::vector<Shape> FlattenShape(const OpAttrs&, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 1U) << "Input: [data]";
  uint32_t target = 1;
  for (size_t i = 1; i < in[0].size(); ++i) target *= static_cast<uint32_t>(in[0][i]);
  return {Shape{in[0][0], static_cast<int64_t>(target)}};
}

std::vector<Shape> ReshapeShape(const OpAttrs& a, const std::vector<Shape>& in) {
  const Shape& target = a.t("shape");
  CVM_VERIFY(target.size() > 0U);
  CVM_VERIFY(in.size() == 1U) << "Input: [data]";
  const Shape& d = in[0];
  Shape o;
  size_t src = 0;
  int infer_idx = -1;
  for (size_t i = 0; i < target.size(); ++i) {
    const int64_t sv = target[i];
    if (sv > 0) {
      o.push_back(sv);
      ++src;
    } else if (sv == 0) {
      CVM_VERIFY(src < d.size());
      o.push_back(d[src++]);
    } else if (sv == -1) {
      CVM_VERIFY(infer_idx < 0) << "One and only one dim can be inferred";
      infer_idx = static_cast<int>(i);
      o.push_back(1);
      ++src;
    } else if (sv == -2) {
      while (src < d.size()) o.push_back(d[src++]);
    } else if (sv == -3) {
      CVM_VERIFY(src + 1 < d.size());
      const int64_t d1 = d[src++], d2 = d[src++];
      o.push_back(d1 * d2);
    } else if (sv == -4) {
      CVM_VERIFY(i + 2 < target.size());
      CVM_VERIFY(src < d.size());
      const int64_t d0 = d[src++];
      int d1 = static_cast<int>(target[++i]), d2 = static_cast<int>(target[++i]);
      CVM_VERIFY(d1 != -1 || d2 != -1) << "Split dims cannot both be -1.";
      if (d1 == -1) d1 = static_cast<int>(d0 / d2);
      if (d2 == -1) d2 = static_cast<int>(d0 / d1);
      CVM_VERIFY(d1 * d2 == static_cast<int>(d0)) << "Split dims " << d1 << ", " << d2 << " do not divide original dim " << d0;
      o.push_back(d1);
      o.push_back(d2);
    }
  }
  if (infer_idx >= 0) {
    // infer_idx counts target entries; the reference writes oshape[infer_idx]
    CVM_VERIFY(static_cast<size_t>(infer_idx) < o.size());
    int new_size = 1;
    for (int64_t x : o) new_size *= static_cast<int>(x);
    CVM_CHECK(new_size != 0);
    o[infer_idx] = shape_size(d) / new_size;
  }
  CVM_VERIFY(shape_size(o) == shape_size(d)) << "Target shape size is different to source. Target: " << shape_str(o)
                                             << " Source: " << shape_str(d);
  return {o};
}

std::vector<Shape> ExpandDimsShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 1U);
  const Shape& d = in[0];
  const int ndim = static_cast<int>(d.size());
  VerifyAttrRange(a.i("axis"), "expand_dims.axis", -ndim - 1, ndim);
  VerifyAttrRange(a.i("num_newaxis"), "expand_dims.num_newaxis");
  const int axis = static_cast<int>(a.i("axis") < 0 ? ndim + a.i("axis") + 1 : a.i("axis"));
  Shape o(d.begin(), d.begin() + axis);
  for (int64_t i = 0; i < a.i("num_newaxis"); ++i) o.push_back(1);
  o.insert(o.end(), d.begin() + axis, d.end());
  return {o};
}

std::vector<Shape> SqueezeShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 1U);
  const Shape& s = in[0];
  const int ndim = static_cast<int>(s.size());
  const Shape& axis = a.t("axis");
  Shape o;
  if (axis.empty()) {
    for (int64_t v : s)
      if (v != 1) o.push_back(v);
  } else {
    std::set<int64_t> sel;
    for (int64_t ax : axis) {
      VerifyAttrRange(ax, "squeeze.axis", -ndim, ndim - 1);
      sel.insert(ax < 0 ? ax + ndim : ax);
    }
    for (int i = 0; i < ndim; ++i) {
      if (!sel.count(i)) o.push_back(s[i]);
      else CVM_VERIFY(s[i] == 1) << "The squeezed axis must have shape 1! Want to squeeze " << i << ", which has shape" << s[i];
    }
  }
  if (o.empty()) o.push_back(1);
  CVM_VERIFY(shape_size(o) == shape_size(s));
  return {o};
}

std::vector<Shape> ConcatShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(!in.empty());
  const int ndim = static_cast<int>(in[0].size());
  VerifyAttrRange(a.i("axis"), "concatenate.axis", -ndim, ndim - 1);
  const int axis = static_cast<int>(a.i("axis") >= 0 ? a.i("axis") : ndim + a.i("axis"));
  for (const Shape& s : in) CVM_VERIFY(static_cast<int>(s.size()) == ndim);
  Shape d = in[0];
  int64_t size = 0;
  for (const Shape& s : in) {
    size += s[axis];
    for (int i = 0; i < ndim; ++i)
      if (i != axis) CVM_VERIFY(s[i] == d[i]) << "concatenate inputs differ outside the axis";
  }
  d[axis] = size;
  return {d};
}

std::vector<Shape> TransposeShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 1U);
  const Shape& s = in[0];
  const int ndim = static_cast<int>(s.size());
  Shape axes = a.t("axes");
  Shape o(ndim);
  if (axes.empty()) {
    for (int i = 0; i < ndim; ++i) o[i] = s[ndim - 1 - i];
  } else {
    CVM_VERIFY(static_cast<int>(axes.size()) == ndim);
    for (int i = 0; i < ndim; ++i) {
      int64_t ax = axes[i];
      VerifyAttrRange(ax, "transpose.axis", -ndim, ndim - 1);
      if (ax < 0) {
        ax += ndim;
        axes[i] = ax;
      }
      for (int j = 0; j < ndim; ++j)
        if (i != j) CVM_VERIFY(ax != axes[j]) << "repeated axis in transpose";
      o[i] = s[ax];
    }
  }
  return {o};
}

std::vector<Shape> StridedSliceShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 1U);
  const Shape& d = in[0];
  const size_t n = d.size();
  Shape b = a.t("begin"), e = a.t("end"), st = a.t("stride");
  // the kernel indexes these per axis of the data (src/runtime/cpu/ops/ops.cc:806-825)
  CVM_VERIFY(b.size() <= n && e.size() <= n && st.size() <= n);
  for (size_t i = b.size(); i < n; ++i) b.push_back(0);
  for (size_t i = e.size(); i < n; ++i) e.push_back(d[i]);
  for (size_t i = st.size(); i < n; ++i) st.push_back(1);
  Shape o = d;
  for (size_t i = 0; i < n; ++i) {
    CVM_VERIFY(st[i] != 0);
    const int64_t lo = st[i] < 0 ? -1 : 0, hi = st[i] < 0 ? d[i] - 1 : d[i];
    int64_t bb = b[i] < 0 ? d[i] + b[i] : b[i];
    int64_t ee = e[i] < 0 ? d[i] + e[i] : e[i];
    bb = std::min(std::max(bb, lo), hi);
    ee = std::min(std::max(ee, lo), hi);
    const int interval = static_cast<int>(std::llabs(ee - bb));
    const int slice = static_cast<int>((interval + std::llabs(st[i]) - 1) / std::llabs(st[i]));
    CVM_VERIFY(st[i] < 0 ? (ee < bb) : (bb < ee)) << ": Input [Begin=" << b[i] << ", End=" << e[i] << "] is invalid for axis=" << i;
    o[i] = slice;
  }
  return {o};
}

std::vector<Shape> TakeShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 2U);
  const Shape &d = in[0], &idx = in[1];
  const int ndim = static_cast<int>(d.size());
  Shape o;
  if (!a.has("axis")) {
    o = idx;
  } else {
    int64_t axis = a.i("axis");
    VerifyAttrRange(axis, "take.axis", -ndim, ndim - 1);
    if (axis < 0) axis += ndim;
    for (int i = 0; i < ndim; ++i) {
      if (i == axis) o.insert(o.end(), idx.begin(), idx.end());
      else o.push_back(d[i]);
    }
  }
  return {o};
}

std::vector<Shape> LutShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 2U);
  CVM_VERIFY(shape_size(in[1]) == a.i("in_dim"));
  return {in[0]};
}

std::vector<Shape> SliceLikeShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 2U);
  const Shape &src = in[0], &tgt = in[1];
  const Shape& axis = a.t("axis");
  CVM_VERIFY(src.size() == tgt.size() || !axis.empty())
      << "input X and shape_like must be of the same shape if no axis is given";
  Shape end = src;
  if (axis.empty()) {
    for (size_t i = 0; i < src.size(); ++i)
      if (i < tgt.size()) {
        end[i] = tgt[i];
        CVM_VERIFY(end[i] <= src[i]) << "End index of axis " << i << " exceeds input shape: " << end[i] << " vs " << src[i];
      }
  } else {
    for (int64_t ax : axis) {
      if (ax < 0) ax += static_cast<int64_t>(src.size());
      VerifyAttrRange(ax, "slice_like.axis", 0, static_cast<int64_t>(std::min(tgt.size(), src.size())) - 1);
      end[ax] = tgt[ax];
      CVM_VERIFY(end[ax] <= src[ax]) << "End index of axis " << ax << " exceeds input shape: " << end[ax] << " vs " << src[ax];
    }
  }
  return {end};
}

std::vector<Shape> RepeatShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 1U);
  const Shape& s = in[0];
  const int ndim = static_cast<int>(s.size());
  CVM_VERIFY(a.i("repeats") > 0) << "operator " << a.node_name << " repeats:" << a.i("repeats") << " must greater than 0";
  VerifyAttrRange(a.i("axis"), "repeat.axis", -ndim, ndim - 1);
  const int pivot = static_cast<int>(a.i("axis") < 0 ? ndim + a.i("axis") : a.i("axis"));
  Shape o = s;
  o[pivot] *= a.i("repeats");
  return {o};
}

std::vector<Shape> TileShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 1U);
  const Shape& s = in[0];
  const Shape& reps = a.t("reps");
  const size_t sdim = s.size(), rdim = reps.size();
  CVM_VERIFY(rdim > 0) << "repetition array is not defined. data.ndim = " << sdim;
  for (int64_t r : reps) VerifyAttrRange(r, "tile.reps", 1);
  const size_t odim = std::max(sdim, rdim);
  Shape o(odim);
  for (size_t i = 0; i < odim; ++i) {
    const int64_t sv = i < sdim ? s[sdim - 1 - i] : 1;
    const int64_t rv = i < rdim ? reps[rdim - 1 - i] : 1;
    o[odim - 1 - i] = sv * rv;
  }
  return {o};
}

std::vector<Shape> UpsamplingShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 1U);
  CVM_VERIFY(in[0].size() == 4U) << "dimension should be 4D, Got: " << shape_str(in[0]);
  CVM_VERIFY(a.s("method") == "NEAREST_NEIGHBOR") << "only accept method = NEAREST_NEIGHBOR ";
  VerifyAttrRange(a.i("scale"), "UpSampling.scale", 1);
  CVM_VERIFY(a.s("layout") == "NCHW") << "UpSampling only supported NCHW layout vs. " << a.s("layout");
  Shape o = in[0];
  o[2] *= a.i("scale");
  o[3] *= a.i("scale");
  return {o};
}

std::vector<Shape> WhereShape(const OpAttrs&, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 3U);
  CVM_VERIFY(in[1] == in[2]) << "x and y must have the same shape: " << shape_str(in[1]) << " vs " << shape_str(in[2]);
  if (in[0] != in[1]) {
    CVM_VERIFY(in[0].size() == 1U) << "Shape of condition " << shape_str(in[0]) << " must be either equal to x or has dimension of 1.";
    CVM_VERIFY(in[0][0] == in[1][0]) << "If dim of condition is 1, it must be the same as the first dimension of input shape.";
  }
  return {in[1]};
}

std::vector<Shape> GetValidShape(const OpAttrs&, const std::vector<Shape>& in) {
  CVM_CHECK(in.size() == 1U);
  const Shape& s = in[0];
  CVM_VERIFY(s.size() == 3U);
  CVM_VERIFY(s[2] < 32 && s[2] >= 2);
  return {Shape{s[0]}, s};
}

std::vector<int> GetValidPrec(const OpAttrs& a, const std::vector<Shape>& shapes, const std::vector<int>& ip) {
  InPrecCheck(a, ip);
  const Shape& s = shapes.at(0);
  return {GetNumberPrecision(shape_size(s) / s[0]), ip.at(0)};
}

std::vector<Shape> NmsShape(const OpAttrs& a, const std::vector<Shape>& in) {
  CVM_VERIFY(in.size() == 2U) << "Inputs: [data, valid_count]";
  const Shape &d = in[0], &v = in[1];
  CVM_VERIFY(d.size() == 3U) << "Input data should be 3-D.";
  CVM_VERIFY(v.size() == 1U) << "Input valid count should be 1-D.";
  CVM_VERIFY(d[2] == 6) << "Data input should have shape (batch_size, num_anchors, 6).";
  CVM_VERIFY(d[0] == v[0]) << "batch_size mismatch.";
  CVM_VERIFY(a.i("coord_start") == 2);
  CVM_VERIFY(a.i("score_index") == 1);
  CVM_VERIFY(a.i("id_index") == 0);
  CVM_VERIFY(a.i("iou_threshold") > 0);
  CVM_VERIFY(a.b("return_indices") == false) << "NonMaximumSuppressionParam only supported return_indices false";
  CVM_VERIFY(a.b("invalid_to_bottom") == true) << "NonMaximumSuppressionParam only supported invalid_to_bottom true";
  return {d};
}

std::vector<OpSchema> BuildTable() {
  std::vector<OpSchema> t;
  auto unary = [&](const char* name, decltype(OpSchema::infer_prec) prec) {
    t.push_back({name, {}, 1, 1, SameShape1, prec});
  };
  t.push_back({"conv2d",
               {{"channels", F_INT, true, ""}, {"kernel_size", F_TUPLE, true, ""}, {"strides", F_TUPLE, false, "(1, 1)"},
                {"padding", F_TUPLE, false, "(0, 0)"}, {"dilation", F_TUPLE, false, "(1, 1)"}, {"groups", F_INT, false, "1"},
                {"layout", F_STR, false, "NCHW"}, {"out_layout", F_STR, false, "__undef__"},
                {"kernel_layout", F_STR, false, "OIHW"}, {"out_dtype", F_STR, false, "same"},
                {"use_bias", F_BOOL, false, "True"}},
               -2, 1, ConvShape, ConvPrec});
  t.push_back({"dense", {{"units", F_INT, true, ""}, {"use_bias", F_BOOL, false, "True"}}, -2, 1, DenseShape, DensePrec});
  unary("relu", SamePrec);
  unary("abs", SamePrec);
  unary("negative", SamePrec);
  unary("cvm_precision", [](const OpAttrs& a, const std::vector<Shape>&, const std::vector<int>& ip) {
    InPrecCheck(a, ip);
    return std::vector<int>{6};
  });
  t.push_back({"max_pool2d",
               {{"pool_size", F_TUPLE, true, ""}, {"strides", F_TUPLE, false, "(1, 1)"}, {"padding", F_TUPLE, false, "(0, 0)"},
                {"layout", F_STR, false, "NCHW"}, {"ceil_mode", F_BOOL, false, "False"}},
               1, 1, PoolShape, SamePrec});
  t.push_back({"elemwise_add", {}, 2, 1, SameShape2, PlusPrec});
  t.push_back({"elemwise_sub", {}, 2, 1, SameShape2, PlusPrec});
  t.push_back({"clip", {{"a_min", F_INT, true, ""}, {"a_max", F_INT, true, ""}}, 1, 1, SameShape1,
               [](const OpAttrs& a, const std::vector<Shape>&, const std::vector<int>& ip) {
                 InPrecCheck(a, ip);
                 const int64_t r = (static_cast<int64_t>(1) << 31) - 1;
                 VerifyAttrRange(a.i("a_max"), "clip.a_max", -r, r);
                 VerifyAttrRange(a.i("a_min"), "clip.a_min", -r, r);
                 CVM_VERIFY(a.i("a_min") < a.i("a_max")) << "clip a_min must less than a_max";
                 const int64_t range = std::max(std::llabs(a.i("a_max")), std::llabs(a.i("a_min")));
                 return std::vector<int>{GetNumberPrecision(range)};
               }});
  t.push_back({"cvm_clip", {{"precision", F_INT, true, ""}, {"is_sign", F_BOOL, false, "True"}}, 1, 1, SameShape1,
               [](const OpAttrs& a, const std::vector<Shape>&, const std::vector<int>& ip) {
                 InPrecCheck(a, ip);
                 VerifyAttrRange(a.i("precision"), "cvm_clip.precision", 1, 32);
                 return std::vector<int>{static_cast<int>(a.i("precision"))};
               }});
  t.push_back({"cvm_left_shift",
               {{"precision", F_INT, true, ""}, {"is_sign", F_BOOL, false, "True"}, {"shift_bit", F_INT, true, ""}},
               1, 1, SameShape1,
               [](const OpAttrs& a, const std::vector<Shape>&, const std::vector<int>& ip) {
                 InPrecCheck(a, ip);
                 VerifyAttrRange(a.i("precision"), "cvm_left_shift.precision", 1, 32);
                 VerifyAttrRange(a.i("shift_bit"), "cvm_left_shift.shift_bit", 1, 32);
                 if (ip.at(0) + a.i("shift_bit") > 32)
                   CVM_FATAL() << "operator cvm_left_shift name=" << a.node_name << ": infer precision failed";
                 return std::vector<int>{static_cast<int>(a.i("precision"))};
               }});
  t.push_back({"cvm_right_shift",
               {{"precision", F_INT, true, ""}, {"is_sign", F_BOOL, false, "True"}, {"shift_bit", F_INT, true, ""}},
               1, 1, SameShape1,
               [](const OpAttrs& a, const std::vector<Shape>&, const std::vector<int>& ip) {
                 InPrecCheck(a, ip);
                 VerifyAttrRange(a.i("precision"), "cvm_right_shift.precision", 1, 32);
                 VerifyAttrRange(a.i("shift_bit"), "cvm_right_shift.shift_bit", 1, 32);
                 return std::vector<int>{static_cast<int>(a.i("precision"))};
               }});
  t.push_back({"broadcast_add", {}, 2, 1, BroadcastShape, PlusPrec});
  t.push_back({"broadcast_sub", {}, 2, 1, BroadcastShape, PlusPrec});
  t.push_back({"broadcast_mul", {}, 2, 1, BroadcastShape, MulPrec});
  t.push_back({"broadcast_max", {}, 2, 1, BroadcastShape, MaxInPrec});
  t.push_back({"broadcast_div", {}, 2, 1, BroadcastShape, SamePrec});
  t.push_back({"broadcast_greater", {}, 2, 1, BroadcastShape, SamePrec});
  const std::vector<Field> reduce_fields = {{"axis", F_TUPLE, false, "()"}, {"keepdims", F_BOOL, false, "False"},
                                            {"exclude", F_BOOL, false, "False"}, {"dtype", F_STR, false, "int32"}};
  t.push_back({"sum", reduce_fields, 1, 1, ReduceShape, SumPrec});
  t.push_back({"max", reduce_fields, 1, 1, ReduceShape, SamePrec});
  t.push_back({"flatten", {}, 1, 1, FlattenShape, SamePrec});
  t.push_back({"reshape", {{"shape", F_TUPLE, true, ""}}, 1, 1, ReshapeShape, SamePrec});
  t.push_back({"expand_dims", {{"axis", F_INT, true, ""}, {"num_newaxis", F_INT, false, "1"}}, 1, 1, ExpandDimsShape, SamePrec});
  t.push_back({"squeeze", {{"axis", F_TUPLE, false, "()"}}, 1, 1, SqueezeShape, SamePrec});
  t.push_back({"concatenate", {{"axis", F_INT, false, "1"}}, -1, 1, ConcatShape, MaxInPrec});
  t.push_back({"transpose", {{"axes", F_TUPLE, false, "()"}}, 1, 1, TransposeShape, SamePrec});
  t.push_back({"strided_slice",
               {{"begin", F_TUPLE, false, "(0,)"}, {"end", F_TUPLE, false, "(1,)"}, {"stride", F_TUPLE, false, "()"}},
               1, 1, StridedSliceShape, SamePrec});
  t.push_back({"take", {{"axis", F_OPT_INT, false, "None"}}, 2, 1, TakeShape, SamePrec});
  t.push_back({"cvm_lut", {{"in_dim", F_INT, true, ""}}, 2, 1, LutShape,
               [](const OpAttrs& a, const std::vector<Shape>&, const std::vector<int>& ip) {
                 InPrecCheck(a, ip);
                 return std::vector<int>{ip.at(1)};
               }});
  t.push_back({"slice_like", {{"axis", F_TUPLE, false, "()"}}, 2, 1, SliceLikeShape, SamePrec});
  t.push_back({"repeat", {{"repeats", F_INT, true, ""}, {"axis", F_INT, false, "0"}}, 1, 1, RepeatShape, SamePrec});
  t.push_back({"tile", {{"reps", F_TUPLE, false, "(0,)"}}, 1, 1, TileShape, SamePrec});
  t.push_back({"upsampling",
               {{"scale", F_INT, true, ""}, {"layout", F_STR, false, "NCHW"}, {"method", F_STR, false, "NEAREST_NEIGHBOR"}},
               1, 1, UpsamplingShape, SamePrec});
  t.push_back({"where", {}, 3, 1, WhereShape, SamePrec});
  t.push_back({"get_valid_counts", {{"score_threshold", F_INT, false, "0"}}, 1, 2, GetValidShape, GetValidPrec});
  t.push_back({"non_max_suppression",
               {{"return_indices", F_BOOL, false, "False"}, {"iou_threshold", F_INT, false, "50"},
                {"force_suppress", F_BOOL, false, "False"}, {"top_k", F_INT, false, "-1"}, {"id_index", F_INT, false, "0"},
                {"coord_start", F_INT, false, "2"}, {"score_index", F_INT, false, "1"},
                {"max_output_size", F_INT, false, "-1"}, {"invalid_to_bottom", F_BOOL, false, "True"}},
               2, 1, NmsShape, SamePrec});
  return t;
}

const std::vector<OpSchema>& Table() {
  static const std::vector<OpSchema> table = BuildTable();
  return table;
}

}  // namespace

const OpSchema* FindOp(const std::string& name) {
  for (const auto& s : Table())
    if (s.name == name) return &s;
  return nullptr;
}

std::vector<std::string> ListOps() {
  std::vector<std::string> names;
  for (const auto& s : Table()) names.push_back(s.name);
  return names;
}

}  // namespace cvmrt
