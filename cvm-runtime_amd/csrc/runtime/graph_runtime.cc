#include "graph_runtime.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <atomic>
#include <mutex>
#include <unordered_set>

#include "../../../include/cvm_hip_ops.h"

namespace cvmrt {

namespace {

// status of a C-ABI call -> the reference's two exception classes
// (src/runtime/cuda/ops/ops_cuda.cc:33-43: codes 10..19 VERIFY, >= 20 CHECK)
void HipCheck(int rc, const char* what) {
  if (rc == CVMHIP_OK) return;
  if (rc < CVMHIP_ERR_RUNTIME) CVM_VERIFY(false) << what << ": " << cvmhip_last_error();
  CVM_CHECK(false) << what << ": " << cvmhip_last_error();
}

size_t AlignUp(size_t v, size_t a) { return (v + a - 1) / a * a; }

// ---- JSON field readers with the reference loader's strictness
const std::string& AsString(const Json& v, const char* what) {
  CVM_CHECK(v.is_string()) << "json: " << what << " must be a string";
  return v.s;
}

int64_t AsInt(const Json& v, const char* what) {
  CVM_CHECK(v.is_int()) << "json: " << what << " must be an integer";
  return v.i;
}

template <typename T>
std::vector<T> AsIntList(const Json& v, const char* what) {
  CVM_CHECK(v.is_array()) << "json: " << what << " must be an array";
  std::vector<T> out;
  for (const Json& e : v.arr) out.push_back(static_cast<T>(AsInt(e, what)));
  return out;
}

// graph attribute of the form ["list_int", [...]]
const Json& TypedAttr(const Json& v, const char* type, const char* key) {
  CVM_CHECK(v.is_array()) << "json: graph attribute " << key << " must be an array";
  CVM_VERIFY(v.arr.size() >= 1U);
  CVM_VERIFY(AsString(v.arr[0], key) == type) << "graph attribute " << key << " must be tagged " << type;
  CVM_VERIFY(v.arr.size() >= 2U);
  CVM_VERIFY(v.arr.size() == 2U);
  return v.arr[1];
}

NodeEntry ReadEntry(const Json& v) {
  CVM_CHECK(v.is_array()) << "json: node entry must be an array";
  CVM_VERIFY(v.arr.size() >= 2U && v.arr.size() <= 3U) << "invalid json format";
  NodeEntry e;
  e.node_id = static_cast<uint32_t>(AsInt(v.arr[0], "entry"));
  e.index = static_cast<uint32_t>(AsInt(v.arr[1], "entry"));
  e.version = v.arr.size() == 3 ? static_cast<uint32_t>(AsInt(v.arr[2], "entry")) : 0;
  return e;
}

// "conv2d_3" -> "conv2d": a trailing _<digits> is dropped (graph_runtime.h:262-270)
std::string StripOpSuffix(const std::string& name) {
  std::string ret = name;
  for (int i = static_cast<int>(name.size()) - 1; i >= 0; --i) {
    if (name[i] >= '0' && name[i] <= '9') continue;
    if (name[i] == '_') ret = name.substr(0, i);
    break;
  }
  return ret;
}

}  // namespace

OpRegistry& OpRegistry::Global() {
  static OpRegistry r;
  return r;
}

std::vector<std::string> OpRegistry::ListNames() const {
  std::vector<std::string> n;
  for (const auto& kv : table_) n.push_back(kv.first);
  return n;
}

// ---------------------------------------------------------------- loading
void HipGraphRuntime::Load(const Json& doc) {
  CVM_CHECK(doc.is_object()) << "json: graph must be an object";
  int mask = 0;
  for (const auto& kv : doc.obj) {
    const std::string& key = kv.first;
    const Json& v = kv.second;
    if (key == "nodes") {
      CVM_CHECK(v.is_array()) << "json: nodes must be an array";
      for (const Json& jn : v.arr) {
        CVM_CHECK(jn.is_object()) << "json: node must be an object";
        Node n;
        int nmask = 0;
        for (const auto& f : jn.obj) {
          if (f.first == "op") {
            n.op_type = AsString(f.second, "op");
            CVM_VERIFY(n.op_type == "cvm_op" || n.op_type == "null")
                << "CVM executor only supported cvm_op or parameter vs. " << n.op_type;
            nmask |= 1;
          } else if (f.first == "name") {
            n.name = AsString(f.second, "name");
            nmask |= 2;
          } else if (f.first == "inputs") {
            CVM_CHECK(f.second.is_array()) << "json: inputs must be an array";
            for (const Json& e : f.second.arr) n.inputs.push_back(ReadEntry(e));
            nmask |= 4;
          } else if (f.first == "attrs") {
            CVM_CHECK(f.second.is_object()) << "json: node attrs must be an object";
            int amask = 0;
            for (const auto& a : f.second.obj) {
              const std::string& value = AsString(a.second, "node attribute");
              if (a.first == "func_name") {
                n.func_name = value;
                amask |= 1;
              } else if (a.first == "num_inputs" || a.first == "num_outputs" || a.first == "op_attrs" ||
                         a.first == "flatten_data") {
              } else {
                CVM_FATAL() << "node attributes do not support key " << a.first;
              }
            }
            CVM_VERIFY(amask == 1) << "invalid format";
          } else if (f.first == "precision") {
            AsInt(f.second, "precision");
          } else {
            CVM_FATAL() << "node do not support key " << f.first;
          }
        }
        CVM_VERIFY(nmask == 7) << "invalid format";
        nodes_.push_back(std::move(n));
      }
      mask |= 1;
    } else if (key == "arg_nodes") {
      input_nodes_ = AsIntList<uint32_t>(v, "arg_nodes");
    } else if (key == "node_row_ptr") {
      node_row_ptr_ = AsIntList<uint32_t>(v, "node_row_ptr");
    } else if (key == "heads") {
      CVM_CHECK(v.is_array()) << "json: heads must be an array";
      for (const Json& e : v.arr) outputs_.push_back(ReadEntry(e));
      mask |= 8;
    } else if (key == "attrs") {
      CVM_CHECK(v.is_object()) << "json: attrs must be an object";
      int amask = 0;
      for (const auto& a : v.obj) {
        if (a.first == "dltype") {
          const Json& l = TypedAttr(a.second, "list_str", "dltype");
          CVM_CHECK(l.is_array());
          for (const Json& e : l.arr) dltype_.push_back(AsString(e, "dltype"));
        } else if (a.first == "storage_id") {
          storage_id_ = AsIntList<int>(TypedAttr(a.second, "list_int", "storage_id"), "storage_id");
          amask |= 2;
        } else if (a.first == "shape") {
          const Json& l = TypedAttr(a.second, "list_shape", "shape");
          CVM_CHECK(l.is_array());
          for (const Json& e : l.arr) shape_.push_back(AsIntList<int64_t>(e, "shape"));
          amask |= 4;
        } else if (a.first == "device_index") {
          device_index_ = AsIntList<int>(TypedAttr(a.second, "list_int", "device_index"), "device_index");
        } else if (a.first == "precision") {
          precision_ = AsIntList<int>(TypedAttr(a.second, "list_int", "precision"), "precision");
        } else if (a.first == "op_attrs") {
          const Json& l = TypedAttr(a.second, "list_str", "op_attrs");
          CVM_CHECK(l.is_array());
          for (const Json& e : l.arr) op_attrs_.push_back(AsString(e, "op_attrs"));
          amask |= 8;
        } else if (a.first == "dtype") {
          CVM_CHECK(a.second.is_array() && a.second.arr.size() == 2U && a.second.arr[0].is_string());
          if (a.second.arr[0].s != "list_int" && a.second.arr[0].s != "list_str")
            CVM_FATAL() << "cannot skip graph attr " << a.first;
        } else {
          CVM_FATAL() << "graph attribute " << a.first << " not supported";
        }
      }
      CVM_VERIFY(amask == (2 | 4 | 8)) << "invalid format";
      mask |= 16;
    } else if (key == "version") {
      version_ = AsString(v, "version");
    } else if (key == "postprocess") {
      postprocess_ = AsString(v, "postprocess");
    } else {
      CVM_FATAL() << "key " << key << " in json is not supported";
    }
  }
  CVM_VERIFY(mask == (1 | 8 | 16)) << "invalid format";
}

// graph_runtime.cc:114-261
void HipGraphRuntime::PrepareGraph() {
  std::unordered_set<std::string> names;
  for (uint32_t nid : input_nodes_) {
    CVM_CHECK(nid < nodes_.size()) << "arg_nodes entry " << nid << " out of range";
    if (!names.insert(nodes_[nid].name).second) CVM_FATAL() << "node name " << nodes_[nid].name << " duplicated in graph";
  }
  CVM_VERIFY(nodes_.size() == op_attrs_.size())
      << "graph attribute op_attrs size: " << op_attrs_.size() << ", Expected " << nodes_.size();
  for (size_t i = 0; i < nodes_.size(); ++i) {
    Node& n = nodes_[i];
    if (n.is_variable()) continue;
    n.func_name = StripOpSuffix(n.func_name);
    n.schema = FindOp(n.func_name);
    if (n.schema == nullptr) CVM_FATAL() << "Operator " << n.func_name << " is not registered";
    Json dict = Json::Parse(op_attrs_[i]);
    CVM_CHECK(dict.is_object()) << "op_attrs entry must be a json object";
    AttrDict ad;
    for (const auto& kv : dict.obj) ad.emplace_back(kv.first, AsString(kv.second, "operator attribute"));
    n.attrs = ParseAttrs(*n.schema, n.name, ad);
    n.num_inputs = static_cast<uint32_t>(NumInputs(*n.schema, n.attrs, n.inputs.size()));
    n.num_outputs = static_cast<uint32_t>(n.schema->num_outputs);
    CVM_VERIFY(n.num_inputs == n.inputs.size())
        << "operator " << n.func_name << " name=" << n.name << "'s inputs length invaild " << n.inputs.size()
        << " vs. " << n.num_inputs;
  }

  num_node_entries_ = 0;
  std::vector<uint32_t> row_ptr, input_nodes;
  for (uint32_t i = 0; i < nodes_.size(); ++i) {
    if (nodes_[i].is_variable()) input_nodes.push_back(i);
    row_ptr.push_back(num_node_entries_);
    num_node_entries_ += nodes_[i].num_outputs;
  }
  row_ptr.push_back(num_node_entries_);

  CVM_VERIFY(num_node_entries_ == storage_id_.size())
      << "graph attribute storage_id size: " << storage_id_.size() << ", Expected " << num_node_entries_;
  for (int sid : storage_id_) CVM_VERIFY(sid >= 0) << "storage id should not less than 0, but " << sid;

  CVM_VERIFY(num_node_entries_ == shape_.size())
      << "graph attribute shape size: " << shape_.size() << ", Expected " << num_node_entries_;
  for (const Shape& s : shape_) {
    uint64_t sx = 1;
    CVM_VERIFY(0 < s.size() && s.size() <= 6) << "shape ndim should between (0, 6], but " << s.size();
    for (int64_t x : s) {
      sx *= static_cast<uint64_t>(x);
      CVM_VERIFY(0 < x && x <= (1 << 24)) << "single dimension should between (0, " << (1 << 24) << "], but " << x;
      CVM_VERIFY(sx <= (1u << 30)) << "shape size shoule not greater than" << (1 << 30) << ", but " << sx;
    }
  }

  CVM_VERIFY(num_node_entries_ == precision_.size())
      << "graph attribute precision size: " << precision_.size() << ", Expected " << num_node_entries_;
  for (int p : precision_) CVM_VERIFY(p == -1 || (0 < p && p <= 32)) << "precision should be -1 or between (0, 32], but " << p;

  CVM_VERIFY(device_index_.empty()) << "attribute device_index must be set empty";

  if (version_ == "cvm_1.0.0") {
    CVM_VERIFY(num_node_entries_ == dltype_.size())
        << "graph attribute dltype size: " << dltype_.size() << ", Expected " << num_node_entries_;
    for (const std::string& t : dltype_) CVM_VERIFY(t == "int32") << "type " << t << " are not supported";
    CVM_VERIFY(node_row_ptr_.size() == row_ptr.size())
        << "node_row_ptr's size: " << node_row_ptr_.size() << ", Expected " << row_ptr.size();
    for (size_t i = 0; i < row_ptr.size(); ++i)
      CVM_VERIFY(row_ptr[i] == node_row_ptr_[i]) << "node_row_ptr is invalid at index " << i;
    CVM_VERIFY(input_nodes_.size() == input_nodes.size())
        << "arg_nodes' size: " << input_nodes_.size() << ", Expected " << input_nodes.size();
    for (size_t i = 0; i < input_nodes.size(); ++i)
      CVM_VERIFY(input_nodes[i] == input_nodes_[i]) << "arg_nodes is invalid at index " << i;
  } else if (version_ == "cvm_1.1.0") {
    node_row_ptr_ = row_ptr;
    input_nodes_ = input_nodes;
  } else {
    CVM_FATAL() << "graph version " << version_ << " not supported";
  }

  // every consumed or exported entry must exist (the reference indexes unchecked)
  for (const Node& n : nodes_)
    for (const NodeEntry& e : n.inputs)
      CVM_VERIFY(e.node_id < nodes_.size() && e.index < nodes_[e.node_id].num_outputs) << "node input out of range";
  for (const NodeEntry& e : outputs_)
    CVM_VERIFY(e.node_id < nodes_.size() && e.index < nodes_[e.node_id].num_outputs) << "graph head out of range";

  // storage may be shared between an operator's input and output only for a
  // fixed list of operators (graph_runtime.cc:150-177)
  static const std::unordered_set<std::string> reused = {
      "flatten", "relu", "expand_dims", "reshape", "squeeze", "abs", "cvm_precision", "elemwise_add",
      "elemwise_sub", "nagetive", "clip", "cvm_clip", "cvm_right_shift", "cvm_left_shift"};
  for (uint32_t nid = 0; nid < nodes_.size(); ++nid) {
    const Node& n = nodes_[nid];
    if (n.is_variable() || reused.count(n.func_name)) continue;
    for (uint32_t oi = 0; oi < n.num_outputs; ++oi) {
      const int out_sid = storage_id_[entry_id(nid, oi)];
      for (const NodeEntry& e : n.inputs)
        CVM_VERIFY(out_sid != storage_id_[entry_id(e)])
            << "operator " << n.func_name << " input: (" << e.node_id << ", " << e.index << ") output: (" << nid << ", "
            << oi << ") used same storage_id " << out_sid;
    }
  }

  for (uint32_t i = 0; i < nodes_.size(); ++i) {
    const uint32_t eid = entry_id(i, 0);
    for (const NodeEntry& e : nodes_[i].inputs)
      CVM_VERIFY(entry_id(e) < eid) << "the graph does not follow the topological order.";
  }
}

// infer_attr.cc:161-217
void HipGraphRuntime::SetupShape() {
  for (uint32_t nid = 0; nid < nodes_.size(); ++nid) {
    const Node& n = nodes_[nid];
    if (n.is_variable()) continue;
    std::vector<Shape> in;
    for (const NodeEntry& e : n.inputs) in.push_back(shape_[entry_id(e)]);
    std::vector<Shape> out = n.schema->infer_shape(n.attrs, in);
    CVM_CHECK(out.size() == n.num_outputs);
    for (uint32_t i = 0; i < n.num_outputs; ++i)
      CVM_VERIFY(out[i] == shape_[entry_id(nid, i)])
          << "Check output shape failed, expected to be " << shape_str(out[i]) << " but "
          << shape_str(shape_[entry_id(nid, i)]) << " " << n.func_name;
  }
}

// infer_attr.cc:31-91
void HipGraphRuntime::SetupPrecision() {
  for (uint32_t nid = 0; nid < nodes_.size(); ++nid) {
    const Node& n = nodes_[nid];
    if (n.is_variable()) {
      CVM_VERIFY(precision_[entry_id(nid, 0)] != -1) << "variable node " << n.name << "'s precision has not been set";
      continue;
    }
    std::vector<Shape> shapes;
    std::vector<int> ip;
    for (const NodeEntry& e : n.inputs) {
      ip.push_back(precision_[entry_id(e)]);
      shapes.push_back(shape_[entry_id(e)]);
    }
    for (uint32_t i = 0; i < n.num_outputs; ++i) shapes.push_back(shape_[entry_id(nid, i)]);
    std::vector<int> op = n.schema->infer_prec(n.attrs, shapes, ip);
    CVM_CHECK(op.size() == n.num_outputs);
    for (uint32_t i = 0; i < n.num_outputs; ++i) {
      precision_[entry_id(nid, i)] = op[i];
      CVM_VERIFY(0 < op[i] && op[i] <= 32) << " nid = " << nid << "i = " << i << " precison = " << op[i]
                                           << " name= " << n.name << " inode.attrs = " << op_attrs_[nid];
    }
  }
}

// graph_runtime.cc:503-531
void HipGraphRuntime::PlanStorage() {
  for (size_t i = 0; i < shape_.size(); ++i) {
    const size_t bytes = static_cast<size_t>(shape_size(shape_[i])) * 4;
    const uint32_t sid = static_cast<uint32_t>(storage_id_[i]);
    if (sid >= pool_.size()) pool_.resize(sid + 1);
    pool_[sid].bytes = std::max(pool_[sid].bytes, bytes);
  }
}

// graph_runtime.cc:565-574
int64_t HipGraphRuntime::GetStorageSize() const {
  int64_t ret = 0;
  const int64_t kMax = static_cast<int64_t>(1) << 32;
  for (const PoolEntry& p : pool_) {
    ret += (static_cast<int64_t>(p.bytes + 3) / 4) * 4;
    CVM_VERIFY(ret <= kMax) << "storage size exceed MAX_STORAGE " << kMax;
  }
  return ret;
}

void HipGraphRuntime::SetupStorage() {
  size_t off = 0;
  for (PoolEntry& p : pool_) {
    p.offset = off;
    off += AlignUp(std::max<size_t>(p.bytes, 4), 256);
  }
  slab_bytes_ = off;
  HipCheck(cvmhip_alloc(&slab_, slab_bytes_), "allocate storage pool");
  HipCheck(cvmhip_memset32(slab_, 0, slab_bytes_ / 4, stream_), "clear storage pool");
  entry_ptr_.resize(num_node_entries_);
  for (uint32_t i = 0; i < num_node_entries_; ++i)
    entry_ptr_[i] = reinterpret_cast<int32_t*>(static_cast<char*>(slab_) + pool_[storage_id_[i]].offset);
}

// graph_runtime.cc:612-698
void HipGraphRuntime::SetupOpExecs() {
  RegisterHipKernels();
  for (uint32_t nid = 0; nid < nodes_.size(); ++nid) {
    const Node& n = nodes_[nid];
    if (n.is_variable()) continue;
    const std::string fname = "cvm.runtime.hip." + n.func_name;
    const OpKernel* k = OpRegistry::Global().Get(fname);
    CVM_VERIFY(k != nullptr) << "function undefined " << fname;
    Exec ex;
    ex.nid = nid;
    ex.kernel = k;
    ex.call.op = n.func_name;
    ex.call.attrs = &nodes_[nid].attrs;
    ex.call.stream = stream_;
    for (const NodeEntry& e : n.inputs) {
      DevTensor t;
      const uint32_t eid = entry_id(e);
      t.data = entry_ptr_[eid];
      t.shape = shape_[eid];
      t.precision = precision_[eid];
      t.is_param = nodes_[e.node_id].is_variable() && !nodes_[e.node_id].is_data();
      ex.call.in.push_back(t);
    }
    for (uint32_t i = 0; i < n.num_outputs; ++i) {
      DevTensor t;
      const uint32_t eid = entry_id(nid, i);
      t.data = entry_ptr_[eid];
      t.shape = shape_[eid];
      t.precision = precision_[eid];
      ex.call.out.push_back(t);
    }
    if (k->workspace_bytes) workspace_bytes_ = std::max(workspace_bytes_, k->workspace_bytes(ex.call));
    execs_.push_back(std::move(ex));
  }
  workspace_bytes_ = AlignUp(std::max<size_t>(workspace_bytes_, 256), 256);
  HipCheck(cvmhip_alloc(&workspace_, workspace_bytes_), "allocate operator workspace");
  for (Exec& ex : execs_) {
    ex.call.workspace = workspace_;
    ex.call.workspace_bytes = workspace_bytes_;
  }
}

HipGraphRuntime::HipGraphRuntime(const std::string& graph_json, int device_id, bool with_device)
    : device_id_(device_id), with_device_(with_device) {
  ReadHooks();
  Load(Json::Parse(graph_json));
  PrepareGraph();
  SetupShape();
  SetupPrecision();
  PlanStorage();
  if (!with_device_) return;
  try {
    int count = 0;
    HipCheck(cvmhip_device_count(&count), "query devices");
    CVM_CHECK(device_id >= 0 && device_id < count) << "device id " << device_id << " out of range, " << count << " device(s) present";
    HipCheck(cvmhip_set_device(device_id), "select device");
    HipCheck(cvmhip_stream_create(&stream_), "create stream");
    SetupStorage();
    SetupOpExecs();
  } catch (...) {
    Release();
    throw;
  }
}

void HipGraphRuntime::ReadHooks() {
  auto env = [](const char* name) { const char* v = std::getenv(name); return std::string(v ? v : ""); };
  hooks_.fuse = env("CVM_HIP_FUSE") != "0";
  hooks_.fold_bias = env("CVM_HIP_FOLDBIAS") != "0";
  hooks_.graph = env("CVM_HIP_GRAPH") != "0";
  hooks_.seq = env("CVM_HIP_SEQ") != "0";
  hooks_.seq_forced = env("CVM_HIP_SEQ") == "1";
  hooks_.seq_chains = env("CVM_HIP_SEQ_CHAIN") != "0";
  hooks_.flat_dense = env("CVM_HIP_FLATDENSE") != "0";
  hooks_.dw_on_mfma = env("CVM_HIP_DW").rfind("v", 0) != 0;
  hooks_.pool_fuse = env("CVM_HIP_POOLFUSE") != "0";
  hooks_.head_pair = env("CVM_HIP_HEADPAIR") != "0";
  hooks_.head_group = env("CVM_HIP_HEADGROUP") != "0";
  hooks_.conv_group = env("CVM_HIP_CONVGROUP") != "0";
  const std::string kind = env("CVM_HIP_CONV"), cfg = env("CVM_HIP_WAVECFG"), tile = env("CVM_HIP_TILE");
  hooks_.conv_kernel = kind.rfind("l", 0) == 0 ? 1 : kind.rfind("w", 0) == 0 ? 2 : kind.rfind("b", 0) == 0 ? 3 : 0;
  if (!cfg.empty() && cfg[0] >= '0' && cfg[0] <= '9') hooks_.wave_cfg = std::atoi(cfg.c_str());
  if (tile.size() >= 3 && tile[1] == ',') {
    hooks_.tile_wm = tile[0] - '0';
    hooks_.tile_wn = tile[2] - '0';
  }
  const std::string spin = env("CVM_HIP_SEQ_SPIN");
  if (!spin.empty() && spin[0] >= '0' && spin[0] <= '9') hooks_.seq_spin = std::atoi(spin.c_str());
  // CVM_HIP_SEQCFG="index:config,index:config,...": the tile configuration of single layers of a sequence launch
  const std::string per_layer = env("CVM_HIP_SEQCFG");
  for (size_t at = 0; at < per_layer.size();) {
    size_t end = per_layer.find(',', at);
    if (end == std::string::npos) end = per_layer.size();
    const size_t colon = per_layer.find(':', at);
    if (colon != std::string::npos && colon < end) {
      const int index = std::atoi(per_layer.substr(at, colon - at).c_str()), config = std::atoi(per_layer.substr(colon + 1, end - colon - 1).c_str());
      if (index >= 0 && index < 64 && config >= 0 && config < 127) hooks_.seq_layer_cfg.emplace_back(index, config);
    }
    at = end + 1;
  }
}

void HipGraphRuntime::ApplyTuning() {
  HipCheck(cvmhip_set_conv_tuning(hooks_.conv_kernel, hooks_.wave_cfg, hooks_.tile_wm, hooks_.tile_wn), "conv tuning");
  HipCheck(cvmhip_set_seq_tuning(hooks_.seq_spin), "sequence tuning");
  HipCheck(cvmhip_set_seq_chains(hooks_.seq_chains ? 1 : 0), "sequence tuning");
  HipCheck(cvmhip_set_seq_layer_config(-1, -1), "sequence tuning");
  for (const auto& kv : hooks_.seq_layer_cfg) HipCheck(cvmhip_set_seq_layer_config(kv.first, kv.second), "sequence tuning");
}

void HipGraphRuntime::Release() {
  if (graph_exec_) { cvmhip_graph_destroy(graph_exec_); graph_exec_ = nullptr; }
  plan_.clear();
  if (seq_counted_) { CountSequenceModel(-1); seq_counted_ = false; }
  seqs_.clear();
  groups_.clear();
  if (seq_sync_) { cvmhip_free(seq_sync_); seq_sync_ = nullptr; }
  if (seq_error_host_) { cvmhip_host_free(seq_error_host_); seq_error_host_ = nullptr; }
  execs_.clear();  // releases per-node device state before the stream goes away
  if (i8_slab_) { cvmhip_free(i8_slab_); i8_slab_ = nullptr; }
  if (in_stage_dev_) { cvmhip_free(in_stage_dev_); in_stage_dev_ = nullptr; }
  if (in_stage_host_) { cvmhip_host_free(in_stage_host_); in_stage_host_ = nullptr; }
  if (out_stage_host_) { cvmhip_host_free(out_stage_host_); out_stage_host_ = nullptr; }
  out_host_.clear();
  if (stream_) cvmhip_stream_sync(stream_);
  own_storage_.clear();
  if (workspace_) cvmhip_free(workspace_);
  if (slab_) cvmhip_free(slab_);
  if (stream_) cvmhip_stream_destroy(stream_);
  workspace_ = slab_ = stream_ = nullptr;
}

HipGraphRuntime::~HipGraphRuntime() { Release(); }

// ---------------------------------------------------------------- parameters and inputs
int HipGraphRuntime::GetInputIndex(const std::string& name) const {
  for (size_t i = 0; i < input_nodes_.size(); ++i)
    if (nodes_[input_nodes_[i]].name == name) return static_cast<int>(i);
  CVM_FATAL() << "cannot find `" << name << "` among input";
  return -1;
}

// graph_runtime.cc:317-397: shape check, precision clamp (data) or check (parameters), copy to the device
void HipGraphRuntime::SetInput(uint32_t input_index, const int32_t* data32, const Shape& shape) {
  CVM_VERIFY(input_index < input_nodes_.size()) << "input index out of range [0, " << input_nodes_.size() << "), but " << input_index;
  const uint32_t nid = input_nodes_[input_index];
  const uint32_t eid = entry_id(nid, 0);
  const Shape& expected = shape_[eid];
  CVM_VERIFY(shape.size() == expected.size()) << "Loaded data shape ndim " << shape.size() << " not matched " << expected.size();
  for (size_t i = 0; i < shape.size(); ++i)
    CVM_VERIFY(shape[i] == expected[i]) << "Loaded data shape at index " << i << " with value " << shape[i] << ", Expected " << expected[i];
  const int64_t size = shape_size(shape);
  const int prec = precision_[eid];
  const int32_t range = static_cast<int32_t>((static_cast<uint32_t>(1) << (prec - 1)) - 1);
  std::vector<int32_t> staged(data32, data32 + size);
  if (nodes_[nid].is_data()) {
    for (int32_t& v : staged) v = v > range ? range : (v < -range ? -range : v);
  } else {
    for (int64_t i = 0; i < size; ++i)
      CVM_VERIFY(-range <= staged[i] && staged[i] <= range)
          << "parameter " << nodes_[nid].name << " at index " << i << " value:" << staged[i] << " exceed of precision " << prec;
  }
  HipCheck(cvmhip_copy_h2d(entry_ptr_[eid], staged.data(), static_cast<size_t>(size) * 4, stream_), "copy input to device");
  HipCheck(cvmhip_stream_sync(stream_), "copy input to device");  // `staged` dies here
}

// `data` given as int8 bytes: staged through pinned memory, widened and clamped on the device.
// Same result as SetData on the widened values; a quarter of the bytes cross the bus and the
// host does one memcpy.
void HipGraphRuntime::SetDataI8(const int8_t* host, const Shape& shape) {
  const int idx = GetInputIndex("data");
  const uint32_t nid = input_nodes_[idx];
  CVM_VERIFY(nodes_[nid].is_data()) << "set input must named `data`";
  const uint32_t eid = entry_id(nid, 0);
  const Shape& expected = shape_[eid];
  CVM_VERIFY(shape.size() == expected.size()) << "Loaded data shape ndim " << shape.size() << " not matched " << expected.size();
  for (size_t i = 0; i < shape.size(); ++i)
    CVM_VERIFY(shape[i] == expected[i]) << "Loaded data shape at index " << i << " with value " << shape[i] << ", Expected " << expected[i];
  const size_t size = static_cast<size_t>(shape_size(shape));
  const int prec = precision_[eid];
  const int32_t range = static_cast<int32_t>((static_cast<uint32_t>(1) << (prec - 1)) - 1);
  if (!in_stage_host_) {
    HipCheck(cvmhip_host_alloc(&in_stage_host_, size), "input staging buffer");
    HipCheck(cvmhip_alloc(&in_stage_dev_, size), "input staging buffer");
  }
  HipCheck(cvmhip_stream_sync(stream_), "copy input to device");  // the previous copy out of the staging buffer is done
  // The caller's bytes go through the pinned buffer in pieces: while the copy engine moves one piece to the device the
  // host already copies the next into the buffer, so of the two copies only the longer one is on the call's clock.
  const size_t piece = std::max<size_t>((size / 4 + 4095) & ~static_cast<size_t>(4095), 256 << 10);
  for (size_t at = 0; at < size; at += piece) {
    const size_t len = std::min(piece, size - at);
    std::memcpy(static_cast<char*>(in_stage_host_) + at, reinterpret_cast<const char*>(host) + at, len);
    HipCheck(cvmhip_copy_h2d(static_cast<char*>(in_stage_dev_) + at, static_cast<char*>(in_stage_host_) + at, len, stream_), "copy input to device");
  }
  HipCheck(cvmhip_widen_clamp_i8(in_stage_dev_, entry_ptr_[eid], static_cast<int64_t>(size), range, stream_), "widen input");
}

void HipGraphRuntime::SetData(const int32_t* host, const Shape& shape) {
  const int idx = GetInputIndex("data");
  CVM_VERIFY(nodes_[input_nodes_[idx]].is_data()) << "set input must named `data`";
  SetInput(static_cast<uint32_t>(idx), host, shape);
}

namespace {

// Little-endian reader over the parameter blob (src/runtime/param_dict.cc:14-38,
// include/cvm/runtime/ndarray.h:485-540).
class BlobReader {
 public:
  explicit BlobReader(const std::string& b) : b_(b), p_(0) {}
  template <typename T>
  bool Read(T* v) {
    if (p_ + sizeof(T) > b_.size()) return false;
    std::memcpy(v, b_.data() + p_, sizeof(T));
    p_ += sizeof(T);
    return true;
  }
  bool ReadBytes(void* dst, size_t n) {
    if (p_ + n > b_.size() || p_ + n < p_) return false;
    std::memcpy(dst, b_.data() + p_, n);
    p_ += n;
    return true;
  }
  size_t remaining() const { return b_.size() - p_; }

 private:
  const std::string& b_;
  size_t p_;
};

const uint64_t kListMagic = 0xF7E58D4F05049CB7ull;
const uint64_t kArrayMagic = 0xDD5E40F096B4A13Full;

}  // namespace

// graph_runtime.cc:476-501
void HipGraphRuntime::LoadParams(const std::string& blob) {
  BlobReader rd(blob);
  uint64_t header = 0, reserved = 0, count = 0;
  CVM_VERIFY(rd.Read(&header)) << "Invalid parameters file format";
  CVM_VERIFY(header == kListMagic) << "Invalid parameters file format";
  CVM_VERIFY(rd.Read(&reserved)) << "Invalid parameters file format";
  CVM_VERIFY(rd.Read(&count)) << "Invalid parameters file format";
  CVM_VERIFY(count <= rd.remaining() / 8) << "Invalid parameters file format";
  std::vector<std::string> names(count);
  for (uint64_t i = 0; i < count; ++i) {
    uint64_t len = 0;
    CVM_VERIFY(rd.Read(&len)) << "Invalid parameters file format";
    CVM_VERIFY(len <= rd.remaining()) << "Invalid parameters file format";
    names[i].resize(len);
    CVM_VERIFY(rd.ReadBytes(&names[i][0], len)) << "Invalid parameters file format";
  }
  uint64_t n_arrays = 0;
  rd.Read(&n_arrays);
  CVM_VERIFY(n_arrays == names.size()) << "Invalid parameters file format";

  std::vector<bool> set_flag(input_nodes_.size(), false);
  for (size_t i = 0; i < names.size(); ++i) {
    uint64_t magic = 0, rsv = 0;
    int32_t dev_type = 0, dev_id = 0, ndim = 0;
    uint8_t code = 0, bits = 0;
    uint16_t lanes = 0;
    CVM_CHECK(rd.Read(&magic)) << "Invalid DLTensor file format";
    CVM_CHECK(rd.Read(&rsv)) << "Invalid DLTensor file format";
    CVM_CHECK(magic == kArrayMagic) << "Invalid DLTensor file format";
    CVM_CHECK(rd.Read(&dev_type) && rd.Read(&dev_id) && rd.Read(&ndim)) << "Invalid DLTensor file format";
    CVM_CHECK(rd.Read(&code) && rd.Read(&bits) && rd.Read(&lanes)) << "Invalid DLTensor file format";
    CVM_CHECK(ndim >= 0 && static_cast<size_t>(ndim) <= rd.remaining() / 8) << "Invalid DLTensor file format";
    Shape shape(ndim);
    for (int d = 0; d < ndim; ++d) CVM_CHECK(rd.Read(&shape[d])) << "Invalid DLTensor file format";
    int64_t nbytes = 0;
    CVM_CHECK(rd.Read(&nbytes)) << "Invalid DLTensor file format";
    int64_t elems = 1;
    for (int64_t s : shape) {
      CVM_CHECK(s >= 0 && (s == 0 || elems <= (static_cast<int64_t>(1) << 40) / s)) << "Invalid DLTensor file format";
      elems *= s;
    }
    const int elem_bytes = (bits + 7) / 8;
    CVM_CHECK(nbytes == elems * elem_bytes) << "Invalid DLTensor file format";
    CVM_CHECK(nbytes >= 0 && static_cast<size_t>(nbytes) <= rd.remaining()) << "Invalid DLTensor file format";
    std::vector<char> raw(static_cast<size_t>(nbytes));
    CVM_CHECK(rd.ReadBytes(raw.data(), raw.size())) << "Invalid DLTensor file format";

    const int in_idx = GetInputIndex(names[i]);
    set_flag[in_idx] = true;
    CVM_VERIFY(code == 0 /* kDLInt */) << "cvm runtime only supported INT NDArray, but (" << int(code) << ")";
    CVM_VERIFY(dev_type == 1 /* kDLCPU */) << "cvm runtime only supported input with `cpu` device, but " << dev_type;
    // shape is compared before the dtype, as the reference does (graph_runtime.cc:335-357)
    const Shape& expected = shape_[entry_id(input_nodes_[in_idx], 0)];
    CVM_VERIFY(shape.size() == expected.size()) << "Loaded data shape ndim " << shape.size() << " not matched " << expected.size();
    for (size_t d = 0; d < shape.size(); ++d)
      CVM_VERIFY(shape[d] == expected[d]) << "Loaded data shape at index " << d << " with value " << shape[d] << ", Expected " << expected[d];
    CVM_VERIFY((bits == 32 || bits == 8) && lanes == 1)
        << "cvm runtime only supported INT8 or INT32 NDArray, but (" << int(code) << ", " << int(bits) << ", " << lanes << ")";
    std::vector<int32_t> wide(static_cast<size_t>(elems));
    if (bits == 8) {
      const int8_t* p = reinterpret_cast<const int8_t*>(raw.data());
      for (int64_t e = 0; e < elems; ++e) wide[e] = p[e];
    } else {
      std::memcpy(wide.data(), raw.data(), raw.size());
    }
    SetInput(static_cast<uint32_t>(in_idx), wide.data(), shape);
  }
  for (size_t i = 0; i < set_flag.size(); ++i) {
    const uint32_t nid = input_nodes_[i];
    CVM_VERIFY(set_flag[i] || nodes_[nid].is_data()) << "parameter nid=" << nid << " name=" << nodes_[nid].name << " has not been loaded";
  }
  ApplyTuning();   // the tables of sequence and grouped launches are built under this model's own kernel choice
  for (Exec& ex : execs_)
    if (ex.kernel->prepare) ex.kernel->prepare(ex.call);
  if (hooks_.fuse) BuildPlan();
  HipCheck(cvmhip_stream_sync(stream_), "prepare operators");
  params_loaded_ = true;
  if (use_seq_ && !hooks_.seq_forced) {
    // With another such model alive both forms would be timed as one launch per layer.  The model stays counted (so the
    // other one keeps to one launch per layer as well: a sequence launch next to ordinary launches of another model is the
    // slowest combination, 43.5 k against 53.7 k images/s for two ResNet-50 models) and makes the comparison at the first
    // run it finds itself alone.
    if (SeqNow()) CalibrateSequences();
    else seq_calibration_pending_ = true;
  }
}

// Layer-sequence launches pay for layers that are bound by latency and cost a little where layers are large:
// which way a model runs faster is measured once, when it is loaded (a few replays each way; timing does not
// depend on the values in the tensors, so whatever the storage holds will do), unless CVM_HIP_SEQ=1 forces them.
void HipGraphRuntime::CalibrateSequences() {
  float ms[2] = {0, 0};
  for (int with_seq = 0; with_seq < 2; ++with_seq) {
    use_seq_ = with_seq != 0;
    if (graph_exec_) { cvmhip_graph_destroy(graph_exec_); graph_exec_ = nullptr; }
    graph_state_ = 0;
    for (int i = 0; i < 3; ++i) Run();   // eager, capture, first replay
    SyncStream();
    if (with_seq && !use_seq_) {          // the launch could not run here: stay with one launch per layer
      ms[1] = 1e30f;
      break;
    }
    ms[with_seq] = TimeRuns(4);
    SyncStream();                         // also reads the launch's error word
    if (with_seq && !use_seq_) {
      ms[1] = 1e30f;
      break;
    }
  }
  use_seq_ = ms[1] < 0.98f * ms[0];   // a clear win only: within the noise of a few replays the plainer form stays
  if (!use_seq_) DropSequences();
  if (graph_exec_) { cvmhip_graph_destroy(graph_exec_); graph_exec_ = nullptr; }
  graph_state_ = 0;
}

// ---------------------------------------------------------------- execution
// A layer-sequence launch occupies every compute unit and waits, inside the kernel, for all of its workgroups:
// two of them in flight at once (two models on two streams) could each hold part of the chip and wait for the
// rest until their bounded waits run out.  So sequence launches are used only while ONE model that has them is
// alive in the process; with two or more, every model runs one launch per layer, which is also the faster form
// for several models in flight (their launches overlap on the chip; serialising sequence launches under a lock
// measured 43.7 k against 55 k images/s for two ResNet-50 models).  The count changes when a model is loaded or
// released; a model notices at its next run and captures its graph again in the other form.  A model that appears
// while another one's sequence launch is in flight drains the device once before its own first launch; its
// ordinary launches next to a later sequence launch of the other model (which read the count a moment too
// early) are harmless: they end without waiting for anybody, so every workgroup of the sequence launch
// becomes resident in the end.
namespace {
std::atomic<int> g_sequence_models{0};
}  // namespace

int HipGraphRuntime::CountSequenceModel(int delta) { return g_sequence_models.fetch_add(delta) + delta; }

bool HipGraphRuntime::SeqNow() const { return use_seq_ && g_sequence_models.load() == 1; }

void HipGraphRuntime::DropSequences() {
  use_seq_ = false;
  if (seq_counted_) { CountSequenceModel(-1); seq_counted_ = false; }
}

void HipGraphRuntime::Launch() {
  // the kernel choice this model was loaded with, for the launches of this thread
  ApplyTuning();
  if (fused_) {
    const bool seq = seq_mode_;
    for (size_t i = 0; i < plan_.size();) {
      if (seq && seq_at_[i] >= 0) {   // (a sequence launch covers whatever grouped launches lie inside its run)
        const SeqRun& r = seqs_[seq_at_[i]];
        HipCheck(cvmhip_conv_seq_launch(r.table, r.nlayers, seq_sync_, r.ops, r.bytes, stream_), "layer-sequence launch");
        seq_ran_ = true;
        i = r.last + 1;
      } else if (!group_at_.empty() && group_at_[i] >= 0) {
        const GroupRun& r = groups_[group_at_[i]];
        if (r.i8) HipCheck(cvmhip_conv_group_launch_i8(r.table, r.nlayers, r.blocks, r.ops, r.bytes, stream_), "grouped convolutions");
        else HipCheck(cvmhip_conv_group_launch(r.table, r.nlayers, r.blocks, r.ops, r.bytes, stream_), "grouped detection heads");
        i = r.last + 1;
      } else {
        RunStep(plan_[i++]);
      }
    }
  } else {
    for (Exec& ex : execs_) ex.kernel->run(ex.call);
  }
}

// The launches of a run never change (shapes, pointers and attributes are
// fixed at load time), so after one eager run they are captured into an
// executable graph and replayed with a single submission.  Per-kernel timing
// needs the eager path (its event pairs must not end up inside a graph);
// CVM_HIP_GRAPH=0 keeps it for good.
void HipGraphRuntime::Run() {
  if (seq_calibration_pending_ && SeqNow()) {   // alone at last: the load-time comparison, now (it runs the graph a few times itself)
    seq_calibration_pending_ = false;
    CalibrateSequences();
  }
  const bool seq_now = SeqNow();
  if (seq_now != seq_mode_) {   // another model with sequence launches appeared or went away: the other form from here on
    if (graph_exec_) { cvmhip_graph_destroy(graph_exec_); graph_exec_ = nullptr; }
    if (graph_state_ == 3) graph_state_ = 2;
    seq_mode_ = seq_now;
  }
  if (graph_state_ == 0) graph_state_ = hooks_.graph ? 1 : -1;
  if (graph_state_ < 0 || cvmhip_kernel_timing_active()) {
    Launch();
    return;
  }
  if (graph_state_ == 1) {  // first run: eager (operators may finish lazy set-up)
    Launch();
    graph_state_ = 2;
    return;
  }
  if (graph_state_ == 2) {
    HipCheck(cvmhip_stream_sync(stream_), "capture");
    if (cvmhip_capture_begin(stream_) == CVMHIP_OK) {
      bool ok = true;
      try {
        Launch();
      } catch (...) {
        ok = false;
      }
      void* exec = nullptr;
      if (cvmhip_capture_end(stream_, &exec) == CVMHIP_OK && ok && exec) {
        graph_exec_ = exec;
        graph_state_ = 3;
      } else {
        if (exec) cvmhip_graph_destroy(exec);
        graph_state_ = -1;  // not capturable: stay eager
        Launch();
        return;
      }
    } else {
      graph_state_ = -1;
      Launch();
      return;
    }
  }
  HipCheck(cvmhip_graph_launch(graph_exec_, stream_), "graph launch");
  if (seq_mode_) seq_ran_ = true;
}

std::map<std::string, double> HipGraphRuntime::ProfileRun() {
  std::map<std::string, double> times;
  void *e0 = nullptr, *e1 = nullptr;
  HipCheck(cvmhip_event_create(&e0), "event");
  HipCheck(cvmhip_event_create(&e1), "event");
  const size_t count = fused_ ? plan_.size() : execs_.size();
  for (size_t i = 0; i < count; ++i) {
    HipCheck(cvmhip_event_record(e0, stream_), "event");
    if (fused_) RunStep(plan_[i]);
    else execs_[i].kernel->run(execs_[i].call);
    HipCheck(cvmhip_event_record(e1, stream_), "event");
    float ms = 0;
    HipCheck(cvmhip_event_elapsed_ms(e0, e1, &ms), "event");
    times[fused_ ? plan_[i].label : execs_[i].call.op] += ms;
  }
  cvmhip_event_destroy(e0);
  cvmhip_event_destroy(e1);
  return times;
}

float HipGraphRuntime::TimeRuns(int iterations) {
  void *e0 = nullptr, *e1 = nullptr;
  HipCheck(cvmhip_event_create(&e0), "event");
  HipCheck(cvmhip_event_create(&e1), "event");
  HipCheck(cvmhip_event_record(e0, stream_), "event");
  for (int i = 0; i < iterations; ++i) Run();
  HipCheck(cvmhip_event_record(e1, stream_), "event");
  float ms = 0;
  HipCheck(cvmhip_event_elapsed_ms(e0, e1, &ms), "event");
  cvmhip_event_destroy(e0);
  cvmhip_event_destroy(e1);
  return ms;
}

void HipGraphRuntime::CopyOutputTo(int index, int32_t* host) {
  CVM_VERIFY(index >= 0 && static_cast<size_t>(index) < outputs_.size());
  const uint32_t eid = entry_id(outputs_[index]);
  HipCheck(cvmhip_copy_d2h(host, entry_ptr_[eid], static_cast<size_t>(shape_size(shape_[eid])) * 4, stream_), "copy output");
  const bool status = RequestSequenceStatus();
  HipCheck(cvmhip_stream_sync(stream_), "copy output");
  if (seq_ran_) {
    CheckSequences(status);
    if (!use_seq_) CopyOutputTo(index, host);   // the run was repeated with one launch per layer
  }
}

// A layer-sequence launch whose bounded waits ran out (its workgroups were not all resident at once) leaves its error
// word set and its results undefined.  Seen after a synchronisation: sequences are switched off for this model for
// good and the run is repeated with one launch per layer.
// The status word travels behind whatever the caller copies back, so that one synchronisation serves both (a second
// copy and wait of its own cost every CVMAPIInference call a round trip to the device).
bool HipGraphRuntime::RequestSequenceStatus() {
  if (!seq_ran_ || !use_seq_ || !seq_sync_) return false;
  const size_t words = cvmhip_conv_seq_sync_bytes() / 4;
  HipCheck(cvmhip_copy_d2h(seq_error_host_, static_cast<uint32_t*>(seq_sync_) + (words - 64), 4, stream_), "sequence status");
  return true;
}

void HipGraphRuntime::CheckSequences(bool requested) {
  seq_ran_ = false;
  if (!use_seq_ || !seq_sync_) return;
  const size_t words = cvmhip_conv_seq_sync_bytes() / 4;
  if (!requested) {
    HipCheck(cvmhip_copy_d2h(seq_error_host_, static_cast<uint32_t*>(seq_sync_) + (words - 64), 4, stream_), "sequence status");
    HipCheck(cvmhip_stream_sync(stream_), "sequence status");
  }
  if (*seq_error_host_ == 0) return;
  std::cerr << "cvm hip: a layer-sequence launch could not keep all its workgroups resident; using one launch per layer\n";
  DropSequences();
  HipCheck(cvmhip_memset32(seq_sync_, 0, words, stream_), "sequence status");
  if (graph_exec_) { cvmhip_graph_destroy(graph_exec_); graph_exec_ = nullptr; }
  graph_state_ = 0;
  Run();
  HipCheck(cvmhip_stream_sync(stream_), "repeat run");
}

const std::vector<const int32_t*>& HipGraphRuntime::FetchOutputs() {
  if (!out_stage_host_) {
    size_t total = 0;
    for (const NodeEntry& e : outputs_) total += AlignUp(static_cast<size_t>(shape_size(shape_[entry_id(e)])) * 4, 64);
    HipCheck(cvmhip_host_alloc(&out_stage_host_, std::max<size_t>(total, 64)), "output staging buffer");
    size_t off = 0;
    for (const NodeEntry& e : outputs_) {
      out_host_.push_back(reinterpret_cast<const int32_t*>(static_cast<char*>(out_stage_host_) + off));
      off += AlignUp(static_cast<size_t>(shape_size(shape_[entry_id(e)])) * 4, 64);
    }
  }
  for (size_t k = 0; k < outputs_.size(); ++k) {
    const uint32_t eid = entry_id(outputs_[k]);
    HipCheck(cvmhip_copy_d2h(const_cast<int32_t*>(out_host_[k]), entry_ptr_[eid], static_cast<size_t>(shape_size(shape_[eid])) * 4,
                             stream_), "copy output");
  }
  const bool status = RequestSequenceStatus();
  HipCheck(cvmhip_stream_sync(stream_), "copy output");
  if (seq_ran_) {
    CheckSequences(status);
    if (!use_seq_) return FetchOutputs();   // the run was repeated with one launch per layer
  }
  return out_host_;
}

int32_t* HipGraphRuntime::DataDevicePtr() {
  const int idx = GetInputIndex("data");
  return entry_ptr_[entry_id(input_nodes_[idx], 0)];
}

void HipGraphRuntime::SyncStream() {
  const bool status = RequestSequenceStatus();
  HipCheck(cvmhip_stream_sync(stream_), "synchronise");
  if (seq_ran_) CheckSequences(status);
}

const Shape& HipGraphRuntime::InputShape() const {
  const int idx = GetInputIndex("data");
  return shape_[entry_id(input_nodes_[idx], 0)];
}

const Shape& HipGraphRuntime::OutputShape(int index) const {
  CVM_VERIFY(index >= 0 && static_cast<size_t>(index) < outputs_.size());
  return shape_[entry_id(outputs_[index])];
}

int HipGraphRuntime::GetInputPrecision() const {
  for (uint32_t i = 0; i < nodes_.size(); ++i)
    if (nodes_[i].is_data()) return precision_[entry_id(i, 0)];
  CVM_FATAL() << "can not find input `data`";
  return -1;
}

int HipGraphRuntime::GetOutputPrecision() const {
  int ret = 0;
  for (const NodeEntry& e : outputs_) ret = std::max(ret, precision_[entry_id(e)]);
  return ret;
}

// infer_attr.cc:93-159 (gas = 5 * elements held + operator cost)
int64_t HipGraphRuntime::GetOps() const {
  int64_t ops = 0, mem_cost = 0;
  const int64_t kMaxBase = static_cast<int64_t>(1) << 30, kMaxOps = static_cast<int64_t>(1) << 40,
                kMaxMem = static_cast<int64_t>(1) << 40;
  for (uint32_t nid = 0; nid < nodes_.size(); ++nid) {
    const Node& n = nodes_[nid];
    if (n.is_variable()) {
      mem_cost += shape_size(shape_[entry_id(nid, 0)]) * 5;
    } else {
      uint32_t out_eid = entry_id(nid, 0);
      int64_t base = 1;
      if (n.func_name == "dense") {
        base = shape_[entry_id(n.inputs[1])][1] * 3;
        if (n.attrs.b("use_bias")) base += 1;
      } else if (n.func_name == "non_max_suppression") {
        base = shape_[entry_id(n.inputs[0])][0] * 20;
      } else if (n.func_name == "conv2d") {
        const Shape& w = shape_[entry_id(n.inputs[1])];
        base = shape_size(w) / w[0] * 3;
        if (n.attrs.b("use_bias")) base += 1;
      } else if (n.func_name == "max_pool2d") {
        base = shape_size(n.attrs.t("pool_size"));
      } else if (n.func_name == "sum") {
        base = shape_size(shape_[entry_id(n.inputs[0])]) / shape_size(shape_[out_eid]);
      }
      CVM_VERIFY(base <= kMaxBase) << "single ops foreach output should not greater than 1G, but " << base;
      base *= shape_size(shape_[out_eid]);
      ops += base;
      CVM_VERIFY(ops <= kMaxOps) << "graph ops exceed MAX_OPS " << kMaxOps;
      int64_t mem = 0;
      for (uint32_t i = 0; i < n.num_outputs; ++i) mem += shape_size(shape_[entry_id(nid, i)]);
      mem_cost += mem * 5;
    }
    CVM_VERIFY(mem_cost <= kMaxMem) << "graph memory cost exceed MAX_MEMORY " << kMaxMem;
  }
  const int64_t ret = mem_cost + ops;
  std::cout << "GetOps: memory cost=" << int(mem_cost / 1000000) << "M percentage=" << 1.f * mem_cost / (ret + 1e-5)
            << " ops=" << int(ops / 1000000) << "M percentage=" << 1.f * ops / (ret + 1e-5) << std::endl;
  return ret;
}

}  // namespace cvmrt
