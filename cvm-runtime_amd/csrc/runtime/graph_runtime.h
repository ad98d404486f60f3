// Host-side graph runtime for the HIP device: loads a CVM graph (JSON) and its
// parameter blob, verifies them with the reference's rules, plans device
// storage and executes the nodes in topological order on one HIP stream.
//
// Mirrors the interface and behaviour of the reference's CvmRuntime
// (src/runtime/graph_runtime.{h,cc}, src/runtime/infer_attr.cc) for a single
// device type, "hip".  Operator kernels are looked up in a registry under
// "cvm.runtime.hip.<op>" -- the naming scheme of graph_runtime.cc:660-664.
#ifndef CVM_RT_GRAPH_RUNTIME_H_
#define CVM_RT_GRAPH_RUNTIME_H_

#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../../../include/cvm_hip_ops.h"
#include "base.h"
#include "json.h"
#include "op_schema.h"

namespace cvmrt {

// A device tensor as an operator sees it: int32, contiguous, row-major.
struct DevTensor {
  int32_t* data = nullptr;
  Shape shape;
  int precision = -1;
  bool is_param = false;  // produced by a variable node other than `data` (constant after load_params)
  int64_t size() const { return shape_size(shape); }
};

struct OpCall;

// What the registry stores for one operator of the device.
struct OpKernel {
  // bytes of device scratch the operator needs for these tensors (the role of
  // FOpExtraSpace, include/cvm/op_attr_types.h:86-90)
  std::function<size_t(const OpCall&)> workspace_bytes;
  // once, after the parameters are on the device (e.g. pre-pack constant filters)
  std::function<void(OpCall&)> prepare;
  // enqueue the operator on call.stream
  std::function<void(OpCall&)> run;
};

// Arguments of one node: inputs, outputs, parsed attributes, scratch, stream --
// the same information CVMArgs carries ([in..., out..., NodeAttrs*] + ext_space).
struct OpCall {
  std::string op;
  std::vector<DevTensor> in, out;
  const OpAttrs* attrs = nullptr;
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  void* stream = nullptr;
  std::shared_ptr<void> state;  // per-node data owned by the kernel (packed filters ...)
};

class OpRegistry {
 public:
  static OpRegistry& Global();
  void Register(const std::string& name, OpKernel k) { table_[name] = std::move(k); }
  const OpKernel* Get(const std::string& name) const {
    auto it = table_.find(name);
    return it == table_.end() ? nullptr : &it->second;
  }
  std::vector<std::string> ListNames() const;

 private:
  std::map<std::string, OpKernel> table_;
};

void RegisterHipKernels();  // fills the registry with cvm.runtime.hip.* (hip_ops.cc)

struct NodeEntry {
  uint32_t node_id = 0, index = 0, version = 0;
};

struct Node {
  std::string op_type;
  std::string name;
  std::string func_name;
  std::vector<NodeEntry> inputs;
  const OpSchema* schema = nullptr;
  OpAttrs attrs;
  uint32_t num_inputs = 1, num_outputs = 1;
  bool is_variable() const { return op_type == "null"; }
  bool is_data() const { return is_variable() && name == "data"; }
};

// One launch of the fused executor (fused_plan.cc).
struct PlanStep {
  enum Kind { NODE, PACK, UNPACK, STEMPACK, CONV, DWCONV, ADD, POOL, SUM } kind = NODE;
  std::string label;            // operator name for the time table
  size_t exec_index = 0;        // NODE: index into execs_
  uint32_t src = 0, src2 = 0, dst = 0;  // entry ids (src2: residual / second addend; UINT32_MAX = none)
  bool out_i8 = false;
  cvmhip_chain chain{}, chain2{};
  const int32_t* bias = nullptr;
  std::shared_ptr<void> weights;  // packed filter (device)
  std::shared_ptr<void> aux;      // row-window copy of the input (device), see cvmhip_pack_stem_input
  bool stem = false;              // CONV through the row-window form
  std::shared_ptr<void> ws;       // CONV: workspace of a K-sliced launch (cvmhip_conv2d_i8_ws), or empty
  size_t ws_bytes = 0;
  bool dw_mfma = false;           // DWCONV through the implicit-GEMM kernel (filter packed as diagonal blocks)
  bool flat = false;              // CONV that is a dense layer over a whole map (kh x kw == h x w): the map is flattened into `aux`
                                  // first (cvmhip_flatten_act_i8) and the layer runs as a 1x1 convolution over h * w * c channels
  bool pool2 = false;             // CONV also takes the 2x2 stride-2 max_pool2d that follows it (cvmhip_conv2d_pool2_i8); dst is the pooled tensor
  bool pool3 = false;             // CONV (stem) also takes the 3x3 stride-2 padding-1 max_pool2d that follows it (cvmhip_conv2d_stem_pool3_i8);
                                  // dst is the pooled tensor, oh x ow its extent
  bool nhwc = false;              // CONV writes int32 pixel-major rows into a slice of entry dst (a fused detection head)
  int64_t dst_off = 0, img_stride = 0;  // that slice: first element, and elements from one image to the next
  // CONV, nhwc: a second head over the same input folded into this launch (cvmhip_conv2d_i8_nhwc_pair): its slice, its
  // channel count, and the merged bias (the first head's, zeros up to a multiple of 32, the second head's)
  bool pair = false;
  uint32_t dst2 = 0;
  int64_t dst_off2 = 0, img_stride2 = 0;
  int oc2 = 0;
  std::shared_ptr<void> pair_bias;
  std::shared_ptr<void> folded_bias;   // CONV, DWCONV: the bias with the chains' rounding terms added (device); `bias` then points here
  uint32_t wsrc = UINT32_MAX, bsrc = UINT32_MAX;   // CONV: entries of the filter and the bias (UINT32_MAX: none)
  int n = 0, c = 0, h = 0, w = 0, oc = 0, kh = 1, kw = 1, sh = 1, sw = 1, ph = 0, pw = 0, dh = 1, dw = 1, oh = 0, ow = 0;
};

class HipGraphRuntime {
 public:
  // with_device == false parses and verifies only (gas estimation from a graph file)
  HipGraphRuntime(const std::string& graph_json, int device_id, bool with_device);
  ~HipGraphRuntime();
  HipGraphRuntime(const HipGraphRuntime&) = delete;
  HipGraphRuntime& operator=(const HipGraphRuntime&) = delete;

  void LoadParams(const std::string& blob);
  // `data` tensor from host memory: int32 values, already widened
  void SetData(const int32_t* host, const Shape& shape);
  void SetDataI8(const int8_t* host, const Shape& shape);   // the same for an input given as int8 bytes
  void Run();      // replays the captured graph once it exists
  void Launch();   // issues every launch of a run on the stream, one by one
  void CopyOutputTo(int index, int32_t* host);  // synchronises the stream
  // every output copied into pinned host memory owned by the runtime (valid until the next call); one synchronisation
  const std::vector<const int32_t*>& FetchOutputs();

  // device-resident variants used to time Run() alone
  int32_t* DataDevicePtr();
  void SyncStream();

  int NumOutputs() const { return static_cast<int>(outputs_.size()); }
  const Shape& InputShape() const;
  const Shape& OutputShape(int index) const;
  int GetInputPrecision() const;
  int GetOutputPrecision() const;
  int64_t GetOps() const;
  int64_t GetStorageSize() const;
  std::string version() const { return version_.substr(0, 32); }
  std::string postprocess_method() const { return postprocess_.substr(0, 32); }

  // per-operator device time of one Run(), in milliseconds, keyed by operator name
  std::map<std::string, double> ProfileRun();
  // elapsed device milliseconds of `iterations` back-to-back Run() calls
  float TimeRuns(int iterations);
  size_t NumNodes() const { return nodes_.size(); }
  // number of launches per Run(): nodes when unfused, plan steps when fused
  size_t NumSteps() const { return fused_ ? plan_.size() : execs_.size(); }
  bool fused() const { return fused_; }
  void LaunchCounts(int* launches, int* sequences, int* layers) const {
    int seq = 0, lay = 0;
    if (SeqNow())
      for (const SeqRun& r : seqs_) { ++seq; lay += r.nlayers; }
    int grouped = 0;   // launches saved by grouped launches; a group inside a sequence launch that is in use saves none
    for (const GroupRun& r : groups_) {
      bool inside = false;
      if (SeqNow())
        for (const SeqRun& q : seqs_) inside = inside || (r.first >= q.first && r.last <= q.last);
      if (!inside) grouped += r.nlayers - 1;
    }
    int extra = 0;   // steps of two launches: a dense layer over a whole map behind the copy that flattens the map
    if (fused_)
      for (const PlanStep& st : plan_) extra += st.flat ? 1 : 0;
    if (launches) *launches = static_cast<int>(NumSteps()) - lay + seq - (fused_ ? grouped : 0) + extra;
    if (sequences) *sequences = seq;
    if (layers) *layers = lay;
  }

 private:
  uint32_t entry_id(uint32_t nid, uint32_t index) const { return node_row_ptr_[nid] + index; }
  uint32_t entry_id(const NodeEntry& e) const { return entry_id(e.node_id, e.index); }
  void Load(const Json& doc);
  void PrepareGraph();
  void SetupShape();
  void SetupPrecision();
  void PlanStorage();
  void SetupStorage();
  void SetupOpExecs();
  void Release();
  void SetInput(uint32_t input_index, const int32_t* data32, const Shape& shape);
  int GetInputIndex(const std::string& name) const;

  std::vector<Node> nodes_;
  std::vector<uint32_t> input_nodes_, node_row_ptr_;
  std::vector<NodeEntry> outputs_;
  uint32_t num_node_entries_ = 0;
  // graph attributes
  std::vector<int> storage_id_, device_index_, precision_;
  std::vector<std::string> dltype_, op_attrs_;
  std::vector<Shape> shape_;
  std::string version_ = "cvm_1.0.0";
  std::string postprocess_;

  struct PoolEntry { size_t bytes = 0; size_t offset = 0; };
  std::vector<PoolEntry> pool_;
  int device_id_ = 0;
  bool with_device_ = false;
  void* slab_ = nullptr;       // one allocation backing every pool entry
  size_t slab_bytes_ = 0;
  void* workspace_ = nullptr;  // shared operator scratch
  size_t workspace_bytes_ = 0;
  void* stream_ = nullptr;
  void* in_stage_host_ = nullptr;  // pinned staging copy of an int8 input
  void* in_stage_dev_ = nullptr;   // its device copy before widening
  void* out_stage_host_ = nullptr; // pinned copies of the outputs, back to back
  std::vector<const int32_t*> out_host_;
  std::vector<int32_t*> entry_ptr_;
  struct Exec { uint32_t nid; const OpKernel* kernel; OpCall call; };
  std::vector<Exec> execs_;
  bool params_loaded_ = false;
  void* graph_exec_ = nullptr;
  int graph_state_ = 0;  // 0 undecided, -1 eager for good, 1 before the first run, 2 ready to capture, 3 captured

  // Test and tuning hooks, read from the environment once, when the model is constructed (never on the
  // launch path): CVM_HIP_FUSE=0 no load-time fusion, CVM_HIP_GRAPH=0 no graph replay, CVM_HIP_SEQ=0 no
  // layer-sequence launches (=1: always, without measuring), CVM_HIP_DW=valu
  // depthwise layers on the vector kernel, CVM_HIP_CONV=lds|wave, CVM_HIP_WAVECFG=<i> and
  // CVM_HIP_TILE="wm,wn" force an implicit-GEMM kernel, a configuration or a tile.
  struct Hooks {
    bool fold_bias = true, fuse = true, graph = true, dw_on_mfma = true, seq = true, seq_forced = false, pool_fuse = true, head_pair = true, head_group = true, conv_group = true;
    int conv_kernel = 0, wave_cfg = -1, tile_wm = 0, tile_wn = 0;
    // layer-sequence launches: CVM_HIP_SEQ_SPIN=<polls> patience of a wait at a layer boundary (0: every wait gives up at once)
    int seq_spin = 2000000;
    bool flat_dense = true;   // CVM_HIP_FLATDENSE=0: a dense layer over a whole map gathers its operand from the map as it lies
    bool seq_chains = true;   // CVM_HIP_SEQ_CHAIN=0: no 1x1 layers chained behind the layer that feeds them (cvmhip_conv_seq_link)
    std::vector<std::pair<int, int>> seq_layer_cfg;   // CVM_HIP_SEQCFG: (layer of a sequence, configuration)
  };
  void ApplyTuning();   // hands the hooks to the kernels' per-thread tuning record
  Hooks hooks_;
  void ReadHooks();

  // ---- fused executor: int8 NHWC activations + folded requantisation chains
  void BuildPlan();
  void RunStep(PlanStep& st);
  bool fused_ = false;
  std::vector<PlanStep> plan_;
  std::vector<void*> i8_ptr_;      // per entry: int8 NHWC form (nullptr if never materialised)
  std::vector<std::shared_ptr<void>> own_storage_;  // int32 tensors the planner moved out of the shared storage pool
  void* i8_slab_ = nullptr;

  // ---- runs of consecutive convolution steps issued as one layer-sequence launch (cvmhip_conv_seq_launch).  The
  // steps stay in plan_: they are what runs when sequences are switched off and after a sequence launch
  // reported that its waits ran out.
  struct SeqRun {
    size_t first = 0, last = 0;         // plan_ indices, inclusive
    std::shared_ptr<void> owner;        // device copy of the layer table
    void* table = nullptr;
    int nlayers = 0;
    double ops = 0, bytes = 0;          // algorithmic operations and HBM bytes of its layers (for the measurement harness)
    std::vector<int> cfgs;              // configuration of the tile kernel per layer
  };
  void FoldRequant();   // rounding terms of the convolutions' requantisation into their biases (cvmhip_fold_requant)
  void BuildSequences();
 public:
  // configurations of the tile kernel chosen for the layers of all sequence launches, in order
  std::vector<int> SequenceConfigs() const {
    std::vector<int> v;
    for (const SeqRun& r : seqs_) v.insert(v.end(), r.cfgs.begin(), r.cfgs.end());
    return v;
  }
 private:
  // Runs of consecutive detection-head steps (int32 pixel-major output, independent of one another) that share one launch
  struct GroupRun {
    size_t first = 0, last = 0;         // plan_ indices, inclusive
    std::shared_ptr<void> owner;        // device copy of the layer table
    void* table = nullptr;
    int nlayers = 0, blocks = 0;
    bool i8 = false;                    // int8 outputs (k_conv_group8) instead of detection heads
    double ops = 0, bytes = 0;
  };
  void BuildGroups();
  std::vector<GroupRun> groups_;
  std::vector<int> group_at_;           // per plan_ index: the group that starts there, or -1
  void CalibrateSequences();            // measures a run with and without sequence launches, keeps the faster
  static int CountSequenceModel(int delta);    // models with sequence launches alive in this process, after the change
  bool SeqNow() const;                  // does the next run use sequence launches?
  bool seq_mode_ = false;               // what the launches being issued (and the captured graph) use
  void DropSequences();                 // sequence launches are off for good for this model
  bool RequestSequenceStatus();         // before a synchronisation: the status word of the sequence launches rides along (true when requested)
  void CheckSequences(bool requested);  // after a synchronisation: did a sequence launch give up?  (fetches the word itself unless requested)
  std::vector<SeqRun> seqs_;
  std::vector<int> seq_at_;             // per plan_ index: the run that starts there, or -1
  void* seq_sync_ = nullptr;            // counters and error word of the sequence launches (device)
  uint32_t* seq_error_host_ = nullptr;  // pinned copy of the error word
  bool use_seq_ = false;
  bool seq_counted_ = false;            // this model is counted among the models with sequence launches
  bool seq_calibration_pending_ = false;   // loaded next to another such model: the two launch forms are compared at the first run alone
  bool seq_ran_ = false;                // a sequence launch was issued since the last check
};

}  // namespace cvmrt
#endif
