// Load-time planning of the fused executor.
//
// The reference runs one kernel per node on int32 NCHW tensors.  Inside a
// verified graph, conv2d/dense operands are proven to fit 8 bits, and the
// nodes that follow a conv2d / dense / elemwise_add / sum are almost always a
// short chain of relu / cvm_right_shift / cvm_clip / clip whose result is again
// 8 bits wide.  The planner therefore
//   * groups  producer -> chain  into one launch whose epilogue applies the
//     chain to the int32 accumulator (the chain's intermediate tensors are
//     never written),
//   * keeps group outputs that are provably within [-128, 127] as int8 NHWC
//     between layers, converting (pack / unpack) only where a node outside the
//     fused set, or a graph head, needs the int32 NCHW tensor,
//   * folds a residual elemwise_add (and its own chain) into the epilogue of
//     the convolution that produces one of its addends,
//   * turns flatten -> dense over a 4-D tensor into a convolution whose kernel
//     covers the whole feature map,
//   * lets a convolution whose result only goes through transpose(0,2,3,1) ->
//     reshape -> concatenate (a detection head) write its pixel-major rows
//     straight into its slice of the concatenated tensor.
// Every value a later node or the caller can observe is computed by the same
// integer arithmetic as in node-by-node execution.
#include <cstring>
#include <algorithm>
#include <climits>
#include <cstdlib>
#include <map>

#include "graph_runtime.h"

namespace cvmrt {

namespace {

const uint32_t kNone = UINT32_MAX;

void Check(int rc, const char* what) {
  if (rc == CVMHIP_OK) return;
  if (rc < CVMHIP_ERR_RUNTIME) CVM_VERIFY(false) << what << ": " << cvmhip_last_error();
  CVM_CHECK(false) << what << ": " << cvmhip_last_error();
}

struct DeviceBuffer {
  void* ptr = nullptr;
  ~DeviceBuffer() { if (ptr) cvmhip_free(ptr); }
};

struct Bound { int64_t lo = INT32_MIN, hi = INT32_MAX; };

bool FitsI8(const Bound& b) { return b.lo >= -128 && b.hi <= 127; }

// value range after one chain stage (only ranges that the stage itself guarantees)
bool ChainStage(const Node& n, cvmhip_stage* st, Bound* b) {
  const OpAttrs& a = n.attrs;
  if (n.func_name == "relu") {
    st->kind = CVMHIP_STAGE_RELU;
    b->lo = std::max<int64_t>(b->lo, 0);
    b->hi = std::max<int64_t>(b->hi, 0);
    return true;
  }
  if (n.func_name == "cvm_right_shift") {
    const int p = (int)a.i("precision"), s = (int)a.i("shift_bit");
    st->kind = CVMHIP_STAGE_RSHIFT;
    st->precision = p;
    st->shift_bit = s;
    const int64_t r = (static_cast<int64_t>(1) << (p - 1)) - 1;
    if (r == 0) { b->lo = b->hi = 0; }
    else if (s >= 31 || p + s >= 32) { *b = Bound(); }  // these regimes do not clip (elemwise.cc:131-137)
    else { b->lo = -r; b->hi = r; }
    return true;
  }
  if (n.func_name == "cvm_clip") {
    const int p = (int)a.i("precision");
    const int64_t r = (static_cast<int64_t>(1) << (p - 1)) - 1;
    st->kind = CVMHIP_STAGE_CLIP;
    st->lo = static_cast<int32_t>(-r);
    st->hi = static_cast<int32_t>(r);
    b->lo = std::max(b->lo, -r);
    b->hi = std::min(b->hi, r);
    return true;
  }
  if (n.func_name == "clip") {
    st->kind = CVMHIP_STAGE_CLIP;
    st->lo = (int32_t)a.i("a_min");
    st->hi = (int32_t)a.i("a_max");
    b->lo = std::max<int64_t>(b->lo, st->lo);
    b->hi = std::min<int64_t>(b->hi, st->hi);
    return true;
  }
  return false;
}

// operators that only move or select input values
bool ValuePreserving(const std::string& op) {
  static const char* kOps[] = {"relu", "max_pool2d", "flatten", "reshape", "expand_dims", "squeeze", "transpose",
                               "concatenate", "strided_slice", "slice_like", "repeat", "tile", "upsampling"};
  for (const char* o : kOps)
    if (op == o) return true;
  return false;
}

bool ConsumesI8(const std::string& op) {
  return op == "conv2d" || op == "dense" || op == "elemwise_add" || op == "max_pool2d" || op == "sum" || op == "flatten";
}

}  // namespace

void HipGraphRuntime::BuildPlan() {
  const uint32_t ne = num_node_entries_;
  std::vector<std::vector<uint32_t>> uses(ne);
  std::vector<bool> is_head(ne, false), has_i8(ne, false), has_i32(ne, false), safe(ne, false);
  std::vector<bool> absorbed(nodes_.size(), false);
  std::vector<uint32_t> fold_src(ne, kNone);     // flatten output -> the 4-D tensor it flattens
  std::vector<int> producer_step(ne, -1);        // plan index of the step that writes the entry's i8 form
  std::vector<size_t> exec_of(nodes_.size(), SIZE_MAX);
  for (size_t i = 0; i < execs_.size(); ++i) exec_of[execs_[i].nid] = i;
  for (uint32_t nid = 0; nid < nodes_.size(); ++nid)
    for (const NodeEntry& e : nodes_[nid].inputs) uses[entry_id(e)].push_back(nid);
  for (const NodeEntry& e : outputs_) is_head[entry_id(e)] = true;

  i8_ptr_.assign(ne, nullptr);
  std::vector<size_t> i8_off(ne, SIZE_MAX);
  size_t i8_bytes = 0;
  auto i8_alloc = [&](uint32_t eid) {
    if (i8_off[eid] != SIZE_MAX) return;
    const Shape& s = shape_[eid];
    const int64_t npix = s.size() == 4 ? s[0] * s[2] * s[3] : s[0];
    i8_off[eid] = i8_bytes;
    i8_bytes += cvmhip_packed_act_bytes(npix, (int)s[1]);
  };
  auto i8_capable_shape = [&](uint32_t eid) { return shape_[eid].size() == 4 || shape_[eid].size() == 2; };
  auto pix = [&](uint32_t eid) { return shape_[eid].size() == 4 ? (int)(shape_[eid][2] * shape_[eid][3]) : 1; };

  // concatenate inputs that a producer has already written into the output tensor
  std::vector<std::vector<bool>> in_place(nodes_.size());
  std::map<uint32_t, std::shared_ptr<DeviceBuffer>> own_storage;
  std::vector<std::vector<bool>> head_safe(ne);  // per concatenated entry: int8 range of each part written in place

  // Moves an int32 tensor to storage of its own and points every node that reads or writes it there.
  // Needed wherever a fused step writes such a tensor earlier than the node that produces it in the
  // graph's order: the graph's storage plan may still lend that storage to another tensor then.
  std::vector<int> sid_users(pool_.size(), 0);
  for (uint32_t e = 0; e < ne; ++e) ++sid_users[storage_id_[e]];
  auto privatize = [&](uint32_t eid) {
    if (own_storage.count(eid)) return;
    auto buf = std::make_shared<DeviceBuffer>();
    Check(cvmhip_alloc(&buf->ptr, std::max<size_t>(static_cast<size_t>(shape_size(shape_[eid])) * 4, 4)), "tensor storage");
    own_storage[eid] = buf;
    own_storage_.push_back(buf);
    entry_ptr_[eid] = static_cast<int32_t*>(buf->ptr);
    for (Exec& e : execs_) {
      const Node& en = nodes_[e.nid];
      for (size_t k = 0; k < en.inputs.size(); ++k)
        if (entry_id(en.inputs[k]) == eid) e.call.in[k].data = entry_ptr_[eid];
      for (uint32_t k = 0; k < en.num_outputs; ++k)
        if (entry_id(e.nid, k) == eid) e.call.out[k].data = entry_ptr_[eid];
    }
  };
  // int32 result of a fused step: written at the position of the step's first node
  auto early_i32 = [&](uint32_t eid) {
    if (sid_users[storage_id_[eid]] > 1) privatize(eid);
  };

  std::vector<PlanStep> plan;
  auto need_i32 = [&](uint32_t eid) {
    if (has_i32[eid]) return;
    CVM_CHECK(has_i8[eid]);
    PlanStep st;
    st.kind = PlanStep::UNPACK;
    st.label = "unpack_nhwc_i8";
    st.src = st.dst = eid;
    st.n = (int)shape_[eid][0];
    st.c = (int)shape_[eid][1];
    st.h = pix(eid);
    plan.push_back(st);
    has_i32[eid] = true;
  };
  auto need_i8 = [&](uint32_t eid) {
    if (has_i8[eid]) return;
    CVM_CHECK(has_i32[eid] && i8_capable_shape(eid));
    i8_alloc(eid);
    PlanStep st;
    st.kind = PlanStep::PACK;
    st.label = "pack_nhwc_i8";
    st.src = st.dst = eid;
    st.n = (int)shape_[eid][0];
    st.c = (int)shape_[eid][1];
    st.h = pix(eid);
    producer_step[eid] = (int)plan.size();
    plan.push_back(st);
    has_i8[eid] = true;
  };

  // follows the unary chain behind `start`; returns the entry the group finally writes
  auto follow_chain = [&](uint32_t start, cvmhip_chain* chain, Bound* bound) {
    uint32_t cur = start;
    chain->count = 0;
    while (chain->count < 4 && uses[cur].size() == 1 && !is_head[cur]) {
      const uint32_t cn = uses[cur][0];
      const Node& c = nodes_[cn];
      if (absorbed[cn]) break;
      cvmhip_stage st = {};
      Bound nb = *bound;
      if (c.func_name == "broadcast_mul" && c.inputs.size() == 2) {
        // the requantisation scale: a product with a constant scalar, its result shaped like the chain's value
        const uint32_t a = entry_id(c.inputs[0]), b = entry_id(c.inputs[1]);
        const uint32_t other = a == cur ? b : a;
        const Node& on = nodes_[(a == cur ? c.inputs[1] : c.inputs[0]).node_id];
        if (a == b || !on.is_variable() || on.is_data() || shape_size(shape_[other]) != 1 ||
            shape_[entry_id(cn, 0)] != shape_[cur])
          break;
        int32_t m = 0;
        Check(cvmhip_copy_d2h(&m, entry_ptr_[other], sizeof(m), stream_), "read scale");
        Check(cvmhip_stream_sync(stream_), "read scale");
        st.kind = CVMHIP_STAGE_MUL;
        st.lo = m;
        const int64_t p = nb.lo * m, q = nb.hi * m;   // |bounds| <= 2^31 and |m| <= 2^31: no int64 overflow
        nb.lo = std::min(p, q);
        nb.hi = std::max(p, q);
        if (nb.lo < INT32_MIN || nb.hi > INT32_MAX) nb = Bound();   // the product may wrap
      } else if (c.inputs.size() != 1 || !ChainStage(c, &st, &nb)) {
        break;
      }
      chain->stage[chain->count++] = st;
      *bound = nb;
      absorbed[cn] = true;
      cur = entry_id(cn, 0);
    }
    return cur;
  };
  // where should a fused group leave its result?
  auto wants_i8 = [&](uint32_t eid, const Bound& b) {
    if (!FitsI8(b) || !i8_capable_shape(eid)) return false;
    for (uint32_t cn : uses[eid])
      if (ConsumesI8(nodes_[cn].func_name)) return true;
    return false;
  };
  auto finish_output = [&](PlanStep* st, uint32_t out, const Bound& b) {
    st->dst = out;
    st->out_i8 = wants_i8(out, b);
    if (st->out_i8) {
      i8_alloc(out);
      has_i8[out] = true;
      safe[out] = true;
      producer_step[out] = (int)plan.size();
    } else {
      has_i32[out] = true;
      safe[out] = FitsI8(b);
      early_i32(out);
    }
  };

  // conv result `out` (N, C, H, W) -> transpose(0,2,3,1) -> reshape/flatten -> one input of a concatenate
  // whose leading dimensions multiply to N: image n's H*W*C pixel-major values are one contiguous run of
  // the concatenated tensor.  Marks the three nodes as done and points the step at that run.
  auto fuse_head = [&](uint32_t out, PlanStep* st) {
    const Shape& os = shape_[out];
    if (os.size() != 4 || is_head[out] || uses[out].size() != 1) return false;
    const uint32_t tn = uses[out][0];
    const Node& t = nodes_[tn];
    if (t.func_name != "transpose" || absorbed[tn] || t.attrs.t("axes") != Shape{0, 2, 3, 1}) return false;
    const uint32_t te = entry_id(tn, 0);
    if (is_head[te] || uses[te].size() != 1) return false;
    const uint32_t rn = uses[te][0];
    const Node& r = nodes_[rn];
    if ((r.func_name != "reshape" && r.func_name != "flatten") || absorbed[rn]) return false;
    const uint32_t re = entry_id(rn, 0);
    if (is_head[re] || uses[re].size() != 1) return false;
    const uint32_t cn = uses[re][0];
    const Node& c = nodes_[cn];
    if (c.func_name != "concatenate" || absorbed[cn]) return false;
    const Shape& rs = shape_[re];
    int64_t axis = c.attrs.i("axis");
    if (axis < 0) axis += (int64_t)rs.size();
    if (axis < 0 || axis >= (int64_t)rs.size()) return false;
    int64_t outer = 1, inner = 1, before = 0;
    for (int64_t d = 0; d < axis; ++d) outer *= rs[d];
    for (size_t d = axis + 1; d < rs.size(); ++d) inner *= rs[d];
    if (outer != os[0]) return false;
    int at = -1;
    for (size_t k = 0; k < c.inputs.size(); ++k) {
      const uint32_t ie = entry_id(c.inputs[k]);
      if (ie == re) {
        if (at >= 0) return false;  // the same tensor twice: leave it to the copy kernels
        at = (int)k;
      } else if (at < 0) {
        before += shape_[ie][axis];
      }
    }
    if (at < 0) return false;
    const uint32_t ce = entry_id(cn, 0);
    // the slice is written long before the concatenate node's place in the order
    privatize(ce);
    st->nhwc = true;
    st->dst = ce;
    st->dst_off = before * inner;
    st->img_stride = shape_[ce][axis] * inner;
    st->out_i8 = false;
    st->label += "+head";
    absorbed[tn] = absorbed[rn] = true;
    if (in_place[cn].empty()) in_place[cn].assign(c.inputs.size(), false);
    in_place[cn][at] = true;
    return true;
  };

  // test and tuning hook: CVM_HIP_DW=valu keeps depthwise layers on the vector kernel
  const bool dw_on_mfma = hooks_.dw_on_mfma;
  for (uint32_t nid = 0; nid < nodes_.size(); ++nid) {
    const Node& n = nodes_[nid];
    if (n.is_variable()) {
      const uint32_t eid = entry_id(nid, 0);
      has_i32[eid] = true;
      safe[eid] = precision_[eid] <= 8;  // `data` is clamped, parameters are range-checked on load
      continue;
    }
    if (absorbed[nid]) continue;
    const uint32_t out0 = entry_id(nid, 0);
    const std::string& op = n.func_name;
    const OpAttrs& a = n.attrs;
    const size_t ex = exec_of[nid];
    bool done = false;

    if (op == "conv2d" || op == "dense") {
      const uint32_t xe = entry_id(n.inputs[0]), we = entry_id(n.inputs[1]);
      const bool has_bias = n.inputs.size() == 3;
      const bool params_const = nodes_[n.inputs[1].node_id].is_variable() && !nodes_[n.inputs[1].node_id].is_data() &&
                                (!has_bias || (nodes_[n.inputs[2].node_id].is_variable() && !nodes_[n.inputs[2].node_id].is_data()));
      PlanStep st;
      st.label = op;
      st.bias = has_bias ? entry_ptr_[entry_id(n.inputs[2])] : nullptr;
      st.wsrc = we;
      st.bsrc = has_bias ? entry_id(n.inputs[2]) : kNone;
      bool ok = params_const;
      uint32_t src = xe;
      if (ok && op == "conv2d") {
        const Shape &x = shape_[xe], &w = shape_[we];
        const int groups = (int)a.i("groups");
        ok = w.size() == 4 && w[0] == a.i("channels") && w[1] == x[1] / groups && w[2] == a.t("kernel_size")[0] &&
             w[3] == a.t("kernel_size")[1];
        st.n = (int)x[0]; st.c = (int)x[1]; st.h = (int)x[2]; st.w = (int)x[3];
        st.oc = (int)w[0]; st.kh = (int)w[2]; st.kw = (int)w[3];
        st.sh = (int)a.t("strides")[0]; st.sw = (int)a.t("strides")[1];
        st.ph = (int)a.t("padding")[0]; st.pw = (int)a.t("padding")[1];
        st.dh = (int)a.t("dilation")[0]; st.dw = (int)a.t("dilation")[1];
        if (groups == 1) {
          st.kind = PlanStep::CONV;
        } else if (groups == x[1] && w[0] == x[1] && w[1] == 1 && safe[xe]) {
          st.kind = PlanStep::DWCONV;  // exact only for operands known to fit int8: this path does not narrow
        } else {
          ok = false;
        }
      } else if (ok) {
        st.kind = PlanStep::CONV;
        if (fold_src[xe] != kNone) {  // flatten(4-D) -> dense == convolution over the whole map
          src = fold_src[xe];
          const Shape& x = shape_[src];
          st.n = (int)x[0]; st.c = (int)x[1]; st.h = (int)x[2]; st.w = (int)x[3];
          st.kh = st.h; st.kw = st.w;
        } else {
          const Shape& x = shape_[xe];
          st.n = (int)x[0]; st.c = (int)x[1]; st.h = st.w = 1;
        }
        st.oc = (int)shape_[we][0];
        ok = shape_[we].size() == 2 && shape_[we][1] == (int64_t)st.c * st.kh * st.kw;
        // dense multiplies the int32 values as they are (ops.cc:53-62; only conv2d narrows), so the int8 form
        // is exact only for operands proven to lie in [-128, 127]; otherwise the node keeps its int32 kernel
        ok = ok && safe[src] && safe[we];
      }
      // A few-channel input that only exists as int32 (the image itself) goes through the
      // row-window form: packed once into a zero-padded int8 tensor, convolved without masks.
      const bool stem = ok && op == "conv2d" && st.kind == PlanStep::CONV && !has_i8[src] && has_i32[src] &&
                        cvmhip_stem_eligible(st.c, st.kh, st.kw, st.dh, st.dw) &&
                        cvmhip_stem_input_bytes(st.n, st.h, st.w, st.kh, st.kw, st.sh, st.sw, st.ph, st.pw) > 0;
      if (stem) {
        auto in = std::make_shared<DeviceBuffer>();
        Check(cvmhip_alloc(&in->ptr, cvmhip_stem_input_bytes(st.n, st.h, st.w, st.kh, st.kw, st.sh, st.sw, st.ph, st.pw)),
              "row-window input buffer");
        auto buf = std::make_shared<DeviceBuffer>();
        Check(cvmhip_alloc(&buf->ptr, cvmhip_packed_stem_weight_bytes(st.oc, st.kh, st.kw)), "filter buffer");
        Check(cvmhip_pack_stem_weights(entry_ptr_[we], buf->ptr, st.oc, st.c, st.kh, st.kw, stream_), "filter pack");
        PlanStep pk = st;
        pk.kind = PlanStep::STEMPACK;
        pk.label = "pack_stem_input";
        pk.src = pk.dst = src;
        pk.aux = in;
        plan.push_back(pk);
        st.stem = true;
        st.aux = in;
        st.weights = buf;
        st.src = src;
        st.src2 = kNone;
        Bound b;
        const uint32_t out = follow_chain(out0, &st.chain, &b);
        finish_output(&st, out, b);
        plan.push_back(st);
        done = true;
      } else if (ok) {
        need_i8(src);
        auto buf = std::make_shared<DeviceBuffer>();
        if (st.kind == PlanStep::CONV) {
          Check(cvmhip_alloc(&buf->ptr, cvmhip_packed_weight_bytes(st.oc, st.c, st.kh, st.kw)), "filter buffer");
          Check(cvmhip_pack_weights(entry_ptr_[we], buf->ptr, st.oc, st.c, st.kh, st.kw, stream_), "filter pack");
        } else if (dw_on_mfma && cvmhip_depthwise_mfma_eligible(st.c, st.kh, st.kw)) {
          // channels in whole tiles of 32: the depthwise layer runs on the matrix cores (diagonal filter blocks)
          Check(cvmhip_alloc(&buf->ptr, cvmhip_packed_depthwise_mfma_bytes(st.c, st.kh, st.kw)), "filter buffer");
          Check(cvmhip_pack_depthwise_weights_mfma(entry_ptr_[we], buf->ptr, st.c, st.kh, st.kw, stream_), "filter pack");
          st.dw_mfma = true;
        } else {
          Check(cvmhip_alloc(&buf->ptr, cvmhip_packed_depthwise_bytes(st.c, st.kh, st.kw)), "filter buffer");
          Check(cvmhip_pack_depthwise_weights(entry_ptr_[we], buf->ptr, st.c, st.kh, st.kw, stream_), "filter pack");
        }
        st.weights = buf;
        st.src = src;
        st.src2 = kNone;
        Bound b;
        const uint32_t out = follow_chain(out0, &st.chain, &b);
        bool paired = false;
        if (st.kind == PlanStep::CONV && fuse_head(out, &st)) {
          head_safe[st.dst].push_back(FitsI8(b));
          // The other head of the same feature map (same input, filter size, strides, padding, dilation and chain):
          // the two become one convolution whose filter is the first head's rows, padded to a multiple of 32,
          // followed by the second head's, and whose workgroups write to the slice their channels belong to.
          for (size_t k = plan.size(); hooks_.head_pair && k-- > 0 && !paired;) {
            PlanStep& o = plan[k];
            if (o.kind != PlanStep::CONV || !o.nhwc || o.pair || o.src != st.src || o.n != st.n || o.c != st.c || o.h != st.h ||
                o.w != st.w || o.kh != st.kh || o.kw != st.kw || o.sh != st.sh || o.sw != st.sw || o.ph != st.ph ||
                o.pw != st.pw || o.dh != st.dh || o.dw != st.dw || std::memcmp(&o.chain, &st.chain, sizeof(st.chain)) != 0)
              continue;
            const int split = (o.oc + 31) / 32 * 32;
            auto both = std::make_shared<DeviceBuffer>();
            Check(cvmhip_alloc(&both->ptr, cvmhip_packed_weight_pair_bytes(o.oc, st.oc, st.c, st.kh, st.kw)), "filter buffer");
            Check(cvmhip_pack_weights_pair(entry_ptr_[o.wsrc], o.oc, entry_ptr_[st.wsrc], st.oc, both->ptr, st.c, st.kh, st.kw, stream_),
                  "filter pack");
            auto bias = std::make_shared<DeviceBuffer>();
            Check(cvmhip_alloc(&bias->ptr, static_cast<size_t>(split + st.oc) * 4), "bias buffer");
            Check(cvmhip_memset32(bias->ptr, 0, static_cast<size_t>(split + st.oc), stream_), "bias buffer");
            if (o.bias) Check(cvmhip_copy_d2d(bias->ptr, o.bias, static_cast<size_t>(o.oc) * 4, stream_), "bias copy");
            if (st.bias)
              Check(cvmhip_copy_d2d(static_cast<int32_t*>(bias->ptr) + split, st.bias, static_cast<size_t>(st.oc) * 4, stream_), "bias copy");
            o.weights = both;
            o.pair_bias = bias;
            o.pair = true;
            o.dst2 = st.dst;
            o.dst_off2 = st.dst_off;
            o.img_stride2 = st.img_stride;
            o.oc2 = st.oc;
            o.label += "+head";
            paired = true;
          }
        } else {
          finish_output(&st, out, b);
        }
        if (!paired) plan.push_back(st);
        done = true;
      }
    } else if (op == "elemwise_add") {
      const uint32_t ae = entry_id(n.inputs[0]), be = entry_id(n.inputs[1]);
      if (has_i8[ae] && has_i8[be] && safe[ae] && safe[be] && ae != be) {
        cvmhip_chain chain;
        Bound b;
        b.lo = -256;
        b.hi = 254;
        const uint32_t out = follow_chain(out0, &chain, &b);
        // A block whose two addends are convolutions -- the main path's last layer and the shortcut projection, which
        // reads the block's input like the main path's first layer does -- is reordered: the projection moves next to
        // that first layer and the main path's last layer takes the add.  Where no layer sequence runs, the two
        // neighbours are independent and share a launch (BuildGroups); inside a layer sequence the order is worth
        // 2 us of ResNet-50's 310 (the projection's large output is written long before the add reads it).
        if (hooks_.conv_group) {
          const int pa = producer_step[ae], pb = producer_step[be];
          const int late = pa > pb ? pa : pb, early = pa > pb ? pb : pa;
          const uint32_t le = pa > pb ? ae : be, ee = pa > pb ? be : ae;
          auto plain = [&](int s, uint32_t e) {
            return s >= 0 && plan[s].kind == PlanStep::CONV && !plan[s].stem && !plan[s].nhwc && plan[s].out_i8 && plan[s].src2 == kNone &&
                   !plan[s].pool2 && plan[s].dst == e && uses[e].size() == 1 && !is_head[e];
          };
          if (early >= 0 && plain(late, le) && plain(early, ee)) {
            int first = -1;   // the first convolution of the main path: reads what the late one reads
            for (int s = 0; s < early && first < 0; ++s)
              if (plan[s].kind == PlanStep::CONV && !plan[s].stem && plan[s].out_i8 && plan[s].src == plan[late].src) first = s;
            if (first >= 0) {
              const int to = first + 1;
              const PlanStep moved = plan[late];
              plan.erase(plan.begin() + late);
              plan.insert(plan.begin() + to, moved);
              for (int& v : producer_step) {
                if (v == late) v = to;
                else if (v >= to && v < late) ++v;
              }
            }
          }
        }
        // fold into the convolution that produced one addend, when the other addend exists by then
        bool folded = false;
        for (int swap = 0; swap < 2 && !folded; ++swap) {
          const uint32_t x = swap ? be : ae, r = swap ? ae : be;
          const int ps = producer_step[x], pr = producer_step[r];
          if (ps < 0 || pr < 0 || pr >= ps || plan[ps].stem) continue;
          PlanStep& cs = plan[ps];
          if (cs.kind != PlanStep::CONV || cs.dst != x || !cs.out_i8 || cs.src2 != kNone) continue;
          if (uses[x].size() != 1 || is_head[x]) continue;
          cs.src2 = r;
          cs.chain2 = chain;
          cs.label += "+add";
          // the conv now writes the add group's output instead of its own
          has_i8[x] = false;
          cs.dst = out;
          cs.out_i8 = wants_i8(out, b);
          if (cs.out_i8) {
            i8_alloc(out);
            has_i8[out] = true;
            safe[out] = true;
            producer_step[out] = ps;
          } else {
            has_i32[out] = true;
            safe[out] = FitsI8(b);
            early_i32(out);
          }
          folded = true;
        }
        if (!folded) {
          PlanStep st;
          st.kind = PlanStep::ADD;
          st.label = "elemwise_add";
          st.src = ae;
          st.src2 = be;
          st.chain = chain;
          st.n = (int)shape_[ae][0];
          st.c = (int)shape_[ae][1];
          st.h = pix(ae);
          finish_output(&st, out, b);
          plan.push_back(st);
        }
        done = true;
      }
    } else if (op == "max_pool2d") {
      const uint32_t xe = entry_id(n.inputs[0]);
      if (has_i8[xe] && safe[xe]) {
        PlanStep st;
        st.kind = PlanStep::POOL;
        st.label = op;
        st.src = xe;
        const Shape &x = shape_[xe], &y = shape_[out0], &pad = a.t("padding");
        st.n = (int)x[0]; st.c = (int)x[1]; st.h = (int)x[2]; st.w = (int)x[3];
        st.oh = (int)y[2]; st.ow = (int)y[3];
        st.kh = (int)a.t("pool_size")[0]; st.kw = (int)a.t("pool_size")[1];
        st.sh = (int)a.t("strides")[0]; st.sw = (int)a.t("strides")[1];
        st.ph = (int)pad[0]; st.pw = pad.size() == 2 ? (int)pad[1] : (int)pad[0];
        Bound b;
        b.lo = -128;
        b.hi = 127;
        finish_output(&st, out0, b);
        // A 2x2 window with stride 2 and no padding over an even extent, fed by a convolution that nobody else reads:
        // the convolution takes the maximum itself and writes the pooled tensor (the full-resolution one is never stored).
        const int ps = producer_step[xe];
        // The head of a ResNet: a 3x3 window with stride 2 and padding 1 behind a row-window convolution with 32 or 64
        // output channels that nobody else reads becomes part of that convolution's launch (at small batches).
        if (st.out_i8 && hooks_.pool_fuse && ps >= 0 && plan[ps].kind == PlanStep::CONV && plan[ps].dst == xe &&
            plan[ps].out_i8 && plan[ps].stem && !plan[ps].pool3 && uses[xe].size() == 1 && !is_head[xe] && st.kh == 3 &&
            st.kw == 3 && st.sh == 2 && st.sw == 2 && st.ph == 1 && st.pw == 1 &&
            // one workgroup per 4 x 8 pooled pixels: worth it while they all run at once (small batches)
            (int64_t)plan[ps].n * ((st.oh + 3) / 4) * ((st.ow + 7) / 8) <= 512 &&
            cvmhip_conv2d_stem_pool3_i8_eligible(plan[ps].n, plan[ps].c, plan[ps].h, plan[ps].w, plan[ps].oc, plan[ps].kh,
                                                 plan[ps].kw, plan[ps].sh, plan[ps].sw, plan[ps].ph, plan[ps].pw, st.oh, st.ow)) {
          PlanStep& cs = plan[ps];
          cs.pool3 = true;
          cs.oh = st.oh;
          cs.ow = st.ow;
          cs.label += "+pool";
          cs.dst = out0;
          has_i8[xe] = false;
          producer_step[out0] = ps;
          done = true;
        } else
        if (st.out_i8 && hooks_.pool_fuse && ps >= 0 && plan[ps].kind == PlanStep::CONV && plan[ps].dst == xe &&
            plan[ps].out_i8 && !plan[ps].stem && !plan[ps].nhwc && plan[ps].src2 == kNone && !plan[ps].pool2 &&
            uses[xe].size() == 1 && !is_head[xe] && st.kh == 2 && st.kw == 2 && st.sh == 2 && st.sw == 2 && st.ph == 0 &&
            st.pw == 0 && st.h % 2 == 0 && st.w % 2 == 0 && st.oh == st.h / 2 && st.ow == st.w / 2 &&
            cvmhip_conv2d_pool2_i8_eligible(plan[ps].n, plan[ps].c, plan[ps].h, plan[ps].w, plan[ps].oc, plan[ps].kh,
                                            plan[ps].kw, plan[ps].sh, plan[ps].sw, plan[ps].ph, plan[ps].pw, plan[ps].dh,
                                            plan[ps].dw)) {
          PlanStep& cs = plan[ps];
          cs.pool2 = true;
          cs.label += "+pool";
          cs.dst = out0;
          has_i8[xe] = false;
          producer_step[out0] = ps;
          done = true;
        } else if (st.out_i8) {
          plan.push_back(st);
          done = true;
        } else {  // nobody downstream reads int8: leave the node to the int32 kernel
          has_i32[out0] = false;
        }
      }
    } else if (op == "sum") {
      const uint32_t xe = entry_id(n.inputs[0]);
      Shape ax = a.t("axis");
      for (auto& v : ax) v = v < 0 ? v + 4 : v;
      std::sort(ax.begin(), ax.end());
      if (has_i8[xe] && safe[xe] && shape_[xe].size() == 4 && ax == Shape{2, 3} && !a.b("exclude")) {
        PlanStep st;
        st.kind = PlanStep::SUM;
        st.label = op;
        st.src = xe;
        st.n = (int)shape_[xe][0];
        st.c = (int)shape_[xe][1];
        st.h = pix(xe);
        Bound b;
        const uint32_t out = follow_chain(out0, &st.chain, &b);
        // (N, C) and (N, C, 1, 1) share one memory image
        const Shape& os = shape_[out];
        const bool flat = os.size() == 2 || (os.size() == 4 && os[2] == 1 && os[3] == 1);
        st.dst = out;
        st.out_i8 = flat && wants_i8(out, b);
        if (st.out_i8) {
          i8_alloc(out);
          has_i8[out] = true;
          safe[out] = true;
          producer_step[out] = (int)plan.size();
        } else {
          has_i32[out] = true;
          safe[out] = FitsI8(b);
          early_i32(out);
        }
        plan.push_back(st);
        done = true;
      }
    } else if (op == "flatten") {
      const uint32_t xe = entry_id(n.inputs[0]);
      if (has_i8[xe] && !is_head[out0] && uses[out0].size() == 1) {
        const Node& c = nodes_[uses[out0][0]];
        const Shape& x = shape_[xe];
        bool to_dense = c.func_name == "dense" && entry_id(c.inputs[0]) == out0;
        for (size_t k = 1; to_dense && k < c.inputs.size(); ++k)
          to_dense = nodes_[c.inputs[k].node_id].is_variable() && !nodes_[c.inputs[k].node_id].is_data();
        if (to_dense && x.size() == 4 && (x[2] > 1 || x[3] > 1) && x[2] <= 64 && x[3] <= 64) {
          fold_src[out0] = xe;  // the dense becomes a convolution over xe
          done = true;
        } else if (to_dense && (x.size() == 2 || (x.size() == 4 && x[2] == 1 && x[3] == 1))) {
          i8_off[out0] = i8_off[xe];  // same bytes, other logical shape
          has_i8[out0] = true;
          safe[out0] = safe[xe];
          producer_step[out0] = producer_step[xe];
          done = true;
        }
      }
    }

    if (done) continue;
    // ---- the node runs as its own int32 kernel
    const std::vector<bool>& placed = in_place[nid];  // concatenate only: inputs already written into the output
    bool all_safe = true, any_left = placed.empty();
    for (size_t k = 0; k < n.inputs.size(); ++k) {
      if (!placed.empty() && placed[k]) {
        execs_[ex].call.in[k].data = nullptr;  // the copy of this input is skipped (cvmhip_concatenate)
        continue;
      }
      need_i32(entry_id(n.inputs[k]));
      all_safe = all_safe && safe[entry_id(n.inputs[k])];
      any_left = true;
    }
    for (bool ok8 : head_safe[out0]) all_safe = all_safe && ok8;
    if (any_left) {
      PlanStep st;
      st.kind = PlanStep::NODE;
      st.label = op;
      st.exec_index = ex;
      plan.push_back(st);
    }
    for (uint32_t i = 0; i < n.num_outputs; ++i) {
      const uint32_t eid = entry_id(nid, i);
      has_i32[eid] = true;
      cvmhip_stage tmp = {};
      Bound b;
      if (ValuePreserving(op)) safe[eid] = all_safe;
      else if (n.inputs.size() == 1 && ChainStage(n, &tmp, &b)) safe[eid] = FitsI8(b);
    }
  }
  for (const NodeEntry& e : outputs_) need_i32(entry_id(e));

  // ---- workspaces of K-sliced launches (layers with a handful of output pixels and a very long K)
  for (PlanStep& st : plan) {
    if (st.kind != PlanStep::CONV || st.stem || st.nhwc) continue;
    // A dense layer over a whole map of at least 64 KiB per image (the first fully connected layer of a VGG) is all filter
    // streaming; gathering its operand from the map costs the stream a quarter of its rate (16 images x 2 halves = 32 cache
    // lines for the 512 useful bytes of a K chunk), so the map is flattened once per run into a tensor whose K chunks are
    // contiguous KiB blocks, and the layer reads that.
    // (from 4 images on: a single image's chunk is two cache lines either way, and the extra launch costs 3 us)
    st.flat = hooks_.flat_dense && st.n >= 4 && st.kh == st.h && st.kw == st.w && st.h * st.w > 1 && st.ph == 0 && st.pw == 0 && st.sh == 1 &&
              st.sw == 1 && st.dh == 1 && st.dw == 1 && (st.c % 32) == 0 && st.src2 == kNone && !st.pool2 &&
              static_cast<int64_t>(st.c) * st.h * st.w >= 8192 && static_cast<int64_t>(st.c) * st.h * st.w < (1 << 24);
    if (st.flat) {
      auto flat = std::make_shared<DeviceBuffer>();
      const size_t fb = cvmhip_packed_act_bytes(st.n, st.c * st.h * st.w);
      Check(cvmhip_alloc(&flat->ptr, fb), "flattened map");
      Check(cvmhip_memset32(flat->ptr, 0, fb / 4, stream_), "flattened map");
      st.aux = flat;
    }
    const size_t bytes = st.flat ? cvmhip_conv2d_i8_workspace_bytes(0, st.n, st.c * st.h * st.w, 1, 1, st.oc, 1, 1, 1, 1, 0, 0, 1, 1)
                                 : cvmhip_conv2d_i8_workspace_bytes(st.src2 != kNone, st.n, st.c, st.h, st.w, st.oc, st.kh, st.kw, st.sh, st.sw,
                                                                    st.ph, st.pw, st.dh, st.dw);
    if (bytes == 0) continue;
    auto buf = std::make_shared<DeviceBuffer>();
    Check(cvmhip_alloc(&buf->ptr, bytes), "K-slice workspace");
    st.ws = buf;
    st.ws_bytes = bytes;
  }

  if (i8_bytes > 0) {
    Check(cvmhip_alloc(&i8_slab_, i8_bytes), "allocate int8 activation storage");
    for (uint32_t e = 0; e < ne; ++e)
      if (i8_off[e] != SIZE_MAX) i8_ptr_[e] = static_cast<char*>(i8_slab_) + i8_off[e];
  }
  plan_ = std::move(plan);
  fused_ = true;
  if (hooks_.fold_bias) FoldRequant();
  if (hooks_.seq) BuildSequences();
  BuildGroups();
}

// The rounding terms of a convolution's requantisation chains move into its bias (one add per channel at load instead
// of one per value in every run), where the bias values and the number of int8 x int8 products prove that nothing
// wraps; CVM_HIP_FOLDBIAS=0 keeps the chains as the graph gives them.
void HipGraphRuntime::FoldRequant() {
  for (PlanStep& st : plan_) {
    const bool conv = st.kind == PlanStep::CONV && !st.pair, dw = st.kind == PlanStep::DWCONV;
    if (!conv && !dw) continue;
    std::vector<int32_t> bias(static_cast<size_t>(st.oc), 0), folded(static_cast<size_t>(st.oc));
    if (st.bias) {
      Check(cvmhip_copy_d2h(bias.data(), st.bias, bias.size() * 4, stream_), "read bias");
      Check(cvmhip_stream_sync(stream_), "read bias");
    }
    const int64_t terms = dw ? static_cast<int64_t>(st.kh) * st.kw : static_cast<int64_t>(st.c) * st.kh * st.kw;
    cvmhip_chain c1{}, c2{};
    const bool residual = conv && st.src2 != kNone;
    if (!cvmhip_fold_requant(st.bias ? bias.data() : nullptr, st.oc, terms * 128 * 128, &st.chain, &st.chain2, residual ? 1 : 0,
                             folded.data(), &c1, &c2))
      continue;
    auto buf = std::make_shared<DeviceBuffer>();
    Check(cvmhip_alloc(&buf->ptr, folded.size() * 4), "folded bias");
    Check(cvmhip_copy_h2d(buf->ptr, folded.data(), folded.size() * 4, stream_), "folded bias");
    Check(cvmhip_stream_sync(stream_), "folded bias");   // the host copy goes away
    st.folded_bias = buf;
    st.bias = static_cast<const int32_t*>(buf->ptr);
    st.chain = c1;
    if (residual) st.chain2 = c2;
  }
}

// Runs of at least three consecutive convolution steps that a layer-sequence launch can take (batch a multiple
// of 8, int8 in and out, channels padded to 32, no K slices) become one launch each.  Consecutive plan steps
// only depend on earlier ones, which is all a sequence needs.
void HipGraphRuntime::BuildSequences() {
  seq_at_.assign(plan_.size(), -1);
  const size_t entry = cvmhip_conv_seq_layer_bytes();
  std::vector<char> table;
  size_t i = 0;
  while (i < plan_.size()) {
    table.clear();
    size_t j = i;
    for (; j < plan_.size(); ++j) {
      const PlanStep& st = plan_[j];
      if (st.kind != PlanStep::CONV || st.stem || st.nhwc || st.ws || st.flat || !st.out_i8 || st.pool2) break;
      table.resize((j - i + 1) * entry);
      const void* res = st.src2 == kNone ? nullptr : i8_ptr_[st.src2];
      const int rc = cvmhip_conv_seq_layer(table.data(), static_cast<int>(j - i), i8_ptr_[st.src],
                                           static_cast<DeviceBuffer*>(st.weights.get())->ptr, st.bias, &st.chain, res, &st.chain2,
                                           i8_ptr_[st.dst], st.n, st.c, st.h, st.w, st.oc, st.kh, st.kw, st.sh, st.sw, st.ph,
                                           st.pw, st.dh, st.dw);
      if (rc != CVMHIP_OK) break;
    }
    const size_t count = j - i;
    if (count >= 3) {
      cvmhip_conv_seq_link(table.data(), static_cast<int>(count));
      auto buf = std::make_shared<DeviceBuffer>();
      Check(cvmhip_alloc(&buf->ptr, count * entry), "layer-sequence table");
      Check(cvmhip_copy_h2d(buf->ptr, table.data(), count * entry, stream_), "layer-sequence table");
      Check(cvmhip_stream_sync(stream_), "layer-sequence table");   // the host copy goes away
      SeqRun r;
      r.first = i;
      r.last = j - 1;
      r.owner = buf;
      r.table = buf->ptr;
      r.nlayers = static_cast<int>(count);
      for (size_t k = i; k < j; ++k) {
        const PlanStep& st = plan_[k];
        const int oh = (st.h + 2 * st.ph - (st.dh * (st.kh - 1) + 1)) / st.sh + 1, ow = (st.w + 2 * st.pw - (st.dw * (st.kw - 1) + 1)) / st.sw + 1;
        const double px = static_cast<double>(st.n) * oh * ow;
        r.ops += 2.0 * px * st.oc * st.c * st.kh * st.kw;
        r.bytes += static_cast<double>(st.n) * st.h * st.w * st.c + static_cast<double>(st.oc) * st.c * st.kh * st.kw +
                   px * st.oc * (st.src2 != kNone ? 2.0 : 1.0);
      }
      for (size_t k = 0; k < count; ++k) r.cfgs.push_back(cvmhip_conv_seq_layer_config(table.data(), static_cast<int>(k)));
      seq_at_[i] = static_cast<int>(seqs_.size());
      seqs_.push_back(r);
    }
    i = j > i ? j : i + 1;
  }
  if (seqs_.empty()) return;
  // a second model with sequence launches: what the first one has in flight is drained once
  if (CountSequenceModel(+1) > 1) Check(cvmhip_device_sync(), "drain the device");
  seq_counted_ = true;
  const size_t words = cvmhip_conv_seq_sync_bytes() / 4;
  Check(cvmhip_alloc(&seq_sync_, words * 4), "layer-sequence counters");
  Check(cvmhip_memset32(seq_sync_, 0, words, stream_), "layer-sequence counters");
  void* host = nullptr;
  Check(cvmhip_host_alloc(&host, 64), "layer-sequence status");
  seq_error_host_ = static_cast<uint32_t*>(host);
  use_seq_ = true;
}

// Consecutive detection-head steps read feature maps and write slices of concatenated tensors, never one another's
// results, and each is a few workgroups: two or more of them become one launch of independent convolutions.
void HipGraphRuntime::BuildGroups() {
  group_at_.assign(plan_.size(), -1);
  const size_t entry = cvmhip_conv_group_layer_bytes();
  std::vector<char> table;
  size_t i = 0;
  while (i < plan_.size()) {
    table.clear();
    int blocks = 0;
    double ops = 0, bytes = 0;
    size_t j = i;
    for (; j < plan_.size(); ++j) {
      const PlanStep& st = plan_[j];
      if (st.kind != PlanStep::CONV || !st.nhwc || st.stem) break;
      table.resize((j - i + 1) * entry);
      int nb = 0;
      const int32_t* bias = st.pair ? static_cast<const int32_t*>(static_cast<DeviceBuffer*>(st.pair_bias.get())->ptr) : st.bias;
      const int rc = cvmhip_conv_group_heads(table.data(), static_cast<int>(j - i), blocks, &nb, i8_ptr_[st.src],
                                             static_cast<DeviceBuffer*>(st.weights.get())->ptr, bias, &st.chain,
                                             entry_ptr_[st.dst] + st.dst_off, st.img_stride, st.oc,
                                             st.pair ? entry_ptr_[st.dst2] + st.dst_off2 : nullptr, st.img_stride2, st.oc2, st.n, st.c,
                                             st.h, st.w, st.kh, st.kw, st.sh, st.sw, st.ph, st.pw, st.dh, st.dw);
      if (rc != CVMHIP_OK) break;
      blocks += nb;
      const int oh = (st.h + 2 * st.ph - (st.dh * (st.kh - 1) + 1)) / st.sh + 1, ow = (st.w + 2 * st.pw - (st.dw * (st.kw - 1) + 1)) / st.sw + 1;
      const double px = static_cast<double>(st.n) * oh * ow, oc = st.oc + (st.pair ? st.oc2 : 0);
      ops += 2.0 * px * oc * st.c * st.kh * st.kw;
      bytes += static_cast<double>(st.n) * st.h * st.w * st.c + oc * st.c * st.kh * st.kw + 4.0 * px * oc;
    }
    const size_t count = j - i;
    if (count >= 2) {
      auto buf = std::make_shared<DeviceBuffer>();
      Check(cvmhip_alloc(&buf->ptr, count * entry), "grouped-heads table");
      Check(cvmhip_copy_h2d(buf->ptr, table.data(), count * entry, stream_), "grouped-heads table");
      Check(cvmhip_stream_sync(stream_), "grouped-heads table");   // the host copy goes away
      GroupRun r;
      r.first = i;
      r.last = j - 1;
      r.owner = buf;
      r.table = buf->ptr;
      r.nlayers = static_cast<int>(count);
      r.blocks = blocks;
      r.ops = ops;
      r.bytes = bytes;
      group_at_[i] = static_cast<int>(groups_.size());
      groups_.push_back(r);
    }
    i = j > i ? j : i + 1;
  }
  if (!hooks_.head_group) { groups_.clear(); group_at_.assign(plan_.size(), -1); }
  // The same for consecutive convolutions with int8 output that do not read one another's results (at a small batch the
  // first 1x1 layer and the shortcut projection of a ResNet block, which the planner has put side by side), as long as
  // all of them together are one round of workgroups (two per CU).  They are what runs when the model's sequence
  // launches are not in use (Launch() takes a sequence launch first where both exist).
  if (!hooks_.conv_group) return;
  i = 0;
  while (i < plan_.size()) {
    table.clear();
    int blocks = 0;
    double ops = 0, bytes = 0;
    std::vector<uint32_t> written;
    size_t j = i;
    for (; j < plan_.size(); ++j) {
      const PlanStep& st = plan_[j];
      if (st.kind != PlanStep::CONV || st.stem || st.nhwc || st.ws || st.flat || !st.out_i8 || st.pool2 || group_at_[j] >= 0) break;
      bool reads_member = false;
      for (uint32_t w : written) reads_member = reads_member || st.src == w || st.src2 == w;
      if (reads_member) break;
      table.resize((j - i + 1) * entry);
      int nb = 0;
      const void* res = st.src2 == kNone ? nullptr : i8_ptr_[st.src2];
      const int rc = cvmhip_conv_group_conv_i8(table.data(), static_cast<int>(j - i), blocks, &nb, i8_ptr_[st.src],
                                               static_cast<DeviceBuffer*>(st.weights.get())->ptr, st.bias, &st.chain, res, &st.chain2,
                                               i8_ptr_[st.dst], st.n, st.c, st.h, st.w, st.oc, st.kh, st.kw, st.sh, st.sw, st.ph, st.pw,
                                               st.dh, st.dw);
      if (rc != CVMHIP_OK || blocks + nb > 512) break;
      blocks += nb;
      written.push_back(st.dst);
      const int oh = (st.h + 2 * st.ph - (st.dh * (st.kh - 1) + 1)) / st.sh + 1, ow = (st.w + 2 * st.pw - (st.dw * (st.kw - 1) + 1)) / st.sw + 1;
      const double px = static_cast<double>(st.n) * oh * ow;
      ops += 2.0 * px * st.oc * st.c * st.kh * st.kw;
      bytes += static_cast<double>(st.n) * st.h * st.w * st.c + static_cast<double>(st.oc) * st.c * st.kh * st.kw +
               px * st.oc * (st.src2 != kNone ? 2.0 : 1.0);
    }
    const size_t count = j - i;
    if (count >= 2) {
      auto buf = std::make_shared<DeviceBuffer>();
      Check(cvmhip_alloc(&buf->ptr, count * entry), "grouped-convolutions table");
      Check(cvmhip_copy_h2d(buf->ptr, table.data(), count * entry, stream_), "grouped-convolutions table");
      Check(cvmhip_stream_sync(stream_), "grouped-convolutions table");
      GroupRun r;
      r.first = i;
      r.last = j - 1;
      r.owner = buf;
      r.table = buf->ptr;
      r.nlayers = static_cast<int>(count);
      r.blocks = blocks;
      r.i8 = true;
      r.ops = ops;
      r.bytes = bytes;
      group_at_[i] = static_cast<int>(groups_.size());
      groups_.push_back(r);
      i = j;
    } else {
      i = i + 1;
    }
  }
}

void HipGraphRuntime::RunStep(PlanStep& st) {
  switch (st.kind) {
    case PlanStep::NODE: {
      Exec& ex = execs_[st.exec_index];
      ex.kernel->run(ex.call);
      break;
    }
    case PlanStep::PACK:
      Check(cvmhip_pack_nhwc_i8(entry_ptr_[st.src], i8_ptr_[st.dst], st.n, st.c, st.h, stream_), "pack");
      break;
    case PlanStep::UNPACK:
      Check(cvmhip_unpack_nhwc_i8(i8_ptr_[st.src], entry_ptr_[st.dst], st.n, st.c, st.h, stream_), "unpack");
      break;
    case PlanStep::STEMPACK:
      Check(cvmhip_pack_stem_input(entry_ptr_[st.src], static_cast<DeviceBuffer*>(st.aux.get())->ptr, st.n, st.c, st.h, st.w,
                                   st.kh, st.kw, st.sh, st.sw, st.ph, st.pw, stream_), "pack_stem_input");
      break;
    case PlanStep::CONV: {
      void* out = st.out_i8 ? i8_ptr_[st.dst] : static_cast<void*>(entry_ptr_[st.dst]);
      if (st.stem && st.pool3) {
        Check(cvmhip_conv2d_stem_pool3_i8(static_cast<DeviceBuffer*>(st.aux.get())->ptr, static_cast<DeviceBuffer*>(st.weights.get())->ptr,
                                          st.bias, &st.chain, out, st.n, st.c, st.h, st.w, st.oc, st.kh, st.kw, st.sh, st.sw, st.ph,
                                          st.pw, st.oh, st.ow, stream_), "conv2d_stem_pool3_i8");
        break;
      }
      if (st.stem) {
        Check(cvmhip_conv2d_stem_i8(static_cast<DeviceBuffer*>(st.aux.get())->ptr, static_cast<DeviceBuffer*>(st.weights.get())->ptr,
                                    st.bias, &st.chain, out, st.out_i8 ? 1 : 0, st.n, st.c, st.h, st.w, st.oc, st.kh, st.kw,
                                    st.sh, st.sw, st.ph, st.pw, stream_), "conv2d_stem_i8");
        break;
      }
      if (st.nhwc && st.pair) {
        Check(cvmhip_conv2d_i8_nhwc_pair(i8_ptr_[st.src], static_cast<DeviceBuffer*>(st.weights.get())->ptr,
                                         static_cast<const int32_t*>(static_cast<DeviceBuffer*>(st.pair_bias.get())->ptr), &st.chain,
                                         entry_ptr_[st.dst] + st.dst_off, st.img_stride, st.oc, entry_ptr_[st.dst2] + st.dst_off2,
                                         st.img_stride2, st.oc2, st.n, st.c, st.h, st.w, st.kh, st.kw, st.sh, st.sw, st.ph, st.pw,
                                         st.dh, st.dw, stream_), "conv2d_i8_nhwc_pair");
        break;
      }
      if (st.nhwc) {
        Check(cvmhip_conv2d_i8_nhwc(i8_ptr_[st.src], static_cast<DeviceBuffer*>(st.weights.get())->ptr, st.bias, &st.chain,
                                    entry_ptr_[st.dst] + st.dst_off, st.img_stride, st.n, st.c, st.h, st.w, st.oc, st.kh,
                                    st.kw, st.sh, st.sw, st.ph, st.pw, st.dh, st.dw, stream_), "conv2d_i8_nhwc");
        break;
      }
      if (st.pool2) {
        Check(cvmhip_conv2d_pool2_i8(i8_ptr_[st.src], static_cast<DeviceBuffer*>(st.weights.get())->ptr, st.bias, &st.chain, out,
                                     st.n, st.c, st.h, st.w, st.oc, st.kh, st.kw, st.sh, st.sw, st.ph, st.pw, st.dh, st.dw,
                                     stream_), "conv2d_pool2_i8");
        break;
      }
      if (st.flat) {
        void* flat = static_cast<DeviceBuffer*>(st.aux.get())->ptr;
        Check(cvmhip_flatten_act_i8(i8_ptr_[st.src], flat, st.n, st.c, st.h * st.w, stream_), "flatten_act_i8");
        Check(cvmhip_conv2d_i8_ws(flat, static_cast<DeviceBuffer*>(st.weights.get())->ptr, st.bias, &st.chain, nullptr, &st.chain2, out,
                                  st.out_i8 ? 1 : 0, st.n, st.c * st.h * st.w, 1, 1, st.oc, 1, 1, 1, 1, 0, 0, 1, 1,
                                  st.ws ? static_cast<DeviceBuffer*>(st.ws.get())->ptr : nullptr, st.ws_bytes, stream_), "conv2d_i8 (flattened map)");
        break;
      }
      const void* res = st.src2 == kNone ? nullptr : i8_ptr_[st.src2];
      Check(cvmhip_conv2d_i8_ws(i8_ptr_[st.src], static_cast<DeviceBuffer*>(st.weights.get())->ptr, st.bias, &st.chain, res,
                                &st.chain2, out, st.out_i8 ? 1 : 0, st.n, st.c, st.h, st.w, st.oc, st.kh, st.kw, st.sh,
                                st.sw, st.ph, st.pw, st.dh, st.dw, st.ws ? static_cast<DeviceBuffer*>(st.ws.get())->ptr : nullptr,
                                st.ws_bytes, stream_), "conv2d_i8");
      break;
    }
    case PlanStep::DWCONV: {
      void* out = st.out_i8 ? i8_ptr_[st.dst] : static_cast<void*>(entry_ptr_[st.dst]);
      if (st.dw_mfma) {
        Check(cvmhip_depthwise_conv2d_mfma_i8(i8_ptr_[st.src], static_cast<DeviceBuffer*>(st.weights.get())->ptr, st.bias,
                                              &st.chain, out, st.out_i8 ? 1 : 0, st.n, st.c, st.h, st.w, st.kh, st.kw,
                                              st.sh, st.sw, st.ph, st.pw, st.dh, st.dw, stream_), "depthwise_conv2d_mfma_i8");
        break;
      }
      Check(cvmhip_depthwise_conv2d_i8(i8_ptr_[st.src], static_cast<DeviceBuffer*>(st.weights.get())->ptr, st.bias,
                                       &st.chain, out, st.out_i8 ? 1 : 0, st.n, st.c, st.h, st.w, st.kh, st.kw, st.sh,
                                       st.sw, st.ph, st.pw, st.dh, st.dw, stream_), "depthwise_conv2d_i8");
      break;
    }
    case PlanStep::ADD: {
      void* out = st.out_i8 ? i8_ptr_[st.dst] : static_cast<void*>(entry_ptr_[st.dst]);
      Check(cvmhip_add_i8(i8_ptr_[st.src], i8_ptr_[st.src2], &st.chain, out, st.out_i8 ? 1 : 0, st.n, st.c, st.h, stream_), "add_i8");
      break;
    }
    case PlanStep::POOL:
      Check(cvmhip_max_pool2d_i8(i8_ptr_[st.src], i8_ptr_[st.dst], st.n, st.c, st.h, st.w, st.oh, st.ow, st.kh, st.kw,
                                 st.sh, st.sw, st.ph, st.pw, stream_), "max_pool2d_i8");
      break;
    case PlanStep::SUM: {
      void* out = st.out_i8 ? i8_ptr_[st.dst] : static_cast<void*>(entry_ptr_[st.dst]);
      Check(cvmhip_sum_hw_i8(i8_ptr_[st.src], &st.chain, out, st.out_i8 ? 1 : 0, st.n, st.c, st.h, stream_), "sum_hw_i8");
      break;
    }
  }
}

}  // namespace cvmrt
