// Graph builder, precision planner and executor of the SCN engine, plus the ONNX loader.
//
// Mirrors the builder / engine surface of the reference
// (libraries/3DSparseConvolution/libspconv/include/spconv/engine.hpp:38-167) behind the C ABI and
// what its loader does with a model file (libraries/3DSparseConvolution/src/onnx-parser.cpp:101-231).
//
// Execution model: build() turns the node list into a flat list of steps (hash build, rulebook
// build, conversion, convolution with fused epilogue, add, relu, dense scatter).  forward() only
// enqueues kernels on the caller's stream: row counts live in device memory, launch sizes come from
// host-side bounds, nothing is allocated after the first call with a given grid size.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <fstream>
#include <functional>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "scn_conv_args.hpp"
#include "scn_kernels.hpp"

namespace scn {

enum class Op { Conv, Add, Relu, Dense, Reshape, Transpose };

static const char* op_name(Op op) {
  switch (op) {
    case Op::Conv: return "SparseConvolution";
    case Op::Add: return "Add";
    case Op::Relu: return "Relu";
    case Op::Dense: return "ScatterDense";
    case Op::Reshape: return "Reshape";
    case Op::Transpose: return "Transpose";
  }
  return "?";
}

struct NodeDesc {
  Op op;
  std::string name;
  std::vector<int> in;
  int out = -1;
  // conv
  std::vector<uint16_t> weight;
  int wshape[5] = {0, 0, 0, 0, 0};
  std::vector<float> wranges;
  std::vector<uint16_t> bias;
  std::string activation;
  int ks[3] = {1, 1, 1}, stride[3] = {1, 1, 1}, pad[3] = {0, 0, 0}, dil[3] = {1, 1, 1};
  float in_range = 0.f;
  bool subm = false;
  bool inverse = false;
  uint32_t max_out = 150000;
  uint32_t fixed_launch_points = 0;
  std::string rulebook;
  int precision = SCN_PRECISION_FP16, out_precision = SCN_PRECISION_FP16;
  // add
  float a_range = 0.f, b_range = 0.f;
  // dense
  std::string format;
  int in_spatial[3] = {0, 0, 0};
  std::vector<int> out_shape;
  float dense_range = 0.f;
  int layout = 1;  // spconv::TensorLayout: 1 NCHW, 2 NCHW32, 3 NHWzC
  // reshape / transpose
  std::vector<int64_t> dims;
};

struct TensorDesc {
  std::string name;
  int producer = -1;  // node index, -1 for graph inputs
};

}  // namespace scn

using namespace scn;

struct scn_builder {
  std::vector<TensorDesc> tensors;
  std::vector<NodeDesc> nodes;
  std::vector<int> inputs, outputs;
  int new_tensor(const char* name, int producer) {
    TensorDesc t;
    t.name = name ? name : "";
    t.producer = producer;
    tensors.push_back(t);
    return (int)tensors.size() - 1;
  }
  bool valid_tensor(int t) const { return t >= 0 && t < (int)tensors.size(); }
};

namespace scn {

// ---------------------------------------------------------------------------------------------
// runtime objects
// ---------------------------------------------------------------------------------------------
struct CoordSet {
  const int32_t* idx = nullptr;
  const uint32_t* n_dev = nullptr;
  uint32_t n_bound = 0;  // host-side bound of the row count for the current forward
  uint32_t cap = 0;      // allocated rows
  int grid[3] = {0, 0, 0};
  CoordLookup lookup;                 // row look-up of these coordinates (valid once has_lookup is set in a forward)
  bool has_lookup = false;
  CoordTable own_table;               // only for graph inputs
  int producer_rulebook = -1;         // strided rulebook that creates this set (-1: graph input)
};

struct RtTensor {
  bool dense = false;
  int dtype = SCN_DTYPE_FP16;
  float range = 0.f;   // int8: dynamic range (amax); value = q * (range / 127)
  int c = 0;           // logical channels
  uint32_t ld = 0;     // row stride in elements
  int coord = -1;      // CoordSet index (sparse)
  DevBuf buf;          // owned storage (not for graph inputs / views)
  void* data = nullptr;
  DevBuf acc;          // raw accumulators (keep-all mode)
  std::vector<int64_t> shape;  // dense
  bool fixed_form = false;     // dense tensor in a vectorised layout: a following Reshape keeps this shape
  int view_of = -1;    // dense view of another tensor (reshape / fused transpose)
  bool materialised = false;  // false: fused away, never written
  bool shared = false;        // storage shared with tensors of disjoint lifetimes: holds this tensor's values only
                              // between the step that writes it and the last step that reads it
};

enum class StepKind { InputCount, HashBuild, RulebookSubm, RulebookSparse, RulebookInverse, Convert, Conv, Add, Relu, Dense, Permute };

struct Step {
  StepKind kind;
  int node = -1;       // graph node this step belongs to (for profiling names)
  std::string label;
  // generic operands
  int t_in = -1, t_in2 = -1, t_out = -1;
  int coord = -1, coord_out = -1;
  int rulebook = -1;
  int conv = -1;
  // convert
  int cv_dtype = 0;
  float cv_range = 0.f;
  uint32_t cv_c = 0;
  int relu = 0;
  // conv epilogue
  float x_range = 0.f;
  bool fused_add = false;
  int mid_dtype = 0;
  float mid_range = 0.f, a_rq = 0.f, b_rq = 0.f;  // dynamic ranges
  int relu2 = 0;
  bool conv_input_is_converted = false;
  int t_conv_in = -1;  // tensor or conversion buffer index actually read
  // add
  float add_a_rq = 0.f, add_b_rq = 0.f;
  // dense
  int dense_shape[5] = {1, 0, 0, 0, 0};
  int perm[5] = {0, 1, 2, 3, 4};
  bool has_perm = false;
  bool form = false;           // int8 output or a vectorised layout: scatter_dense_form
  int form_layout = 1, zaxis = 0;
  // profiling
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  float last_ms = 0.f;
};

struct RbSlot {
  Rulebook rb;
  bool subm = false;
  int coord_in = -1, coord_out = -1;
  int ks[3], stride[3], pad[3], dil[3];
  uint32_t max_out = 0;
  int inverse_of = -1;   // >= 0: the strided rulebook this one swaps (SparseInverseConvolution)
  bool initialised = false;
  bool want_plan = false;   // some convolution on this rulebook runs the tile-plan kernel
  bool plan_sorted = false; // ... with the rows sorted by their offset sets (SCN_BUILD_TILE_PLANS)
};

}  // namespace scn

struct scn_engine {
  std::vector<NodeDesc> nodes;
  std::vector<TensorDesc> tdesc;
  std::vector<int> inputs, outputs;
  int precision = SCN_PRECISION_FP16;
  unsigned flags = 0;
  std::vector<RtTensor> tensors;      // graph tensors followed by conversion buffers
  std::vector<CoordSet> coords;
  std::vector<std::unique_ptr<RbSlot>> rulebooks;
  std::vector<std::unique_ptr<ConvWeights>> convs;
  std::vector<Step> steps;
  std::vector<char> dense_precleared;  // per step: the forward's batched fill zeroed its dense output (1) or reset its row map (2)
  DevBuf amax_buf;                     // collect_amax: one 16-byte slot per tensor
  bool dense_map_built = false;        // the step about to run had its row map built on the auxiliary stream
  std::vector<DevBuf> dense_maps;      // per step: cell -> row map of a ScatterDense whose layout allows the dense-major pass
  std::vector<DevBuf> arena;           // storage shared by sparse tensors whose lifetimes do not overlap
  std::map<std::string, int> tensor_by_name;
  // input binding
  const void* in_feat = nullptr;
  const int32_t* in_idx = nullptr;
  uint32_t in_n = 0, in_c = 0;
  int in_grid[3] = {0, 0, 0};
  const uint32_t* dds = nullptr;
  DevBuf in_count;   // device uint32 holding N when no DDS pointer is bound
  uint32_t input_cap = 0;
  bool allocated = false;
  int alloc_grid[3] = {0, 0, 0};
  bool profiling = false;
  bool input_set = false;
  // SCN_BUILD_AUX_STREAM: hash and rulebook construction depend on coordinates only, so they run on a
  // second stream ahead of the convolutions; a convolution waits for its rulebook's event.
  hipStream_t aux = nullptr;
  hipEvent_t ev_fork = nullptr, ev_join = nullptr;
  std::vector<hipEvent_t> rb_ready;   // per rulebook
  std::vector<int> rb_seq;            // per rulebook: position in the auxiliary stream's order (this forward)
  std::vector<int> coord_rb;          // per coordinate set: rulebook that produced it (-1: graph input)
  std::vector<char> map_built;        // per step: the dense output's row map was built on the auxiliary stream
  ~scn_engine() {
    for (auto& s : steps) {
      if (s.ev0) (void)hipEventDestroy(s.ev0);
      if (s.ev1) (void)hipEventDestroy(s.ev1);
    }
    for (auto ev : rb_ready)
      if (ev) (void)hipEventDestroy(ev);
    if (ev_fork) (void)hipEventDestroy(ev_fork);
    if (ev_join) (void)hipEventDestroy(ev_join);
    if (aux) (void)hipStreamDestroy(aux);
  }
};

namespace scn {

// ---------------------------------------------------------------------------------------------
// planning
// ---------------------------------------------------------------------------------------------
struct Plan {
  std::vector<int> comp, outp;             // per node effective precisions
  std::vector<float> range;                // per tensor dynamic range, <= 0 when no consumer fixes one
  std::vector<std::vector<std::pair<int, int>>> consumers;  // per tensor: (node, slot)
};

static Plan make_plan(const std::vector<NodeDesc>& nodes, size_t ntensors, int engine_precision) {
  Plan p;
  p.comp.assign(nodes.size(), SCN_PRECISION_FP16);
  p.outp.assign(nodes.size(), SCN_PRECISION_FP16);
  p.consumers.resize(ntensors);
  for (size_t i = 0; i < nodes.size(); ++i) {
    const NodeDesc& n = nodes[i];
    for (size_t s = 0; s < n.in.size(); ++s) p.consumers[n.in[s]].push_back({(int)i, (int)s});
    if (engine_precision != SCN_PRECISION_INT8) {
      if ((n.op == Op::Conv || n.op == Op::Add) && n.precision == SCN_PRECISION_INT8)
        SCN_LOGV("Ignore the layer[%s] precision[int8] because the model precision configured fp16", n.name.c_str());
      continue;
    }
    if (n.op == Op::Conv) {
      const bool ok = n.in_range > 0.f && (int)n.wranges.size() == n.wshape[0];
      p.comp[i] = (n.precision == SCN_PRECISION_INT8 && ok) ? SCN_PRECISION_INT8 : SCN_PRECISION_FP16;
      p.outp[i] = n.out_precision == SCN_PRECISION_INT8 ? SCN_PRECISION_INT8 : SCN_PRECISION_FP16;
    } else if (n.op == Op::Add) {
      const bool ok = n.a_range > 0.f && n.b_range > 0.f;
      p.comp[i] = (n.precision == SCN_PRECISION_INT8 && ok) ? SCN_PRECISION_INT8 : SCN_PRECISION_FP16;
      p.outp[i] = n.out_precision == SCN_PRECISION_INT8 ? SCN_PRECISION_INT8 : SCN_PRECISION_FP16;
    }
  }
  // dynamic range of a tensor = what its consumers expect: int8 conv first, then through Relu, then int8 Add,
  // then an int8 ScatterDense range.
  p.range.assign(ntensors, -1.f);
  std::vector<int> state(ntensors, 0);
  std::function<float(int)> req = [&](int t) -> float {
    if (state[t]) return p.range[t];
    state[t] = 1;
    float res = -1.f;
    for (auto& c : p.consumers[t]) {
      const NodeDesc& n = nodes[c.first];
      if (n.op == Op::Conv && p.comp[c.first] == SCN_PRECISION_INT8) {
        res = n.in_range;
        break;
      }
    }
    if (res <= 0.f)
      for (auto& c : p.consumers[t]) {
        const NodeDesc& n = nodes[c.first];
        if (n.op == Op::Relu) {
          res = req(n.out);
          if (res > 0.f) break;
        }
      }
    if (res <= 0.f)
      for (auto& c : p.consumers[t]) {
        const NodeDesc& n = nodes[c.first];
        if (n.op == Op::Add && p.comp[c.first] == SCN_PRECISION_INT8) {
          res = c.second == 0 ? n.a_range : n.b_range;
          break;
        }
      }
    if (res <= 0.f)
      for (auto& c : p.consumers[t]) {
        const NodeDesc& n = nodes[c.first];
        if (n.op == Op::Dense && n.dense_range > 0.f) {
          res = n.dense_range;
          break;
        }
      }
    p.range[t] = res;
    return res;
  };
  for (size_t t = 0; t < ntensors; ++t) req((int)t);
  return p;
}

static uint32_t round_up(uint32_t v, uint32_t m) { return (v + m - 1) / m * m; }

// ---------------------------------------------------------------------------------------------
// build
// ---------------------------------------------------------------------------------------------
static bool build_engine(scn_engine& e) {
  const auto& nodes = e.nodes;
  const size_t nt = e.tdesc.size();
  const bool keep_all = (e.flags & SCN_BUILD_KEEP_ALL) != 0;
  Plan plan = make_plan(nodes, nt, e.precision);
  e.tensors.reserve(nt + 2 * nodes.size() + 8);  // conversion buffers are appended; references stay valid
  e.tensors.resize(nt);
  std::set<int> graph_outputs(e.outputs.begin(), e.outputs.end());
  if (e.inputs.size() != 1) {
    set_error("the engine supports exactly one sparse input (got %zu)", e.inputs.size());
    return false;
  }
  // ---- graph input
  const int tin = e.inputs[0];
  {
    e.coords.emplace_back();
    RtTensor& t = e.tensors[tin];
    t.coord = 0;
    t.dtype = SCN_DTYPE_FP16;
    t.materialised = true;
    // capacity of the input = output bound of its first convolution consumer
    uint32_t cap = 0;
    for (auto& c : plan.consumers[tin])
      if (nodes[c.first].op == Op::Conv) cap = std::max(cap, nodes[c.first].max_out);
    if (cap == 0) cap = 150000;
    e.input_cap = cap;
    e.coords[0].cap = cap;
  }
  Step s0;
  s0.kind = StepKind::InputCount;
  s0.label = "input";
  e.steps.push_back(s0);

  std::map<std::string, int> rb_by_key;
  std::map<std::string, int> conversions;  // (tensor, dtype, scale, c) -> conversion buffer tensor
  std::vector<bool> fused_away(nodes.size(), false);

  auto ensure_table = [&](int coord, int node) {
    // graph-input coordinates need an explicit hash build; strided outputs get theirs from the rulebook
    CoordSet& cs = e.coords[coord];
    if (cs.producer_rulebook >= 0) return;
    for (auto& st : e.steps)
      if (st.kind == StepKind::HashBuild && st.coord == coord) return;
    Step st;
    st.kind = StepKind::HashBuild;
    st.coord = coord;
    st.node = node;
    st.label = "hash(input)";
    e.steps.push_back(st);
  };

  auto single_consumer = [&](int t) -> int {
    if (graph_outputs.count(t) || plan.consumers[t].size() != 1) return -1;
    return plan.consumers[t][0].first;
  };

  for (size_t i = 0; i < nodes.size(); ++i) {
    if (fused_away[i]) continue;
    const NodeDesc& n = nodes[i];
    switch (n.op) {
      case Op::Conv: {
        RtTensor& x = e.tensors[n.in[0]];
        if (x.dense || x.coord < 0) {
          set_error("node %s: input is not a sparse tensor", n.name.c_str());
          return false;
        }
        const int cout = n.wshape[0], cin = n.wshape[4];
        if (x.c == 0) x.c = cin;  // graph input: channel count comes from its first consumer
        if (x.c != cin) {
          set_error("node %s: input has %d channels, weight expects %d", n.name.c_str(), x.c, cin);
          return false;
        }
        // rulebook
        const std::string key =
            n.rulebook.empty() ? "" : std::string(n.inverse ? "inv:" : n.subm ? "subm:" : "conv:") + n.rulebook;
        int rbi = -1;
        if (n.inverse) {
          const auto fw = rb_by_key.find("conv:" + n.rulebook);
          if (fw == rb_by_key.end() || e.rulebooks[fw->second]->coord_out != x.coord) {
            set_error("node %s: inverse convolution needs the rulebook '%s' of an earlier strided convolution whose "
                      "output it runs on", n.name.c_str(), n.rulebook.c_str());
            return false;
          }
          const RbSlot& fs = *e.rulebooks[fw->second];
          if (memcmp(fs.ks, n.ks, 12) != 0) {
            set_error("node %s: kernel size differs from that of rulebook '%s'", n.name.c_str(), n.rulebook.c_str());
            return false;
          }
          if (rb_by_key.count(key)) {
            rbi = rb_by_key[key];
          } else {
            auto slot = std::make_unique<RbSlot>();
            slot->subm = false;
            slot->inverse_of = fw->second;
            slot->coord_in = x.coord;
            slot->coord_out = fs.coord_in;
            memcpy(slot->ks, fs.ks, 12);
            memcpy(slot->stride, fs.stride, 12);
            memcpy(slot->pad, fs.pad, 12);
            memcpy(slot->dil, fs.dil, 12);
            rbi = (int)e.rulebooks.size();
            e.rulebooks.push_back(std::move(slot));
            rb_by_key[key] = rbi;
            Step st;
            st.kind = StepKind::RulebookInverse;
            st.rulebook = rbi;
            st.coord = x.coord;
            st.coord_out = e.rulebooks[rbi]->coord_out;
            st.node = (int)i;
            st.label = std::string("rulebook(inverse ") + n.rulebook + ")";
            e.steps.push_back(st);
          }
        } else if (!key.empty() && rb_by_key.count(key)) {
          rbi = rb_by_key[key];
          RbSlot& slot = *e.rulebooks[rbi];
          const bool same = slot.coord_in == x.coord && !memcmp(slot.ks, n.ks, 12) && !memcmp(slot.dil, n.dil, 12) &&
                            (slot.subm || (!memcmp(slot.stride, n.stride, 12) && !memcmp(slot.pad, n.pad, 12)));
          if (!same) {
            SCN_LOGW("node %s: rulebook '%s' is shared with a different geometry or input; building a private one",
                     n.name.c_str(), n.rulebook.c_str());
            rbi = -1;
          }
        }
        if (rbi < 0) {
          ensure_table(x.coord, (int)i);
          auto slot = std::make_unique<RbSlot>();
          slot->subm = n.subm;
          slot->coord_in = x.coord;
          memcpy(slot->ks, n.ks, 12);
          memcpy(slot->stride, n.stride, 12);
          memcpy(slot->pad, n.pad, 12);
          memcpy(slot->dil, n.dil, 12);
          slot->max_out = n.max_out;
          rbi = (int)e.rulebooks.size();
          if (n.subm) {
            slot->coord_out = x.coord;
          } else {
            e.coords.emplace_back();
            CoordSet& oc = e.coords.back();
            oc.cap = n.max_out;
            oc.producer_rulebook = rbi;
            slot->coord_out = (int)e.coords.size() - 1;
          }
          e.rulebooks.push_back(std::move(slot));
          if (!key.empty() && !rb_by_key.count(key)) rb_by_key[key] = rbi;
          Step st;
          st.kind = n.subm ? StepKind::RulebookSubm : StepKind::RulebookSparse;
          st.rulebook = rbi;
          st.coord = x.coord;
          st.coord_out = e.rulebooks[rbi]->coord_out;
          st.node = (int)i;
          st.label = std::string("rulebook(") + (n.rulebook.empty() ? n.name : n.rulebook) + ")";
          e.steps.push_back(st);
        }
        RbSlot& slot = *e.rulebooks[rbi];
        // weights
        auto w = std::make_unique<ConvWeights>();
        const int comp = plan.comp[i];
        if (!w->init(n.weight.data(), n.wshape, comp == SCN_PRECISION_INT8 ? n.wranges.data() : nullptr,
                     n.bias.empty() ? nullptr : n.bias.data(), comp))
          return false;
        const int ci = (int)e.convs.size();
        // Tile plans: the narrow layers run the tile-plan kernel on rows sorted by offset set inside 1024-row windows.
        // Built only on request (SCN_BUILD_TILE_PLANS).  The reference's sortmask flag is a hint to skip more empty
        // work where that is faster, and on this GPU it is faster nowhere: measured on a 123,646-voxel frame, plans
        // cost the first four rulebooks 30 .. 60 us each (masks, sort, re-ordered table), the 16-channel layers stay
        // within 2 us and the 32-channel layers go from 27 to 37 .. 45 us (re-ordered rows gather with less
        // locality); in row order (masks only) the tile-plan kernel is level with the LDS-staged one and the masks
        // still cost 10 us per rulebook.  So SCN_BUILD_SORTMASK alone builds no plan.
        if ((e.flags & SCN_BUILD_TILE_PLANS) && slot.inverse_of < 0 && conv_tile_covers(*w)) {
          slot.want_plan = true;
          slot.plan_sorted = true;
        }
        // input form the kernel needs
        Step st;
        st.kind = StepKind::Conv;
        st.node = (int)i;
        st.label = n.name;
        st.conv = ci;
        st.rulebook = rbi;
        st.coord = x.coord;
        st.coord_out = slot.coord_out;
        st.t_in = n.in[0];
        const int want_dtype = comp == SCN_PRECISION_INT8 ? SCN_DTYPE_INT8 : SCN_DTYPE_FP16;
        float want_range = 0.f;
        bool need_convert = false;
        if (comp == SCN_PRECISION_INT8) {
          if (x.dtype == SCN_DTYPE_INT8) {
            st.x_range = x.range;
          } else {
            want_range = n.in_range;
            st.x_range = want_range;
            need_convert = true;
          }
        } else if (x.dtype == SCN_DTYPE_INT8) {
          need_convert = true;  // dequantise
        }
        const bool is_graph_input = n.in[0] == tin;
        if (!need_convert && (is_graph_input || x.ld < w->cin_pad)) need_convert = true;  // re-pad rows
        st.t_conv_in = n.in[0];
        if (need_convert) {
          char keybuf[128];
          snprintf(keybuf, sizeof(keybuf), "%d:%d:%a:%u", n.in[0], want_dtype, (double)want_range, w->cin_pad);
          auto it = conversions.find(keybuf);
          if (it == conversions.end()) {
            e.tensors.emplace_back();
            RtTensor& cv = e.tensors.back();
            RtTensor& xx = e.tensors[n.in[0]];  // (re-take: the vector may have grown)
            cv.dtype = want_dtype;
            cv.range = want_range;
            cv.c = xx.c;
            cv.ld = w->cin_pad;
            cv.coord = xx.coord;
            cv.materialised = true;
            const int cvi = (int)e.tensors.size() - 1;
            conversions[keybuf] = cvi;
            Step cs;
            cs.kind = StepKind::Convert;
            cs.node = (int)i;
            cs.label = std::string(want_dtype == SCN_DTYPE_INT8 ? "quantize(" : (xx.dtype == SCN_DTYPE_INT8 ? "dequantize(" : "pad(")) +
                       e.tdesc[n.in[0]].name + ")";
            cs.t_in = n.in[0];
            cs.t_out = cvi;
            cs.coord = xx.coord;
            e.steps.push_back(cs);
            st.t_conv_in = cvi;
          } else {
            st.t_conv_in = it->second;
          }
        }
        // output tensor + fusion of a following Add (+Relu) / Relu
        int t_out = n.out;
        st.relu = n.activation == "ReLU" ? 1 : 0;   // (anything but ReLU / None was refused by push_sparse_conv)
        int out_dtype = (plan.outp[i] == SCN_PRECISION_INT8 && plan.range[n.out] > 0.f) ? SCN_DTYPE_INT8 : SCN_DTYPE_FP16;
        float out_range = out_dtype == SCN_DTYPE_INT8 ? plan.range[n.out] : 0.f;
        if (plan.outp[i] == SCN_PRECISION_INT8 && out_dtype != SCN_DTYPE_INT8)
          SCN_LOGW("node %s: int8 output requested but no consumer provides a dynamic range; using fp16", n.name.c_str());
        if (!keep_all) {
          int c1 = single_consumer(n.out);
          if (c1 >= 0 && nodes[c1].op == Op::Add && nodes[c1].in[0] != nodes[c1].in[1]) {
            const NodeDesc& an = nodes[c1];
            const int slot_a = an.in[0] == n.out ? 0 : 1;
            const int other = an.in[1 - slot_a];
            const RtTensor& ot = e.tensors[other];
            // every node between the conv and the Add must be unrelated to the fusion and the
            // residual must already exist
            bool ok = ot.materialised && !ot.dense && ot.coord == slot.coord_out && ot.c == cout && c1 == (int)i + 1;
            if (ok) {
              st.fused_add = true;
              st.t_in2 = other;
              st.mid_dtype = out_dtype;
              st.mid_range = out_range;
              const bool add_i8 = plan.comp[c1] == SCN_PRECISION_INT8;
              const float rq_self = add_i8 ? (slot_a == 0 ? an.a_range : an.b_range) : 0.f;
              const float rq_other = add_i8 ? (slot_a == 0 ? an.b_range : an.a_range) : 0.f;
              st.a_rq = (add_i8 && out_dtype == SCN_DTYPE_FP16) ? rq_self : 0.f;
              st.b_rq = (add_i8 && ot.dtype == SCN_DTYPE_FP16) ? rq_other : 0.f;
              fused_away[c1] = true;
              e.tensors[n.out].coord = slot.coord_out;
              e.tensors[n.out].c = cout;
              t_out = an.out;
              out_dtype = (plan.outp[c1] == SCN_PRECISION_INT8 && plan.range[an.out] > 0.f) ? SCN_DTYPE_INT8 : SCN_DTYPE_FP16;
              out_range = out_dtype == SCN_DTYPE_INT8 ? plan.range[an.out] : 0.f;
              int c2 = single_consumer(an.out);
              if (c2 >= 0 && nodes[c2].op == Op::Relu && c2 == c1 + 1) {
                st.relu2 = 1;
                fused_away[c2] = true;
                e.tensors[an.out].coord = slot.coord_out;
                e.tensors[an.out].c = cout;
                t_out = nodes[c2].out;  // same dtype and scale as the Add output
              }
              st.label += "+" + an.name + (st.relu2 ? "+relu" : "");
            }
          } else if (c1 >= 0 && nodes[c1].op == Op::Relu && c1 == (int)i + 1 && !st.relu) {
            st.relu = 1;
            fused_away[c1] = true;
            e.tensors[n.out].coord = slot.coord_out;
            e.tensors[n.out].c = cout;
            t_out = nodes[c1].out;
            st.label += "+relu";
          }
        }
        RtTensor& o = e.tensors[t_out];
        o.dtype = out_dtype;
        o.range = out_range;
        o.c = cout;
        o.ld = (uint32_t)w->mtiles * 16;
        o.coord = slot.coord_out;
        o.materialised = true;
        st.t_out = t_out;
        e.convs.push_back(std::move(w));
        e.steps.push_back(st);
        break;
      }
      case Op::Add: {
        const RtTensor& a = e.tensors[n.in[0]];
        const RtTensor& b = e.tensors[n.in[1]];
        if (a.dense || b.dense || a.coord != b.coord || a.c != b.c || a.ld != b.ld) {
          set_error("node %s: operands of Add must be sparse tensors on the same coordinates and channels", n.name.c_str());
          return false;
        }
        Step st;
        st.kind = StepKind::Add;
        st.node = (int)i;
        st.label = n.name;
        st.t_in = n.in[0];
        st.t_in2 = n.in[1];
        st.coord = a.coord;
        const bool add_i8 = plan.comp[i] == SCN_PRECISION_INT8;
        st.add_a_rq = (add_i8 && a.dtype == SCN_DTYPE_FP16) ? n.a_range : 0.f;
        st.add_b_rq = (add_i8 && b.dtype == SCN_DTYPE_FP16) ? n.b_range : 0.f;
        int t_out = n.out;
        const int out_dtype = (plan.outp[i] == SCN_PRECISION_INT8 && plan.range[n.out] > 0.f) ? SCN_DTYPE_INT8 : SCN_DTYPE_FP16;
        const float out_range = out_dtype == SCN_DTYPE_INT8 ? plan.range[n.out] : 0.f;
        if (!keep_all) {
          int c1 = single_consumer(n.out);
          if (c1 >= 0 && nodes[c1].op == Op::Relu && c1 == (int)i + 1) {
            st.relu = 1;
            fused_away[c1] = true;
            e.tensors[n.out].coord = a.coord;
            e.tensors[n.out].c = a.c;
            t_out = nodes[c1].out;
            st.label += "+relu";
          }
        }
        RtTensor& o = e.tensors[t_out];
        o.dtype = out_dtype;
        o.range = out_range;
        o.c = a.c;
        o.ld = a.ld;
        o.coord = a.coord;
        o.materialised = true;
        st.t_out = t_out;
        e.steps.push_back(st);
        break;
      }
      case Op::Relu: {
        const RtTensor& x = e.tensors[n.in[0]];
        if (x.dense) {
          set_error("node %s: Relu on a dense tensor is not supported", n.name.c_str());
          return false;
        }
        Step st;
        st.kind = StepKind::Relu;
        st.node = (int)i;
        st.label = n.name;
        st.t_in = n.in[0];
        st.t_out = n.out;
        st.coord = x.coord;
        RtTensor& o = e.tensors[n.out];
        o.dtype = x.dtype;
        o.range = x.range;
        o.c = x.c;
        o.ld = x.ld;
        o.coord = x.coord;
        o.materialised = true;
        e.steps.push_back(st);
        break;
      }
      case Op::Dense: {
        const RtTensor& x = e.tensors[n.in[0]];
        if (x.dense || n.out_shape.size() != 5 || n.out_shape[0] != 1 || n.out_shape[1] != x.c) {
          set_error("node %s: ScatterDense needs a sparse input and output_shape [1, C=%d, D0, D1, D2]", n.name.c_str(), x.c);
          return false;
        }
        Step st;
        st.kind = StepKind::Dense;
        st.node = (int)i;
        st.label = n.name;
        st.t_in = n.in[0];
        st.coord = x.coord;
        for (int j = 0; j < 5; ++j) st.dense_shape[j] = n.out_shape[j];
        int t_out = n.out;
        std::vector<int64_t> shape(n.out_shape.begin(), n.out_shape.end());
        const bool out_i8 = n.dense_range > 0.f && e.precision == SCN_PRECISION_INT8;
        st.form = out_i8 || n.layout != 1;
        st.form_layout = n.layout;
        st.zaxis = n.format == "xyz" ? 2 : 0;
        int c1 = single_consumer(n.out);
        const bool next_is_transpose = c1 >= 0 && nodes[c1].op == Op::Transpose && nodes[c1].dims.size() == 5;
        if (n.layout != 1) {
          // a vectorised layout is defined on the [1, C * Z, H, W] view; the exporter's tail for "xyz" tensors
          // brings z to the front with Transpose (0, 1, 4, 2, 3) first, which the layout already accounts for
          for (size_t u = i + 1; u < nodes.size(); ++u)
            if (nodes[u].op == Op::Transpose && !nodes[u].in.empty() && nodes[u].in[0] == n.out) {
              const auto& d = nodes[u].dims;
              const bool z_front = st.zaxis == 2 && d.size() == 5 && d[0] == 0 && d[1] == 1 && d[2] == 4 && d[3] == 2 && d[4] == 3;
              if (!z_front || (int)u != c1) {
                set_error("node %s: a %s output cannot be transposed", n.name.c_str(), n.layout == 2 ? "NCHW32" : "NHWzC");
                return false;
              }
            }
          if (next_is_transpose) {
            fused_away[c1] = true;
            e.tensors[n.out].dense = true;
            t_out = nodes[c1].out;
            st.label += "+" + nodes[c1].name;
          }
          const int64_t C = n.out_shape[1], Z = n.out_shape[2 + st.zaxis], H = n.out_shape[st.zaxis == 0 ? 3 : 2],
                        W = n.out_shape[st.zaxis == 0 ? 4 : 3];
          if (n.layout == 2) shape = {1, (C * Z + 31) / 32, H, W, 32};
          else shape = {1, H, W, Z, C};
        }
        // fold a following Transpose (and Reshape views) into the scatter
        if (!keep_all && n.layout == 1) {
          if (next_is_transpose) {
            bool okp = true;
            bool seen[5] = {false, false, false, false, false};
            for (int j = 0; j < 5; ++j) {
              int64_t d = nodes[c1].dims[j];
              if (d < 0 || d > 4 || seen[d]) okp = false; else seen[d] = true;
            }
            if (okp) {
              st.has_perm = true;
              std::vector<int64_t> ts(5);
              for (int j = 0; j < 5; ++j) {
                st.perm[j] = (int)nodes[c1].dims[j];
                ts[j] = shape[st.perm[j]];
              }
              shape = ts;
              fused_away[c1] = true;
              e.tensors[n.out].dense = true;
              t_out = nodes[c1].out;
              st.label += "+" + nodes[c1].name;
            }
          }
        }
        RtTensor& o = e.tensors[t_out];
        o.dense = true;
        o.dtype = out_i8 ? SCN_DTYPE_INT8 : SCN_DTYPE_FP16;
        o.range = out_i8 ? n.dense_range : 0.f;
        o.fixed_form = n.layout != 1;
        o.shape = shape;
        o.materialised = true;
        st.t_out = t_out;
        e.steps.push_back(st);
        break;
      }
      case Op::Reshape: {
        RtTensor& x = e.tensors[n.in[0]];
        if (!x.dense) {
          set_error("node %s: Reshape needs a dense input", n.name.c_str());
          return false;
        }
        if (x.fixed_form) {
          // the tensor is already the vectorised form of the network's final 4-D tensor: an alias with that shape
          RtTensor& o = e.tensors[n.out];
          o.dense = true;
          o.dtype = x.dtype;
          o.range = x.range;
          o.shape = x.shape;
          o.fixed_form = true;
          o.view_of = x.view_of >= 0 ? x.view_of : n.in[0];
          o.materialised = true;
          break;
        }
        int64_t numel = 1, known = 1;
        int infer = -1;
        for (auto v : x.shape) numel *= v;
        std::vector<int64_t> shape = n.dims;
        for (size_t j = 0; j < shape.size(); ++j) {
          if (shape[j] == -1) infer = (int)j; else known *= shape[j];
        }
        if (infer >= 0 && known > 0) shape[infer] = numel / known;
        int64_t chk = 1;
        for (auto v : shape) chk *= v;
        if (chk != numel) {
          set_error("node %s: Reshape to a different element count", n.name.c_str());
          return false;
        }
        RtTensor& o = e.tensors[n.out];
        o.dense = true;
        o.dtype = x.dtype;
        o.range = x.range;
        o.shape = shape;
        o.view_of = x.view_of >= 0 ? x.view_of : n.in[0];
        o.materialised = true;
        break;
      }
      case Op::Transpose: {
        // reached only when the Transpose was not folded into the preceding ScatterDense
        RtTensor& x = e.tensors[n.in[0]];
        if (!x.dense || x.shape.size() != 5 || n.dims.size() != 5 || x.fixed_form || x.dtype != SCN_DTYPE_FP16) {
          set_error("node %s: Transpose needs a dense 5-D fp16 input in the NCHW layout and 5 dims", n.name.c_str());
          return false;
        }
        Step st;
        st.kind = StepKind::Permute;
        st.node = (int)i;
        st.label = n.name;
        st.t_in = n.in[0];
        st.t_out = n.out;
        bool seen[5] = {false, false, false, false, false};
        std::vector<int64_t> shape(5);
        for (int j = 0; j < 5; ++j) {
          const int64_t d = n.dims[j];
          if (d < 0 || d > 4 || seen[d]) {
            set_error("node %s: dims is not a permutation", n.name.c_str());
            return false;
          }
          seen[d] = true;
          st.perm[j] = (int)d;
          shape[j] = x.shape[d];
        }
        RtTensor& o = e.tensors[n.out];
        o.dense = true;
        o.dtype = x.dtype;
        o.shape = shape;
        o.materialised = true;
        e.steps.push_back(st);
        break;
      }
    }
  }
  for (size_t t = 0; t < nt; ++t) e.tensor_by_name[e.tdesc[t].name] = (int)t;
  for (int o : e.outputs)
    if (!e.tensors[o].materialised) {
      set_error("output tensor %s is never produced", e.tdesc[o].name.c_str());
      return false;
    }
  if (!e.in_count.alloc(64)) return false;
  if (hipMemset(e.in_count.p, 0, 64) != hipSuccess) return false;
  return true;
}

// Allocates everything whose size depends on the grid (first forward, or when the grid changes).
static int allocate_runtime(scn_engine& e) {
  CoordSet& c0 = e.coords[0];
  memcpy(c0.grid, e.in_grid, 12);
  if (!c0.own_table.buf.p && !c0.own_table.alloc_for(c0.cap)) return SCN_ERR_HIP;
  if (!c0.own_table.alloc_filter(c0.grid)) return SCN_ERR_HIP;
  // propagate grids and capacities through the strided rulebooks (they were created in order)
  for (auto& up : e.rulebooks) {
    RbSlot& s = *up;
    const CoordSet& ci = e.coords[s.coord_in];
    if (s.inverse_of >= 0) {
      const uint32_t max_in_i = ci.cap, max_out_i = e.coords[s.coord_out].cap;
      const int kvol_i = s.ks[0] * s.ks[1] * s.ks[2];
      if (!s.initialised || s.rb.max_in < max_in_i || s.rb.max_out < max_out_i) {
        if (!s.rb.init(max_in_i, max_out_i, kvol_i)) return SCN_ERR_HIP;
        s.initialised = true;
      }
      continue;
    }
    if (!s.subm) {
      CoordSet& co = e.coords[s.coord_out];
      uint64_t vol = 1;
      for (int a = 0; a < 3; ++a) {
        co.grid[a] = (ci.grid[a] + 2 * s.pad[a] - s.dil[a] * (s.ks[a] - 1) - 1) / s.stride[a] + 1;
        SCN_REQUIRE(co.grid[a] >= 1, SCN_ERR_INVALID, "grid %dx%dx%d is too small for the network", e.in_grid[0],
                    e.in_grid[1], e.in_grid[2]);
        vol *= (uint64_t)co.grid[a];
      }
      co.cap = (uint32_t)std::min<uint64_t>(std::min<uint64_t>(s.max_out, vol), (uint64_t)ci.cap * 27ull);
    }
    const uint32_t max_in = ci.cap, max_out = s.subm ? ci.cap : e.coords[s.coord_out].cap;
    const int kvol = s.ks[0] * s.ks[1] * s.ks[2];
    if (!s.initialised || s.rb.max_in < max_in || s.rb.max_out < max_out) {
      if (!s.rb.init(max_in, max_out, kvol)) return SCN_ERR_HIP;
      s.initialised = true;
    }
    // everything a build would allocate lazily is allocated here: forward() must not allocate
    int rc = s.subm ? s.rb.reserve_subm(false) : s.rb.reserve_sparse(e.coords[s.coord_out].grid, false);
    if (rc) return rc;
    if (s.want_plan) {
      rc = s.rb.reserve_plan(s.plan_sorted);
      if (rc) return rc;
    }
  }
  const bool keep_all = (e.flags & SCN_BUILD_KEEP_ALL) != 0;
  // Lifetime of every tensor in step order (the feature kernels run in that order on one stream, with or without
  // the auxiliary stream): from the step that writes it to the last step that reads it.  Sparse tensors whose
  // lifetimes do not overlap share storage; a tensor written by a step never shares with one that step reads.
  // Graph outputs and everything in keep-all engines own their storage.
  const int never = 1 << 30;
  std::vector<int> born(e.tensors.size(), never), dies(e.tensors.size(), -1);
  for (size_t si = 0; si < e.steps.size(); ++si) {
    const Step& st = e.steps[si];
    for (int t : {st.t_in, st.t_in2, st.t_conv_in})
      if (t >= 0 && t < (int)e.tensors.size()) dies[t] = std::max(dies[t], (int)si);
    if (st.t_out >= 0 && st.t_out < (int)e.tensors.size()) {
      born[st.t_out] = std::min(born[st.t_out], (int)si);
      dies[st.t_out] = std::max(dies[st.t_out], (int)si);
    }
  }
  for (int o : e.outputs) dies[o] = never;
  struct Shared {
    size_t bytes;
    int busy_until;
  };
  std::vector<Shared> pool;
  std::vector<int> slot_of(e.tensors.size(), -1);
  {
    std::vector<int> order;
    for (size_t t = 0; t < e.tensors.size(); ++t) {
      const RtTensor& x = e.tensors[t];
      if (!x.materialised || (int)t == e.inputs[0] || x.dense || keep_all || born[t] == never || dies[t] == never) continue;
      order.push_back((int)t);
    }
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return born[a] < born[b]; });
    for (int t : order) {
      const RtTensor& x = e.tensors[t];
      const size_t bytes = ((size_t)e.coords[x.coord].cap * x.ld * (x.dtype == SCN_DTYPE_INT8 ? 1 : 2) + 255) & ~(size_t)255;
      int best = -1;
      for (size_t k = 0; k < pool.size(); ++k)   // the free block that is closest in size
        if (pool[k].busy_until < born[t]) {
          if (best < 0) best = (int)k;
          else {
            const bool fits = pool[k].bytes >= bytes, best_fits = pool[best].bytes >= bytes;
            if ((fits && !best_fits) || (fits == best_fits && (fits ? pool[k].bytes < pool[best].bytes : pool[k].bytes > pool[best].bytes)))
              best = (int)k;
          }
        }
      if (best < 0) {
        pool.push_back(Shared{bytes, dies[t]});
        best = (int)pool.size() - 1;
      } else {
        pool[best].bytes = std::max(pool[best].bytes, bytes);
        pool[best].busy_until = dies[t];
      }
      slot_of[t] = best;
    }
  }
  if (e.arena.size() < pool.size()) e.arena.resize(pool.size());
  for (size_t k = 0; k < pool.size(); ++k)
    if (e.arena[k].bytes < pool[k].bytes) {
      if (!e.arena[k].alloc(pool[k].bytes)) return SCN_ERR_HIP;
      SCN_HIP(hipMemset(e.arena[k].p, 0, pool[k].bytes));
    }
  for (size_t t = 0; t < e.tensors.size(); ++t) {
    RtTensor& x = e.tensors[t];
    if (!x.materialised || (int)t == e.inputs[0]) continue;
    if (x.dense) {
      if (x.view_of >= 0) continue;
      size_t numel = 1;
      for (auto v : x.shape) numel *= (size_t)v;
      const size_t dbytes = (numel * (x.dtype == SCN_DTYPE_INT8 ? 1 : 2) + 15) & ~(size_t)15;
      if (x.buf.bytes < dbytes && !x.buf.alloc(dbytes)) return SCN_ERR_HIP;
      x.data = x.buf.p;
      continue;
    }
    x.shared = slot_of[t] >= 0;
    if (x.shared) {
      x.buf.release();
      x.data = e.arena[slot_of[t]].p;
      continue;
    }
    const size_t rows = e.coords[x.coord].cap;
    const size_t bytes = rows * x.ld * (x.dtype == SCN_DTYPE_INT8 ? 1 : 2);
    if (x.buf.bytes < bytes) {
      if (!x.buf.alloc(bytes)) return SCN_ERR_HIP;
      SCN_HIP(hipMemset(x.buf.p, 0, bytes));
    }
    x.data = x.buf.p;
  }
  for (auto& x : e.tensors)
    if (x.dense && x.view_of >= 0) x.data = e.tensors[x.view_of].data;
  e.dense_maps.resize(e.steps.size());
  for (size_t si = 0; si < e.steps.size(); ++si) {
    const Step& st = e.steps[si];
    if (st.kind != StepKind::Dense || st.form) continue;
    const size_t cells = scatter_dense_map_cells(st.dense_shape, st.has_perm ? st.perm : nullptr);
    if (cells && e.dense_maps[si].bytes < cells * 4 && !e.dense_maps[si].alloc(cells * 4)) return SCN_ERR_HIP;
  }
  if (keep_all) {
    for (auto& st : e.steps)
      if (st.kind == StepKind::Conv) {
        RtTensor& o = e.tensors[st.t_out];
        const size_t bytes = (size_t)e.coords[o.coord].cap * o.ld * 4;
        if (o.acc.bytes < bytes && !o.acc.alloc(bytes)) return SCN_ERR_HIP;
      }
  }
  if ((e.flags & SCN_BUILD_AUX_STREAM) && !e.aux) {
    SCN_HIP(hipStreamCreateWithFlags(&e.aux, hipStreamNonBlocking));  // default priority
    SCN_HIP(hipEventCreateWithFlags(&e.ev_fork, hipEventDisableTiming));
    SCN_HIP(hipEventCreateWithFlags(&e.ev_join, hipEventDisableTiming));
    e.rb_ready.assign(e.rulebooks.size(), nullptr);
    for (auto& ev : e.rb_ready) SCN_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
  }
  memcpy(e.alloc_grid, e.in_grid, 12);
  e.allocated = true;
  return SCN_OK;
}

static int run_step(scn_engine& e, Step& st, hipStream_t stream) {
  switch (st.kind) {
    case StepKind::InputCount: {
      CoordSet& c0 = e.coords[0];
      uint32_t n = e.in_n;
      if (n > c0.cap) {
        SCN_LOGW("The number of input points %u exceeds the theoretical maximum number %u; truncate", n, c0.cap);
        n = c0.cap;
      }
      c0.idx = e.in_idx;
      c0.n_bound = n;
      c0.has_lookup = false;
      // One launch publishes the clamped input count and clears everything this forward builds into:
      // the input hash (+ its occupancy filter), the output bitmaps of the strided rulebooks and the
      // dense outputs.  The steps that own those buffers then skip their own fills.
      FillJob jobs[kMaxFillJobs];
      int nj = 0;
      auto add = [&](void* p, size_t words, uint32_t value) {
        if (!p || words == 0 || nj >= kMaxFillJobs) return false;
        jobs[nj++] = FillJob{p, words, value};
        return true;
      };
      e.dense_precleared.assign(e.steps.size(), 0);
      for (size_t si = 0; si < e.steps.size(); ++si) {
        const Step& s2 = e.steps[si];
        if (s2.kind == StepKind::HashBuild && s2.coord == 0) {
          CoordTable& t = c0.own_table;
          const size_t words = hash_capacity_for(n) * 2;
          if (words <= t.cap * 2 && nj + (t.filter_words ? 2 : 1) <= kMaxFillJobs) {
            add(t.slots(), words, 0xFFFFFFFFu);
            if (t.filter_words) add(t.filter.p, t.filter_fill_words(), 0u);
            t.precleared_for = n;
          }
        } else if (s2.kind == StepKind::RulebookSparse) {
          Rulebook& rb = e.rulebooks[s2.rulebook]->rb;
          if (rb.bitmap.p && rb.bitmap_words && add(rb.bitmap.p, rb.bitmap_words, 0u)) rb.bitmap_precleared = true;
        } else if (s2.kind == StepKind::Dense && !s2.form) {
          RtTensor& o = e.tensors[s2.t_out];
          size_t numel = 1;
          for (int j = 0; j < 5; ++j) numel *= (size_t)s2.dense_shape[j];
          if (si < e.dense_maps.size() && e.dense_maps[si].p) {
            if (add(e.dense_maps[si].p, e.dense_maps[si].bytes / 4, 0xFFFFFFFFu)) e.dense_precleared[si] = 2;
          } else if (numel % 2 == 0 && add(o.data, numel / 2, 0u)) {
            e.dense_precleared[si] = 1;
          }
        }
      }
      int rc = fill_multi(jobs, nj, e.in_count.as<uint32_t>(), e.dds, n, stream);
      if (rc) return rc;
      c0.n_dev = e.in_count.as<uint32_t>();
      RtTensor& t = e.tensors[e.inputs[0]];
      t.data = const_cast<void*>(e.in_feat);
      t.ld = e.in_c;
      return SCN_OK;
    }
    case StepKind::HashBuild: {
      CoordSet& cs = e.coords[st.coord];
      int rc = hash_build(cs.own_table, cs.idx, cs.n_bound, cs.n_dev, cs.grid, nullptr, stream);
      if (rc) return rc;
      cs.lookup = cs.own_table.lookup();
      cs.has_lookup = true;
      return SCN_OK;
    }
    case StepKind::RulebookSubm: {
      RbSlot& s = *e.rulebooks[st.rulebook];
      CoordSet& cs = e.coords[s.coord_in];
      int rc = s.rb.build_subm(cs.idx, cs.n_bound, cs.n_dev, cs.grid, s.ks, s.dil, cs.has_lookup ? &cs.lookup : nullptr,
                               stream);
      if (rc == SCN_OK && s.want_plan) rc = s.rb.build_plan(s.plan_sorted, stream);
      return rc;
    }
    case StepKind::RulebookSparse: {
      RbSlot& s = *e.rulebooks[st.rulebook];
      CoordSet& ci = e.coords[s.coord_in];
      CoordSet& co = e.coords[s.coord_out];
      int rc = s.rb.build_sparse(ci.idx, ci.n_bound, ci.n_dev, ci.grid, s.ks, s.stride, s.pad, s.dil,
                                 ci.has_lookup ? &ci.lookup : nullptr, stream);
      if (rc) return rc;
      if (s.want_plan) {
        rc = s.rb.build_plan(s.plan_sorted, stream);
        if (rc) return rc;
      }
      co.idx = s.rb.out_indices;
      co.n_dev = s.rb.n_out_dev();
      co.n_bound = s.rb.n_bound_out;
      co.lookup = s.rb.out_lookup();
      co.has_lookup = true;
      return SCN_OK;
    }
    case StepKind::RulebookInverse: {
      RbSlot& s = *e.rulebooks[st.rulebook];
      const RbSlot& f = *e.rulebooks[s.inverse_of];
      return s.rb.build_inverse(f.rb, e.coords[s.coord_out].n_dev, stream);
    }
    case StepKind::Convert: {
      const RtTensor& x = e.tensors[st.t_in];
      RtTensor& o = e.tensors[st.t_out];
      const CoordSet& cs = e.coords[x.coord];
      return convert_rows(x.data, x.dtype, (uint32_t)x.c, x.ld, x.range, o.data, o.dtype, o.ld, o.ld, o.range, 0,
                          cs.n_bound, cs.n_dev, stream);
    }
    case StepKind::Conv: {
      const RtTensor& x = e.tensors[st.t_conv_in];
      RtTensor& o = e.tensors[st.t_out];
      RbSlot& s = *e.rulebooks[st.rulebook];
      scn_conv_io io;
      memset(&io, 0, sizeof(io));
      io.x_dev = x.data;
      io.x_ld = x.ld;
      io.x_dynamic_range = st.x_range;
      io.relu = st.relu;
      io.out_dtype = o.dtype;
      io.out_dynamic_range = o.range;
      io.out_dev = o.data;
      io.out_ld = o.ld;
      io.acc_dev = o.acc.p;
      io.fixed_launch_points = e.nodes[st.node].fixed_launch_points;
      if (st.fused_add) {
        const RtTensor& r = e.tensors[st.t_in2];
        io.res_dev = r.data;
        io.res_dtype = r.dtype;
        io.res_dynamic_range = r.range;
        io.res_ld = r.ld;
        io.mid_dtype = st.mid_dtype;
        io.mid_dynamic_range = st.mid_range;
        io.a_requant_range = st.a_rq;
        io.b_requant_range = st.b_rq;
        io.relu_after_add = st.relu2;
      }
      PlanView pv;
      const TilePlan& tp = s.rb.plan;
      const bool planned = s.want_plan && tp.built;
      if (planned) {
        pv.tmask = tp.tmask.as<uint32_t>();
        if (tp.sorted) {
          pv.perm = tp.perm.as<uint32_t>();
          pv.nbr = tp.nbr.as<int32_t>();
        }
      }
      return conv_forward(*e.convs[st.conv], s.rb.nbr.as<int32_t>(), s.rb.ld, s.rb.n_out_dev(), s.rb.n_bound_out,
                          s.rb.n_out_hint(), io, stream, planned ? &pv : nullptr);
    }
    case StepKind::Add: {
      const RtTensor& a = e.tensors[st.t_in];
      const RtTensor& b = e.tensors[st.t_in2];
      RtTensor& o = e.tensors[st.t_out];
      const CoordSet& cs = e.coords[a.coord];
      return add_relu(a.data, a.dtype, a.range, st.add_a_rq, b.data, b.dtype, b.range, st.add_b_rq, o.data, o.dtype,
                      o.range, st.relu, a.ld, cs.n_bound, cs.n_dev, stream);
    }
    case StepKind::Relu: {
      const RtTensor& x = e.tensors[st.t_in];
      RtTensor& o = e.tensors[st.t_out];
      const CoordSet& cs = e.coords[x.coord];
      // value-preserving re-store with ReLU: a range of 127 makes the int8 <-> value mapping the identity
      return convert_rows(x.data, x.dtype, x.ld, x.ld, 127.f, o.data, o.dtype, o.ld, o.ld, 127.f, 1, cs.n_bound, cs.n_dev,
                          stream);
    }
    case StepKind::Dense: {
      const RtTensor& x = e.tensors[st.t_in];
      RtTensor& o = e.tensors[st.t_out];
      const CoordSet& cs = e.coords[x.coord];
      if (st.form)
        return scatter_dense_form(x.data, x.dtype, x.range, (uint32_t)x.c, x.ld, cs.idx, cs.n_bound, cs.n_dev, st.dense_shape,
                                  st.has_perm ? st.perm : nullptr, st.zaxis, st.form_layout, o.dtype, o.range, o.data, stream);
      const size_t si = (size_t)(&st - e.steps.data());
      const int pre = si < e.dense_precleared.size() ? e.dense_precleared[si] : 0;
      int32_t* map = si < e.dense_maps.size() ? e.dense_maps[si].as<int32_t>() : nullptr;
      return scatter_dense(x.data, x.dtype, x.range, (uint32_t)x.c, x.ld, cs.idx, cs.n_bound, cs.n_dev, st.dense_shape,
                           st.has_perm ? st.perm : nullptr, o.data, stream, pre == 1, map, pre == 2, e.dense_map_built);
    }
    case StepKind::Permute: {
      const RtTensor& x = e.tensors[st.t_in];
      RtTensor& o = e.tensors[st.t_out];
      int64_t shape[5];
      for (int j = 0; j < 5; ++j) shape[j] = x.shape[j];
      return permute_dense(x.data, shape, st.perm, o.data, stream);
    }
  }
  return SCN_ERR_INVALID;
}

// ---------------------------------------------------------------------------------------------
// ONNX reading (protobuf wire format, only the messages the dialect uses)
// field numbers: libraries/3DSparseConvolution/src/onnx/onnx-ml.proto:116-176,181-215,342-382,441-462,486-587
// ---------------------------------------------------------------------------------------------
struct PbReader {
  const uint8_t* p;
  const uint8_t* end;
  bool ok = true;
  PbReader(const uint8_t* b, size_t n) : p(b), end(b + n) {}
  bool done() const { return p >= end || !ok; }
  uint64_t varint() {
    uint64_t v = 0;
    int shift = 0;
    while (p < end && shift < 64) {
      const uint8_t b = *p++;
      v |= (uint64_t)(b & 0x7f) << shift;
      if (!(b & 0x80)) return v;
      shift += 7;
    }
    ok = false;
    return 0;
  }
  // reads one field header; for length-delimited fields sets [data, len)
  bool next(int* field, int* wt, uint64_t* val, const uint8_t** data, size_t* len) {
    if (done()) return false;
    const uint64_t key = varint();
    if (!ok) return false;
    *field = (int)(key >> 3);
    *wt = (int)(key & 7);
    *val = 0;
    *data = nullptr;
    *len = 0;
    switch (*wt) {
      case 0: *val = varint(); break;
      case 1:
        if (end - p < 8) { ok = false; return false; }
        memcpy(val, p, 8);
        p += 8;
        break;
      case 2: {
        const uint64_t n = varint();
        if (!ok || (uint64_t)(end - p) < n) { ok = false; return false; }
        *data = p;
        *len = (size_t)n;
        p += n;
        break;
      }
      case 5: {
        if (end - p < 4) { ok = false; return false; }
        uint32_t v32;
        memcpy(&v32, p, 4);
        *val = v32;
        p += 4;
        break;
      }
      default: ok = false; return false;
    }
    return ok;
  }
};

struct OnnxAttr {
  std::string name, s;
  float f = 0.f;
  int64_t i = 0;
  std::vector<float> floats;
  std::vector<int64_t> ints;
};
struct OnnxNode {
  std::string name, op_type;
  std::vector<std::string> input, output;
  std::vector<OnnxAttr> attrs;
  const OnnxAttr* find(const char* n) const {
    for (auto& a : attrs)
      if (a.name == n) return &a;
    return nullptr;
  }
};
struct OnnxTensor {
  std::string name;
  std::vector<int64_t> dims;
  int data_type = 0;
  std::string raw;
};
struct OnnxGraph {
  std::vector<OnnxNode> nodes;
  std::vector<OnnxTensor> inits;
  std::vector<std::string> inputs, outputs;
};

static bool parse_attr(const uint8_t* b, size_t n, OnnxAttr& a) {
  PbReader r(b, n);
  int f, wt;
  uint64_t v;
  const uint8_t* d;
  size_t len;
  while (r.next(&f, &wt, &v, &d, &len)) {
    if (f == 1 && wt == 2) a.name.assign((const char*)d, len);
    else if (f == 2 && wt == 5) { uint32_t u = (uint32_t)v; memcpy(&a.f, &u, 4); }
    else if (f == 3 && wt == 0) a.i = (int64_t)v;
    else if (f == 4 && wt == 2) a.s.assign((const char*)d, len);
    else if (f == 7 && wt == 2) { for (size_t k = 0; k + 4 <= len; k += 4) { float x; memcpy(&x, d + k, 4); a.floats.push_back(x); } }
    else if (f == 7 && wt == 5) { uint32_t u = (uint32_t)v; float x; memcpy(&x, &u, 4); a.floats.push_back(x); }
    else if (f == 8 && wt == 2) { PbReader q(d, len); while (!q.done()) { uint64_t x = q.varint(); if (q.ok) a.ints.push_back((int64_t)x); } }
    else if (f == 8 && wt == 0) a.ints.push_back((int64_t)v);
  }
  return r.ok;
}

static bool parse_node(const uint8_t* b, size_t n, OnnxNode& node) {
  PbReader r(b, n);
  int f, wt;
  uint64_t v;
  const uint8_t* d;
  size_t len;
  while (r.next(&f, &wt, &v, &d, &len)) {
    if (wt != 2) continue;
    if (f == 1) node.input.emplace_back((const char*)d, len);
    else if (f == 2) node.output.emplace_back((const char*)d, len);
    else if (f == 3) node.name.assign((const char*)d, len);
    else if (f == 4) node.op_type.assign((const char*)d, len);
    else if (f == 5) { OnnxAttr a; if (!parse_attr(d, len, a)) return false; node.attrs.push_back(std::move(a)); }
  }
  return r.ok;
}

static bool parse_tensor(const uint8_t* b, size_t n, OnnxTensor& t) {
  PbReader r(b, n);
  int f, wt;
  uint64_t v;
  const uint8_t* d;
  size_t len;
  while (r.next(&f, &wt, &v, &d, &len)) {
    if (f == 1 && wt == 0) t.dims.push_back((int64_t)v);
    else if (f == 1 && wt == 2) { PbReader q(d, len); while (!q.done()) { uint64_t x = q.varint(); if (q.ok) t.dims.push_back((int64_t)x); } }
    else if (f == 2 && wt == 0) t.data_type = (int)v;
    else if (f == 8 && wt == 2) t.name.assign((const char*)d, len);
    else if (f == 9 && wt == 2) t.raw.assign((const char*)d, len);
  }
  return r.ok;
}

static bool parse_value_info_name(const uint8_t* b, size_t n, std::string& name) {
  PbReader r(b, n);
  int f, wt;
  uint64_t v;
  const uint8_t* d;
  size_t len;
  while (r.next(&f, &wt, &v, &d, &len))
    if (f == 1 && wt == 2) name.assign((const char*)d, len);
  return r.ok;
}

static bool parse_model(const std::string& bytes, OnnxGraph& g) {
  PbReader r((const uint8_t*)bytes.data(), bytes.size());
  int f, wt;
  uint64_t v;
  const uint8_t* d;
  size_t len;
  const uint8_t* gd = nullptr;
  size_t glen = 0;
  while (r.next(&f, &wt, &v, &d, &len))
    if (f == 7 && wt == 2) { gd = d; glen = len; }
  if (!r.ok || !gd) return false;
  PbReader gr(gd, glen);
  while (gr.next(&f, &wt, &v, &d, &len)) {
    if (wt != 2) continue;
    if (f == 1) { OnnxNode n; if (!parse_node(d, len, n)) return false; g.nodes.push_back(std::move(n)); }
    else if (f == 5) { OnnxTensor t; if (!parse_tensor(d, len, t)) return false; g.inits.push_back(std::move(t)); }
    else if (f == 11) { std::string s; if (!parse_value_info_name(d, len, s)) return false; g.inputs.push_back(s); }
    else if (f == 12) { std::string s; if (!parse_value_info_name(d, len, s)) return false; g.outputs.push_back(s); }
  }
  return gr.ok;
}

}  // namespace scn

// =============================================================================================
// C ABI
// =============================================================================================
extern "C" {

scn_builder* scn_builder_create(void) { return new scn_builder(); }
void scn_builder_destroy(scn_builder* b) { delete b; }

int scn_builder_push_input(scn_builder* b, const char* name) {
  if (!b) return -1;
  const int t = b->new_tensor(name, -1);
  b->inputs.push_back(t);
  return t;
}

static void copy3(int dst[3], const int* src, int dflt) {
  for (int a = 0; a < 3; ++a) dst[a] = src ? src[a] : dflt;
}

int scn_builder_push_sparse_conv(scn_builder* b, const char* name, int x, const uint16_t* weight,
                                 const int weight_shape[5], const float* weight_dynamic_ranges,
                                 int n_weight_dynamic_ranges, const uint16_t* bias, int n_bias, const char* activation,
                                 const int kernel_size[3], const int stride[3], const int padding[3],
                                 const int dilation[3], float input_dynamic_range, int submanifold,
                                 uint32_t max_output_points, uint32_t fixed_launch_points, const char* rulebook,
                                 int precision, int output_precision, const char* output_name, int inverse) {
  if (!b || !b->valid_tensor(x) || !weight || !weight_shape || !kernel_size) {
    set_error("push_sparse_conv(%s): invalid arguments", name ? name : "");
    return -1;
  }
  // What cannot be computed is refused when it is pushed, so that the builder and the loader return nullptr
  // instead of an engine with different arithmetic (the loader's contract for a model it cannot run,
  // libraries/3DSparseConvolution/src/onnx-parser.cpp:216-219).  The exporters can write other activations
  // (CUDA-CenterPoint/qat/onnx_export/exptool.py:167-172).
  if (activation && *activation && strcmp(activation, "ReLU") != 0 && strcmp(activation, "None") != 0) {
    set_error("push_sparse_conv(%s): activation '%s' is not supported (ReLU or None)", name ? name : "", activation);
    return -1;
  }
  if (inverse && (submanifold || !rulebook || !*rulebook)) {
    set_error("push_sparse_conv(%s): an inverse convolution names the rulebook of an earlier strided convolution",
              name ? name : "");
    return -1;
  }
  NodeDesc n;
  n.op = Op::Conv;
  n.name = name ? name : "";
  n.in = {x};
  size_t vol = 1;
  for (int j = 0; j < 5; ++j) {
    if (weight_shape[j] <= 0) {
      set_error("push_sparse_conv(%s): invalid weight shape", n.name.c_str());
      return -1;
    }
    n.wshape[j] = weight_shape[j];
    vol *= (size_t)weight_shape[j];
  }
  if (weight_shape[1] != kernel_size[0] || weight_shape[2] != kernel_size[1] || weight_shape[3] != kernel_size[2]) {
    set_error("push_sparse_conv(%s): weight shape [Cout,K0,K1,K2,Cin] does not match kernel_size", n.name.c_str());
    return -1;
  }
  n.weight.assign(weight, weight + vol);
  if (weight_dynamic_ranges && n_weight_dynamic_ranges > 0)
    n.wranges.assign(weight_dynamic_ranges, weight_dynamic_ranges + n_weight_dynamic_ranges);
  if (bias && n_bias > 0) {
    if (n_bias != weight_shape[0]) {
      set_error("push_sparse_conv(%s): bias has %d elements, Cout is %d", n.name.c_str(), n_bias, weight_shape[0]);
      return -1;
    }
    n.bias.assign(bias, bias + n_bias);
  }
  n.activation = activation ? activation : "";
  copy3(n.ks, kernel_size, 1);
  copy3(n.stride, stride, 1);
  copy3(n.pad, padding, 0);
  copy3(n.dil, dilation, 1);
  for (int a = 0; a < 3; ++a) {
    if (n.stride[a] <= 0) n.stride[a] = 1;  // attributes missing from the model read as 0
    if (n.dil[a] <= 0) n.dil[a] = 1;
  }
  n.in_range = input_dynamic_range;
  n.subm = submanifold != 0;
  n.inverse = inverse != 0;
  n.max_out = max_output_points ? max_output_points : 150000;
  n.fixed_launch_points = fixed_launch_points;
  n.rulebook = rulebook ? rulebook : "";
  n.precision = precision;
  n.out_precision = output_precision;
  n.out = b->new_tensor(output_name, (int)b->nodes.size());
  b->nodes.push_back(std::move(n));
  return b->nodes.back().out;
}

int scn_builder_push_add(scn_builder* b, const char* name, int a, int b_tensor, float a_dynamic_range,
                         float b_dynamic_range, const char* output_name, int precision, int output_precision,
                         uint32_t fixed_launch_points) {
  (void)fixed_launch_points;
  if (!b || !b->valid_tensor(a) || !b->valid_tensor(b_tensor)) {
    set_error("push_add(%s): invalid arguments", name ? name : "");
    return -1;
  }
  NodeDesc n;
  n.op = Op::Add;
  n.name = name ? name : "";
  n.in = {a, b_tensor};
  n.a_range = a_dynamic_range;
  n.b_range = b_dynamic_range;
  n.precision = precision;
  n.out_precision = output_precision;
  n.out = b->new_tensor(output_name, (int)b->nodes.size());
  b->nodes.push_back(std::move(n));
  return b->nodes.back().out;
}

int scn_builder_push_relu(scn_builder* b, const char* name, int x, const char* output_name) {
  if (!b || !b->valid_tensor(x)) {
    set_error("push_relu(%s): invalid arguments", name ? name : "");
    return -1;
  }
  NodeDesc n;
  n.op = Op::Relu;
  n.name = name ? name : "";
  n.in = {x};
  n.out = b->new_tensor(output_name, (int)b->nodes.size());
  b->nodes.push_back(std::move(n));
  return b->nodes.back().out;
}

int scn_builder_push_dense(scn_builder* b, const char* name, int x, const char* format, const char* output_name,
                           const int input_spatial_shape[3], const int* output_shape, int n_output_shape,
                           int output_layout, float input_dynamic_range, uint32_t input_bound) {
  (void)input_bound;
  if (!b || !b->valid_tensor(x) || !output_shape || n_output_shape <= 0) {
    set_error("push_dense(%s): invalid arguments", name ? name : "");
    return -1;
  }
  if (output_layout < 0 || output_layout > 3) {
    set_error("push_dense(%s): unknown output layout %d", name ? name : "", output_layout);
    return -1;
  }
  if (n_output_shape != 5) {
    set_error("push_dense(%s): output_shape must be [1, C, D0, D1, D2]", name ? name : "");
    return -1;
  }
  NodeDesc n;
  n.op = Op::Dense;
  n.name = name ? name : "";
  n.in = {x};
  n.format = format ? format : "";
  copy3(n.in_spatial, input_spatial_shape, 0);
  n.out_shape.assign(output_shape, output_shape + n_output_shape);
  n.dense_range = input_dynamic_range > 0.f ? input_dynamic_range : 0.f;  // > 0: int8 output under an int8 engine
  n.layout = output_layout == 0 ? 1 : output_layout;
  n.out = b->new_tensor(output_name, (int)b->nodes.size());
  b->nodes.push_back(std::move(n));
  return b->nodes.back().out;
}

int scn_builder_push_reshape(scn_builder* b, const char* name, int x, const int64_t* shape, int n_shape,
                             const char* output_name) {
  if (!b || !b->valid_tensor(x) || !shape || n_shape <= 0) {
    set_error("push_reshape(%s): invalid arguments", name ? name : "");
    return -1;
  }
  NodeDesc n;
  n.op = Op::Reshape;
  n.name = name ? name : "";
  n.in = {x};
  n.dims.assign(shape, shape + n_shape);
  n.out = b->new_tensor(output_name, (int)b->nodes.size());
  b->nodes.push_back(std::move(n));
  return b->nodes.back().out;
}

int scn_builder_push_transpose(scn_builder* b, const char* name, int x, const int64_t* dims, int n_dims,
                               const char* output_name) {
  if (!b || !b->valid_tensor(x) || !dims || n_dims <= 0) {
    set_error("push_transpose(%s): invalid arguments", name ? name : "");
    return -1;
  }
  NodeDesc n;
  n.op = Op::Transpose;
  n.name = name ? name : "";
  n.in = {x};
  n.dims.assign(dims, dims + n_dims);
  n.out = b->new_tensor(output_name, (int)b->nodes.size());
  b->nodes.push_back(std::move(n));
  return b->nodes.back().out;
}

int scn_builder_push_output(scn_builder* b, int tensor) {
  if (!b || !b->valid_tensor(tensor)) {
    set_error("push_output: invalid tensor");
    return SCN_ERR_INVALID;
  }
  b->outputs.push_back(tensor);
  return SCN_OK;
}

scn_engine* scn_builder_build(scn_builder* b, int precision, unsigned flags, void* stream) {
  (void)stream;
  if (!b) return nullptr;
  if (precision != SCN_PRECISION_FP16 && precision != SCN_PRECISION_INT8) {
    set_error("build: precision must be Float16 (1) or Int8 (2)");
    return nullptr;
  }
  auto* e = new scn_engine();
  e->nodes = b->nodes;
  e->tdesc = b->tensors;
  e->inputs = b->inputs;
  e->outputs = b->outputs;
  e->precision = precision;
  e->flags = flags;
  if (!build_engine(*e)) {
    delete e;
    return nullptr;
  }
  SCN_LOGV("engine built: %zu nodes -> %zu steps, %zu rulebooks, precision %s", e->nodes.size(), e->steps.size(),
           e->rulebooks.size(), precision == SCN_PRECISION_INT8 ? "int8" : "fp16");
  return e;
}

static std::vector<int> attr_ints3(const OnnxNode& n, const char* name) {
  std::vector<int> out;
  if (const OnnxAttr* a = n.find(name))
    for (auto v : a->ints) out.push_back((int)v);
  return out;
}

static scn_engine* create_from_model_bytes(const std::string& bytes, const char* onnx_file, int precision, unsigned flags,
                                           unsigned fixed_launch_points, const scn_load_options* options, void* stream);

scn_engine* scn_engine_create_from_onnx(const char* onnx_file, int precision, unsigned flags,
                                        unsigned fixed_launch_points, void* stream) {
  return scn_engine_create_from_onnx_ex(onnx_file, precision, flags, fixed_launch_points, nullptr, stream);
}

scn_engine* scn_engine_create_from_onnx_ex(const char* onnx_file, int precision, unsigned flags,
                                           unsigned fixed_launch_points, const scn_load_options* options,
                                           void* stream) {
  if (!onnx_file) return nullptr;
  SCN_LOGV("Load onnx from: %s", onnx_file);
  std::ifstream fin(onnx_file, std::ios::binary);
  if (!fin) {
    set_error("Parse onnx failed: %s (cannot open)", onnx_file);
    return nullptr;
  }
  const std::string bytes((std::istreambuf_iterator<char>(fin)), std::istreambuf_iterator<char>());
  return create_from_model_bytes(bytes, onnx_file, precision, flags, fixed_launch_points, options, stream);
}

scn_engine* scn_engine_create_from_onnx_memory(const void* model_bytes, size_t size, int precision, unsigned flags,
                                               unsigned fixed_launch_points, const scn_load_options* options,
                                               void* stream) {
  if (!model_bytes && size) {
    set_error("create_from_onnx_memory: null model");
    return nullptr;
  }
  const std::string bytes(static_cast<const char*>(model_bytes), size);
  return create_from_model_bytes(bytes, "(memory)", precision, flags, fixed_launch_points, options, stream);
}

static scn_engine* create_from_model_bytes(const std::string& bytes, const char* onnx_file, int precision, unsigned flags,
                                           unsigned fixed_launch_points, const scn_load_options* options, void* stream) {
  const scn_precision_override* overrides = options ? options->overrides : nullptr;
  const int n_overrides = options ? options->n_overrides : 0;
  const scn_tensor_amax* ranges = options ? options->ranges : nullptr;
  const int n_ranges = options ? options->n_ranges : 0;
  if (n_overrides < 0 || (n_overrides > 0 && !overrides) || n_ranges < 0 || (n_ranges > 0 && !ranges)) {
    set_error("create_from_onnx: invalid load options");
    return nullptr;
  }
  // calibrated |max| of a tensor, or 0 when the options hold none for it
  auto range_of = [&](const std::string& tensor) {
    float r = 0.f;
    for (int i = 0; i < n_ranges; ++i)
      if (ranges[i].tensor && tensor == ranges[i].tensor) r = ranges[i].amax;
    return r;
  };
  OnnxGraph g;
  if (bytes.empty() || !parse_model(bytes, g)) {
    set_error("Parse onnx failed: %s", onnx_file);
    return nullptr;
  }
  std::unique_ptr<scn_builder, void (*)(scn_builder*)> b(scn_builder_create(), scn_builder_destroy);
  std::map<std::string, int> tmap;
  for (auto& name : g.inputs) {
    bool is_init = false;
    for (auto& t : g.inits) is_init |= t.name == name;
    if (!is_init) tmap[name] = scn_builder_push_input(b.get(), name.c_str());
  }
  auto find_init = [&](const std::string& name, std::vector<uint16_t>& data, std::vector<int>& shape) -> bool {
    for (auto& t : g.inits)
      if (t.name == name) {
        if (t.data_type != 10) {
          set_error("Can not support non float data type[%d] for initializer data.", t.data_type);
          return false;
        }
        size_t vol = 1;
        shape.clear();
        for (auto d : t.dims) {
          // (each dimension and the volume stay far inside int and size_t, so that the builder's own products of
          // the int shape cannot differ from this one)
          if (d < 1 || d > (1 << 24) || vol > ((size_t)1 << 31) / (size_t)d) {
            set_error("Invalid dimensions of initializer '%s'.", name.c_str());
            return false;
          }
          shape.push_back((int)d);
          vol *= (size_t)d;
        }
        if (t.dims.empty() || vol * 2 != t.raw.size()) {
          set_error("Invalid parameter data size. %zu != %zu", vol * 2, t.raw.size());
          return false;
        }
        data.resize(vol);
        memcpy(data.data(), t.raw.data(), vol * 2);
        return true;
      }
    set_error("Can not find initializer '%s' in ONNX.", name.c_str());
    return false;
  };
  auto tensor_of = [&](const std::string& name) -> int {
    auto it = tmap.find(name);
    if (it == tmap.end()) {
      set_error("tensor '%s' is used before it is produced", name.c_str());
      return -1;
    }
    return it->second;
  };
  // the node's own attribute unless an override names the node or its operator type (the last match wins)
  auto prec_of = [&](const OnnxNode& n, const char* attr) {
    const OnnxAttr* a = n.find(attr);
    int p = (a && a->s == "int8") ? SCN_PRECISION_INT8 : SCN_PRECISION_FP16;
    const bool is_output = !strcmp(attr, "output_precision");
    for (int i = 0; i < n_overrides; ++i) {
      const scn_precision_override& o = overrides[i];
      if (!o.selector) continue;
      const std::string& subject = o.by_optype ? n.op_type : n.name;
      const bool add_alias = o.by_optype && (n.op_type == "Add" || n.op_type == "QuantAdd") &&
                             (!strcmp(o.selector, "Add") || !strcmp(o.selector, "QuantAdd"));
      if (subject != o.selector && !add_alias) continue;
      const int v = is_output ? o.output_precision : o.precision;
      if (v == SCN_PRECISION_FP16 || v == SCN_PRECISION_INT8) p = v;
    }
    return p;
  };
  for (auto& n : g.nodes) {
    unsigned flp = fixed_launch_points;
    if (const OnnxAttr* a = n.find("fixed_launch_points")) flp = (unsigned)a->i;
    int out = -1;
    if (n.op_type == "SparseConvolution") {
      if (n.input.size() < 3 || n.output.empty()) {
        set_error("node %s: SparseConvolution needs inputs [x, weight, bias]", n.name.c_str());
        return nullptr;
      }
      const int x = tensor_of(n.input[0]);
      if (x < 0) return nullptr;
      std::vector<uint16_t> w, bias;
      std::vector<int> wshape, bshape;
      if (!find_init(n.input[1], w, wshape) || !find_init(n.input[2], bias, bshape)) return nullptr;
      if (wshape.size() != 5) {
        set_error("node %s: weight must be [Cout,K0,K1,K2,Cin]", n.name.c_str());
        return nullptr;
      }
      std::vector<float> wr;
      if (const OnnxAttr* a = n.find("weight_dynamic_ranges")) wr = a->floats;
      if (wr.empty() && n_ranges > 0) {
        // calibration supplies activation ranges only: per-output-channel |max| of the weights, as the
        // exporter writes them
        const size_t per = w.size() / (size_t)wshape[0];
        wr.assign((size_t)wshape[0], 0.f);
        for (size_t i = 0; i < w.size(); ++i) wr[i / per] = std::max(wr[i / per], std::fabs(half_bits_to_float(w[i])));
      }
      unsigned bound = 150000;
      if (const OnnxAttr* a = n.find("output_bound")) bound = (unsigned)a->i;
      else SCN_LOGV("using default output_bound: %u", bound);
      const OnnxAttr* rb = n.find("rulebook");
      const OnnxAttr* act = n.find("activation");
      auto ks = attr_ints3(n, "kernel_size"), st = attr_ints3(n, "stride"), pd = attr_ints3(n, "padding"),
           dl = attr_ints3(n, "dilation");
      if (ks.size() != 3) {
        set_error("node %s: kernel_size must have 3 entries", n.name.c_str());
        return nullptr;
      }
      const OnnxAttr* idr = n.find("input_dynamic_range");
      const OnnxAttr* subm = n.find("subm");
      const OnnxAttr* inv = n.find("inverse");
      out = scn_builder_push_sparse_conv(
          b.get(), n.name.c_str(), x, w.data(), wshape.data(), wr.empty() ? nullptr : wr.data(), (int)wr.size(),
          bias.data(), (int)bias.size(), act ? act->s.c_str() : "", ks.data(), st.size() == 3 ? st.data() : nullptr,
          pd.size() == 3 ? pd.data() : nullptr, dl.size() == 3 ? dl.data() : nullptr,
          range_of(n.input[0]) > 0.f ? range_of(n.input[0]) : (idr ? idr->f : 0.f),
          subm ? (int)subm->i : 0, bound, flp, rb ? rb->s.c_str() : "", prec_of(n, "precision"),
          prec_of(n, "output_precision"), n.output[0].c_str(), inv ? (int)inv->i : 0);
    } else if (n.op_type == "Add" || n.op_type == "QuantAdd") {
      if (n.input.size() < 2 || n.output.empty()) {
        set_error("node %s: Add needs two inputs", n.name.c_str());
        return nullptr;
      }
      const int a = tensor_of(n.input[0]), c = tensor_of(n.input[1]);
      if (a < 0 || c < 0) return nullptr;
      const OnnxAttr* r0 = n.find("input0_dynamic_range");
      const OnnxAttr* r1 = n.find("input1_dynamic_range");
      float ra = r0 ? r0->f : 0.f, rb = r1 ? r1->f : 0.f;
      // calibrated: one shared range for both operands, the larger of the two (what the exporter writes)
      const float shared = std::max(range_of(n.input[0]), range_of(n.input[1]));
      if (shared > 0.f) ra = rb = shared;
      out = scn_builder_push_add(b.get(), n.name.c_str(), a, c, ra, rb, n.output[0].c_str(),
                                 prec_of(n, "precision"), prec_of(n, "output_precision"), fixed_launch_points);
    } else if (n.op_type == "Relu") {
      const int x = n.input.empty() ? -1 : tensor_of(n.input[0]);
      if (x < 0 || n.output.empty()) return nullptr;
      out = scn_builder_push_relu(b.get(), n.name.c_str(), x, n.output[0].c_str());
    } else if (n.op_type == "ScatterDense") {
      const int x = n.input.empty() ? -1 : tensor_of(n.input[0]);
      if (x < 0 || n.output.empty()) return nullptr;
      auto iss = attr_ints3(n, "input_spatial_shape");
      auto os = attr_ints3(n, "output_shape");
      const OnnxAttr* fmt = n.find("format");
      const OnnxAttr* idr = n.find("input_dynamic_range");
      const OnnxAttr* lay = n.find("output_layout");
      int layout = 1;
      if (lay && lay->s == "NCHW32") layout = 2;
      else if (lay && lay->s == "NHWzC") layout = 3;
      out = scn_builder_push_dense(b.get(), n.name.c_str(), x, fmt ? fmt->s.c_str() : "", n.output[0].c_str(),
                                   iss.size() == 3 ? iss.data() : nullptr, os.data(), (int)os.size(), layout,
                                   idr ? idr->f : 0.f, fixed_launch_points);
    } else if (n.op_type == "Reshape" || n.op_type == "Transpose") {
      const int x = n.input.empty() ? -1 : tensor_of(n.input[0]);
      if (x < 0 || n.output.empty()) return nullptr;
      std::vector<int64_t> dims;
      if (const OnnxAttr* a = n.find("dims")) dims = a->ints;
      out = n.op_type == "Reshape"
                ? scn_builder_push_reshape(b.get(), n.name.c_str(), x, dims.data(), (int)dims.size(), n.output[0].c_str())
                : scn_builder_push_transpose(b.get(), n.name.c_str(), x, dims.data(), (int)dims.size(), n.output[0].c_str());
    } else {
      set_error("Unsupport operator [%s]", n.op_type.c_str());
      return nullptr;
    }
    if (out < 0) return nullptr;
    tmap[n.output[0]] = out;
  }
  for (auto& name : g.outputs) {
    const int t = tensor_of(name);
    if (t < 0) return nullptr;
    scn_builder_push_output(b.get(), t);
  }
  return scn_builder_build(b.get(), precision, flags, stream);
}

void scn_engine_destroy(scn_engine* e) { delete e; }
int scn_engine_num_input(const scn_engine* e) { return e ? (int)e->inputs.size() : 0; }
int scn_engine_num_output(const scn_engine* e) { return e ? (int)e->outputs.size() : 0; }

int scn_engine_set_input(scn_engine* e, int index, const void* features_fp16_dev, uint32_t n, uint32_t channels,
                         const int32_t* indices_dev, const int grid_size[3]) {
  SCN_REQUIRE(e && index == 0 && grid_size, SCN_ERR_INVALID, "set_input: invalid engine / index");
  SCN_REQUIRE((features_fp16_dev && indices_dev) || n == 0, SCN_ERR_INVALID, "set_input: null pointers with n > 0");
  const RtTensor& t = e->tensors[e->inputs[0]];
  SCN_REQUIRE(t.c == 0 || (uint32_t)t.c == channels, SCN_ERR_INVALID, "set_input: the model expects %d input channels, got %u",
              t.c, channels);
  SCN_REQUIRE(((uintptr_t)indices_dev & 15) == 0, SCN_ERR_INVALID, "set_input: indices must be 16-byte aligned");
  e->in_feat = features_fp16_dev;
  e->in_idx = indices_dev;
  e->in_n = n;
  e->in_c = channels;
  memcpy(e->in_grid, grid_size, 12);
  e->input_set = true;
  return SCN_OK;
}

int scn_engine_set_num_points_device_ptr(scn_engine* e, int index, const uint32_t* n_dev) {
  SCN_REQUIRE(e && index == 0, SCN_ERR_INVALID, "set_num_points_device_ptr: invalid engine / index");
  e->dds = n_dev;
  return SCN_OK;
}

int scn_engine_prepare(scn_engine* e, const int grid_size[3]) {
  SCN_REQUIRE(e && grid_size, SCN_ERR_INVALID, "prepare: invalid arguments");
  if (e->allocated && memcmp(e->alloc_grid, grid_size, 12) == 0) return SCN_OK;
  memcpy(e->in_grid, grid_size, 12);
  return allocate_runtime(*e);
}

int scn_engine_forward(scn_engine* e, void* stream_) {
  SCN_REQUIRE(e, SCN_ERR_INVALID, "forward: null engine");
  SCN_REQUIRE(e->input_set, SCN_ERR_INVALID, "forward: no input has been set");
  hipStream_t stream = (hipStream_t)stream_;
  if (!e->allocated || memcmp(e->alloc_grid, e->in_grid, 12) != 0) {
    int rc = allocate_runtime(*e);
    if (rc) return rc;
  }
  // Two streams unless per-step profiling is on.  Coordinate work (hash, rulebooks, row maps of the
  // dense outputs) depends on the input coordinates alone, so all of it is enqueued on the auxiliary
  // stream first, in graph order, and runs as far ahead of the feature kernels as the GPU allows; the
  // main stream then waits per rulebook.  The auxiliary stream is in order, so waiting for a rulebook's
  // event also covers everything built before it.
  const bool debug = debug_sync_enabled();
  const bool dual = e->aux != nullptr && !e->profiling && !debug;
  auto is_coord_step = [](const Step& st) {
    return st.kind == StepKind::HashBuild || st.kind == StepKind::RulebookSubm || st.kind == StepKind::RulebookSparse ||
           st.kind == StepKind::RulebookInverse;
  };
  auto fail = [](const Step& st, int rc) {
    SCN_LOGE("forward failed at step %s", st.label.c_str());
    return rc;
  };
  if (dual) {
    int aux_seq = 0, waited_seq = 0;
    e->rb_seq.assign(e->rulebooks.size(), 0);
    e->coord_rb.assign(e->coords.size(), -1);
    e->map_built.assign(e->steps.size(), 0);
    // pass 1: the input count (which also clears what the coordinate kernels build into), then the
    // coordinate steps.  What the first convolution needs (the input hash and its rulebook) stays on the
    // caller's stream: a dependency across streams costs ~12 us from the event to the dependent kernel's
    // start when the waiting stream is idle, and the first convolution would pay that twice (fork and
    // wait).  The auxiliary stream starts as soon as the coordinates and look-ups it reads exist.
    size_t first_conv = e->steps.size();
    for (size_t si = 0; si < e->steps.size(); ++si)
      if (e->steps[si].kind == StepKind::Conv) {
        first_conv = si;
        break;
      }
    bool aux_started = false;
    for (size_t si = 0; si < e->steps.size(); ++si) {
      Step& st = e->steps[si];
      if (st.kind == StepKind::InputCount) {
        int rc = run_step(*e, st, stream);
        if (rc) return fail(st, rc);
        SCN_HIP(hipEventRecord(e->ev_fork, stream));
      } else if (is_coord_step(st) && si < first_conv) {
        int rc = run_step(*e, st, stream);
        if (rc) return fail(st, rc);
        if (st.kind == StepKind::RulebookSparse) e->coord_rb[e->rulebooks[st.rulebook]->coord_out] = st.rulebook;
        // (a submanifold table is read by the convolutions only; the others produce what later builds read)
        if (st.kind != StepKind::RulebookSubm) SCN_HIP(hipEventRecord(e->ev_fork, stream));
      } else if (is_coord_step(st)) {
        if (!aux_started) SCN_HIP(hipStreamWaitEvent(e->aux, e->ev_fork, 0));
        aux_started = true;
        int rc = run_step(*e, st, e->aux);
        if (rc) return fail(st, rc);
        if (st.kind != StepKind::HashBuild) {
          SCN_HIP(hipEventRecord(e->rb_ready[st.rulebook], e->aux));
          e->rb_seq[st.rulebook] = ++aux_seq;
          if (st.kind == StepKind::RulebookSparse) e->coord_rb[e->rulebooks[st.rulebook]->coord_out] = st.rulebook;
        }
      } else if (st.kind == StepKind::Dense && si < e->dense_maps.size() && e->dense_maps[si].p &&
                 e->dense_precleared[si] == 2) {
        if (!aux_started) SCN_HIP(hipStreamWaitEvent(e->aux, e->ev_fork, 0));
        aux_started = true;
        const CoordSet& cs = e->coords[e->tensors[st.t_in].coord];
        int rc = scatter_dense_build_map(cs.idx, cs.n_bound, cs.n_dev, st.dense_shape, st.has_perm ? st.perm : nullptr,
                                         e->dense_maps[si].as<int32_t>(), true, e->aux);
        if (rc) return fail(st, rc);
        e->map_built[si] = 1;
      }
    }
    if (!aux_started) SCN_HIP(hipStreamWaitEvent(e->aux, e->ev_fork, 0));
    SCN_HIP(hipEventRecord(e->ev_join, e->aux));
    // pass 2: the feature kernels
    for (size_t si = 0; si < e->steps.size(); ++si) {
      Step& st = e->steps[si];
      if (st.kind == StepKind::InputCount || is_coord_step(st)) continue;
      // rulebook this step depends on: its own (convolutions) or the one that produced its rows
      int rb = -1;
      if (st.kind == StepKind::Conv) {
        rb = st.rulebook;
      } else if (st.t_in >= 0 && st.t_in < (int)e->tensors.size()) {
        const int c = e->tensors[st.t_in].coord;
        if (c >= 0 && c < (int)e->coord_rb.size()) rb = e->coord_rb[c];
      }
      if (e->map_built[si] && waited_seq <= aux_seq) {
        SCN_HIP(hipStreamWaitEvent(stream, e->ev_join, 0));  // row maps come after every rulebook
        waited_seq = aux_seq + 1;
      } else if (rb >= 0 && e->rb_seq[rb] > waited_seq) {
        // A wait on the other stream costs ~2 us even when its event has long fired.  The table of a strided
        // convolution is followed on the auxiliary stream by the submanifold table of its output
        // coordinates, and the layers that use that one come next: one wait covers both.
        int target = rb;
        if (!e->rulebooks[rb]->subm)
          for (size_t r2 = 0; r2 < e->rb_seq.size(); ++r2)
            if (e->rb_seq[r2] == e->rb_seq[rb] + 1 && e->rulebooks[r2]->subm &&
                e->rulebooks[r2]->coord_in == e->rulebooks[rb]->coord_out)
              target = (int)r2;
        if (e->rb_seq[target] == aux_seq) {
          // the last table: what follows it on the auxiliary stream (row maps) is short; wait for all of it
          SCN_HIP(hipStreamWaitEvent(stream, e->ev_join, 0));
          waited_seq = aux_seq + 1;
        } else {
          SCN_HIP(hipStreamWaitEvent(stream, e->rb_ready[target], 0));
          waited_seq = e->rb_seq[target];
        }
      }
      e->dense_map_built = e->map_built[si] != 0;
      int rc = run_step(*e, st, stream);
      e->dense_map_built = false;
      if (rc) return fail(st, rc);
    }
    if (waited_seq <= aux_seq) SCN_HIP(hipStreamWaitEvent(stream, e->ev_join, 0));
    return SCN_OK;
  }
  for (auto& st : e->steps) {
    if (e->profiling) {
      if (!st.ev0) {
        SCN_HIP(hipEventCreate(&st.ev0));
        SCN_HIP(hipEventCreate(&st.ev1));
      }
      SCN_HIP(hipEventRecord(st.ev0, stream));
    }
    int rc = run_step(*e, st, stream);
    if (rc == SCN_OK && debug) rc = debug_sync_check(stream, st.label.c_str());
    if (rc) return fail(st, rc);
    if (e->profiling) SCN_HIP(hipEventRecord(st.ev1, stream));
  }
  if (e->profiling) {
    SCN_HIP(hipStreamSynchronize(stream));
    for (auto& st : e->steps) SCN_HIP(hipEventElapsedTime(&st.last_ms, st.ev0, st.ev1));
  }
  return SCN_OK;
}

static void fill_view(scn_engine* e, int t, scn_tensor_view* v) {
  const RtTensor& x = e->tensors[t];
  memset(v, 0, sizeof(*v));
  v->name = (t < (int)e->tdesc.size()) ? e->tdesc[t].name.c_str() : "";
  v->features_dev = x.data;
  v->dtype = x.dtype;
  v->dynamic_range = x.range;
  if (x.dense) {
    v->ndim = (int)std::min<size_t>(x.shape.size(), 8);
    for (int j = 0; j < v->ndim; ++j) v->shape[j] = x.shape[j];
  } else {
    const CoordSet& cs = e->coords[x.coord];
    v->ndim = 2;
    v->shape[0] = cs.n_bound;
    v->shape[1] = x.ld;
    v->indices_dev = cs.idx;
    v->num_dev = cs.n_dev;
    memcpy(v->grid_size, cs.grid, 12);
  }
}

int scn_engine_output(scn_engine* e, int index, scn_tensor_view* view) {
  SCN_REQUIRE(e && view && index >= 0 && index < (int)e->outputs.size(), SCN_ERR_INVALID, "output: invalid index");
  fill_view(e, e->outputs[index], view);
  return SCN_OK;
}

int scn_engine_tensor(scn_engine* e, const char* name, scn_tensor_view* view, void** acc_dev) {
  SCN_REQUIRE(e && name && view, SCN_ERR_INVALID, "tensor: invalid arguments");
  auto it = e->tensor_by_name.find(name);
  SCN_REQUIRE(it != e->tensor_by_name.end(), SCN_ERR_INVALID, "tensor '%s' does not exist", name);
  SCN_REQUIRE(e->tensors[it->second].materialised, SCN_ERR_INVALID,
              "tensor '%s' was fused away (build with SCN_BUILD_KEEP_ALL to keep it)", name);
  // (decided by allocate_runtime; before the first forward / prepare nothing is shared yet, and nothing holds values)
  SCN_REQUIRE(!e->tensors[it->second].shared, SCN_ERR_INVALID,
              "tensor '%s' shares its storage with other intermediate tensors and does not hold its values after a "
              "forward (build with SCN_BUILD_KEEP_ALL to keep it, or make it a graph output)", name);
  fill_view(e, it->second, view);
  if (acc_dev) *acc_dev = e->tensors[it->second].acc.p;
  return SCN_OK;
}

int scn_engine_collect_amax(scn_engine* e, void* stream_, scn_tensor_amax* out, int capacity) {
  if (!e || !out || capacity < 0) {
    set_error("collect_amax: invalid arguments");
    return -1;
  }
  hipStream_t stream = (hipStream_t)stream_;
  std::vector<int> which;
  for (size_t t = 0; t < e->tdesc.size() && t < e->tensors.size(); ++t) {
    const RtTensor& x = e->tensors[t];
    if (x.dense || x.coord < 0 || !x.materialised || x.shared) continue;   // (shared storage holds another tensor's bytes by now)
    if ((int)t == e->inputs[0] ? e->in_feat == nullptr : x.data == nullptr) continue;
    which.push_back((int)t);
  }
  if ((int)which.size() > capacity) {
    set_error("collect_amax: %zu tensors, room for %d", which.size(), capacity);
    return -1;
  }
  if (which.empty()) return 0;
  if (e->amax_buf.bytes < which.size() * 16 && !e->amax_buf.alloc(which.size() * 16)) return -1;
  for (size_t i = 0; i < which.size(); ++i) {
    const int t = which[i];
    const RtTensor& x = e->tensors[t];
    const CoordSet& cs = e->coords[x.coord];
    const bool is_input = t == e->inputs[0];
    const int rc = absmax_rows(is_input ? e->in_feat : x.data, is_input ? SCN_DTYPE_FP16 : x.dtype, x.range,
                               (uint32_t)(is_input ? e->in_c : x.c), is_input ? e->in_c : x.ld, cs.n_bound, cs.n_dev,
                               reinterpret_cast<float*>(e->amax_buf.as<char>() + i * 16), stream);
    if (rc) return -1;
  }
  std::vector<float> host(which.size() * 4);
  if (hipMemcpyAsync(host.data(), e->amax_buf.p, which.size() * 16, hipMemcpyDeviceToHost, stream) != hipSuccess ||
      hipStreamSynchronize(stream) != hipSuccess) {
    set_error("collect_amax: copy failed");
    return -1;
  }
  for (size_t i = 0; i < which.size(); ++i) {
    out[i].tensor = e->tdesc[which[i]].name.c_str();
    out[i].amax = host[i * 4];
  }
  return (int)which.size();
}

int scn_engine_set_profiling(scn_engine* e, int enabled) {
  SCN_REQUIRE(e, SCN_ERR_INVALID, "null engine");
  e->profiling = enabled != 0;
  return SCN_OK;
}
int scn_engine_num_nodes(const scn_engine* e) { return e ? (int)e->steps.size() : 0; }
int scn_engine_node_info(scn_engine* e, int node, const char** name, const char** kind, float* last_ms) {
  SCN_REQUIRE(e && node >= 0 && node < (int)e->steps.size(), SCN_ERR_INVALID, "node_info: invalid index");
  static const char* kinds[] = {"input", "hash", "rulebook_subm", "rulebook_sparse", "rulebook_inverse", "convert", "conv", "add", "relu", "dense", "transpose"};
  const Step& s = e->steps[node];
  if (name) *name = s.label.c_str();
  if (kind) *kind = kinds[(int)s.kind];
  if (last_ms) *last_ms = s.last_ms;
  return SCN_OK;
}

}  // extern "C"
