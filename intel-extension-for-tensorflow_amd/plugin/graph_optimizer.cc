// TF_InitGraph: the graph-optimizer half of the plugin.  It carries the quantized subset of the reference's
// native-format pass (itex/core/graph/native_layout/native_layout.cc:113-198, 402-500 and the rewrite rules /
// attribute copies in itex/core/graph/utils/layout_utils.cc:315-355, 497-545): nodes placed on this plugin's
// device whose op has an _ITEX twin are renamed to it, with the attributes the twin adds.  For QuantizeV2
// that rename is not cosmetic: _ITEXQuantizeV2 receives classic_asymmetric_algorithm = "all consumers are
// Dequantize", which selects the zero-point form of MIN_FIRST instead of the legacy one.
// ITEX_AMD_NATIVE_FORMAT=0 leaves graphs untouched.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>
#include <string>
#include <vector>

#include "graph_def.h"
#include "tf_grappler_subset.h"

namespace itex_amd {
namespace {

constexpr int kDtFloat = 1, kDtQint8 = 11, kDtQuint8 = 12;

enum class Copy { kAll, kQuantize, kQuantizedMatMul, kQuantizedConv2D };
enum class Rule { kAlways, kQuantize, kQint8Only };

struct Rename {
  const char* from;
  const char* to;
  Copy copy;
  Rule rule;
};

// the INT8 rows of the reference's table whose targets this plugin registers kernels for
const Rename kTable[] = {
    {"Dequantize", "_ITEXDequantize", Copy::kAll, Rule::kQuantize},
    {"QuantizeV2", "_ITEXQuantizeV2", Copy::kQuantize, Rule::kQuantize},
    {"QuantizedConv2D", "_ITEXQuantizedConv2D", Copy::kQuantizedConv2D, Rule::kAlways},
    {"QuantizedConv2DAndRequantize", "_ITEXQuantizedConv2DAndRequantize", Copy::kQuantizedConv2D, Rule::kAlways},
    {"QuantizedConv2DPerChannel", "_ITEXQuantizedConv2DPerChannel", Copy::kQuantizedConv2D, Rule::kAlways},
    {"QuantizedConv2DWithBias", "_ITEXQuantizedConv2DWithBias", Copy::kQuantizedConv2D, Rule::kAlways},
    {"QuantizedConv2DWithBiasAndRelu", "_ITEXQuantizedConv2DWithBiasAndRelu", Copy::kQuantizedConv2D, Rule::kAlways},
    {"QuantizedConv2DWithBiasAndReluAndRequantize", "_ITEXQuantizedConv2DWithBiasAndReluAndRequantize", Copy::kQuantizedConv2D, Rule::kAlways},
    {"QuantizedConv2DWithBiasAndRequantize", "_ITEXQuantizedConv2DWithBiasAndRequantize", Copy::kQuantizedConv2D, Rule::kAlways},
    {"QuantizedConv2DWithBiasSumAndReluAndRequantize", "_ITEXQuantizedConv2DWithBiasSumAndReluAndRequantize", Copy::kQuantizedConv2D, Rule::kAlways},
    {"QuantizedConv2DWithBiasSignedSumAndReluAndRequantize", "_ITEXQuantizedConv2DWithBiasSignedSumAndReluAndRequantize", Copy::kQuantizedConv2D, Rule::kAlways},
    {"_QuantizedConv2D", "_ITEXQuantizedConv2DV2", Copy::kAll, Rule::kAlways},
    {"QuantizedDepthwiseConv2D", "_ITEXQuantizedDepthwiseConv2D", Copy::kQuantizedConv2D, Rule::kAlways},
    {"QuantizedDepthwiseConv2DWithBias", "_ITEXQuantizedDepthwiseConv2DWithBias", Copy::kQuantizedConv2D, Rule::kAlways},
    {"QuantizedDepthwiseConv2DWithBiasAndRelu", "_ITEXQuantizedDepthwiseConv2DWithBiasAndRelu", Copy::kQuantizedConv2D, Rule::kAlways},
    {"QuantizedDepthwiseConv2DWithBiasAndReluAndRequantize", "_ITEXQuantizedDepthwiseConv2DWithBiasAndReluAndRequantize", Copy::kQuantizedConv2D, Rule::kAlways},
    {"_QuantizedDepthwiseConv2D", "_ITEXQuantizedDepthwiseConv2DV2", Copy::kAll, Rule::kAlways},
    {"QuantizedMatMulWithBias", "_ITEXQuantizedMatMulWithBias", Copy::kQuantizedMatMul, Rule::kAlways},
    {"QuantizedMatMulWithBiasAndDequantize", "_ITEXQuantizedMatMulWithBiasAndDequantize", Copy::kQuantizedMatMul, Rule::kAlways},
    {"QuantizedMatMulWithBiasAndRelu", "_ITEXQuantizedMatMulWithBiasAndRelu", Copy::kQuantizedMatMul, Rule::kAlways},
    {"QuantizedMatMulWithBiasAndReluAndRequantize", "_ITEXQuantizedMatMulWithBiasAndReluAndRequantize", Copy::kQuantizedMatMul,
     Rule::kAlways},
    {"QuantizedMatMulWithBiasAndRequantize", "_ITEXQuantizedMatMulWithBiasAndRequantize", Copy::kQuantizedMatMul, Rule::kAlways},
    {"_QuantizedBatchMatMul", "_ITEXQuantizedBatchMatMul", Copy::kAll, Rule::kAlways},
    {"_QuantizedBatchMatMulV2AndDequantize", "_ITEXQuantizedBatchMatMulV2AndDequantize", Copy::kAll, Rule::kAlways},
    {"_QuantizedFusedBatchMatMulV2AndDequantize", "_ITEXQuantizedFusedBatchMatMulV2AndDequantize", Copy::kAll, Rule::kAlways},
    {"_QuantizedFusedMatMul", "_ITEXQuantizedFusedMatMul", Copy::kQuantizedMatMul, Rule::kAlways},
    {"_QuantizedFusedMatMulAndDequantize", "_ITEXQuantizedFusedMatMulAndDequantize", Copy::kQuantizedMatMul, Rule::kAlways},
    {"_QuantizedFusedMatMulAndRequantize", "_ITEXQuantizedFusedMatMulAndRequantize", Copy::kQuantizedMatMul, Rule::kAlways},
    {"_QuantizedMatMul", "_ITEXQuantizedMatMul", Copy::kAll, Rule::kAlways},
    {"QuantizedReshape", "_ITEXQuantizedReshape", Copy::kAll, Rule::kQint8Only},  // RewriteQuantizeReshape, layout_utils.cc:392-400
    {"_QuantizedTranspose", "_ITEXQuantizedTranspose", Copy::kAll, Rule::kAlways},
};

std::string DeviceType() {
  const char* dev = std::getenv("ITEX_AMD_DEVICE_TYPE");
  return dev && dev[0] ? dev : "XPU";
}

// the producer named by a data input: "name", "name:port"; control inputs ("^name") carry no tensor
bool SplitInput(const std::string& in, std::string* name, int* port) {
  if (in.empty() || in[0] == '^') return false;
  const size_t colon = in.rfind(':');
  if (colon == std::string::npos) { *name = in; *port = 0; return true; }
  *name = in.substr(0, colon);
  *port = std::atoi(in.c_str() + colon + 1);
  return true;
}

// layout_utils.cc:661-677: QuantizeV2 / Dequantize are only rewritten for T in {qint8, quint8}
bool SupportedType(const graph::Node& n) {
  if (n.op != "QuantizeV2" && n.op != "Dequantize") return true;
  int t = 0;
  const std::string* a = n.FindAttr("T");
  return a && graph::AttrType(*a, &t) && (t == kDtQint8 || t == kDtQuint8);
}

// layout_utils.cc:315-355.  (Its refusal of MIN_FIRST Dequantize on a GPU does not apply: the kernel
// this plugin registers implements that mode.)
bool RewriteQuantize(const graph::Node& n) {
  std::string mode, round_mode;
  const std::string* m = n.FindAttr("mode");
  if (!m || !graph::AttrString(*m, &mode)) return false;
  if (mode == "MIN_COMBINED") return false;
  const std::string* r = n.FindAttr("round_mode");
  if (r && graph::AttrString(*r, &round_mode) && mode == "SCALED" && round_mode != "HALF_TO_EVEN") return false;
  return true;
}

// "name" and "name:0" name the same tensor
std::string Canonical(const std::string& in) {
  std::string name;
  int port = 0;
  if (!SplitInput(in, &name, &port)) return in;
  return name + ":" + std::to_string(port);
}

std::vector<std::string> DataInputs(const graph::Node& n) {
  std::vector<std::string> v;
  for (const std::string& in : n.inputs)
    if (!in.empty() && in[0] != '^') v.push_back(in);
  return v;
}

// QuantizeV2(x, Min(Reshape(x, [-1]), 0), Max(Reshape(x, [-1]), 0)): the per-tensor dynamic-range quantization that
// TensorFlow's graph quantization tools emit.  Without Min / Max kernels for this device TensorFlow would place the
// two reductions on the CPU and copy the whole float tensor to the host for them; the fused op computes the range on
// the device.  The reference has no such fusion for QuantizeV2 (its remapper fuses QuantizeV2 into convolutions only,
// itex/core/graph/remapper/remapper.cc:2099-2114).  Returns true when node q matches.
bool MatchDynamicRange(const graph::Node& q, const std::map<std::string, const graph::Node*>& by_name) {
  int axis = -1;
  const std::string* a = q.FindAttr("axis");
  if (a && !a->empty() && !graph::AttrInt(*a, &axis)) return false;
  if (axis != -1) return false;
  const std::vector<std::string> in = DataInputs(q);
  if (in.size() != 3) return false;
  auto node_of = [&](const std::string& input, int want_port) -> const graph::Node* {
    std::string name;
    int port = 0;
    if (!SplitInput(input, &name, &port) || port != want_port) return nullptr;
    const auto it = by_name.find(name);
    return it == by_name.end() ? nullptr : it->second;
  };
  auto const_ints = [&](const std::string& input, int* rank, std::vector<int64_t>* vals) {
    const graph::Node* c = node_of(input, 0);
    if (!c || c->op != "Const") return false;
    const std::string* v = c->FindAttr("value");
    return v && graph::AttrIntTensor(*v, rank, vals);
  };
  const graph::Node* mn = node_of(in[1], 0);
  const graph::Node* mx = node_of(in[2], 0);
  if (!mn || !mx || mn->op != "Min" || mx->op != "Max") return false;
  std::string reduced;
  for (const graph::Node* red : {mn, mx}) {
    bool keep = false;
    const std::string* k = red->FindAttr("keep_dims");
    if (k && (!graph::AttrBool(*k, &keep) || keep)) return false;
    const std::vector<std::string> rin = DataInputs(*red);
    if (rin.size() != 2) return false;
    int rank = 0;
    std::vector<int64_t> idx;
    if (!const_ints(rin[1], &rank, &idx) || rank > 1 || idx.size() != 1 || idx[0] != 0) return false;  // reduce dimension 0
    if (reduced.empty()) reduced = Canonical(rin[0]);
    else if (reduced != Canonical(rin[0])) return false;
  }
  const graph::Node* flat = node_of(reduced, 0);  // of a tensor flattened to one dimension
  if (!flat || flat->op != "Reshape") return false;
  const std::vector<std::string> fin = DataInputs(*flat);
  if (fin.size() != 2 || Canonical(fin[0]) != Canonical(in[0])) return false;
  int rank = 0;
  std::vector<int64_t> shape;
  return const_ints(fin[1], &rank, &shape) && rank == 1 && shape.size() == 1 && shape[0] == -1;
}

// _ITEXQuantizeV2DynamicRange(x) -> _ITEXQuantizedMatMul becomes one node, _ITEXQuantizedMatMulDynamicInput(x, ...): the
// range of x, its quantization and the product are enqueued back to back and the range never crosses to the host
// (as separate nodes, output_min / output_max of the first are host tensors, so every step waits for the reduction).
// The reference fuses QuantizeV2 into its consumer for convolutions only (remapper.cc:2099-2114).  Conditions: the
// MatMul is the only reader of all three outputs, both nodes sit on the same device, the quantization parameters
// agree (T1 / input_quant_mode), the MatMul has no addend and a Requantize or Dequantize output (the range of a
// qint32 result is host math on the activation range).  Returns the number of fused pairs.
int FuseDynamicQuantizeIntoMatMul(graph::Graph* g, const std::set<std::string>& preserve) {
  std::map<std::string, size_t> index;
  std::map<std::string, std::vector<size_t>> readers;  // by producer name: every node with a data or control input from it
  for (size_t i = 0; i < g->nodes.size(); ++i) {
    index[g->nodes[i].name] = i;
    for (const std::string& in : g->nodes[i].inputs) {
      std::string producer;
      int port = 0;
      if (!in.empty() && in[0] == '^') producer = in.substr(1);
      else if (!SplitInput(in, &producer, &port)) continue;
      readers[producer].push_back(i);
    }
  }
  std::vector<bool> dead(g->nodes.size(), false);
  int fused = 0;
  for (size_t mi = 0; mi < g->nodes.size(); ++mi) {
    graph::Node& m = g->nodes[mi];
    if (m.op != "_ITEXQuantizedMatMul") continue;
    const std::vector<std::string> data = DataInputs(m);
    if (data.size() != 7 && data.size() != 9) continue;  // a, w, bias, min_a, max_a, min_b, max_b [, min_out, max_out]
    std::string qname;
    int port = 0;
    if (!SplitInput(data[0], &qname, &port) || port != 0) continue;
    const auto qi = index.find(qname);
    if (qi == index.end() || dead[qi->second]) continue;
    const graph::Node& q = g->nodes[qi->second];
    if (q.op != "_ITEXQuantizeV2DynamicRange" || q.device != m.device) continue;
    // a fetched or preserved quantize node has readers outside the graph (its tensor or its range is a session
    // result): it stays, as the reference keeps preserved nodes out of every fusion (remapper.cc:6373-6390)
    if (preserve.count(qname)) continue;
    if (Canonical(data[3]) != qname + ":1" || Canonical(data[4]) != qname + ":2") continue;
    bool only_reader = true;
    for (size_t r : readers[qname]) only_reader = only_reader && r == mi;
    if (!only_reader) continue;
    // the MatMul's side
    std::vector<int> dev_types, host_types;
    std::vector<std::string> fused_ops;
    const std::string *tdi = m.FindAttr("Tdevice_inputs"), *thi = m.FindAttr("Thost_inputs"), *fo = m.FindAttr("fused_ops");
    if (!tdi || !thi || !fo || !graph::AttrTypeList(*tdi, &dev_types) || !graph::AttrTypeList(*thi, &host_types) ||
        !graph::AttrStringList(*fo, &fused_ops))
      continue;
    if (dev_types.size() != 3 || host_types.size() + 3 != data.size()) continue;
    bool out_given = false, has_add = false;
    for (const std::string& f : fused_ops) {
      out_given = out_given || f == "Requantize" || f == "Dequantize";
      has_add = has_add || f == "Add";
    }
    if (!out_given || has_add) continue;
    bool transpose_a = false;
    if (const std::string* ta = m.FindAttr("transpose_a")) {
      if (!graph::AttrBool(*ta, &transpose_a) || transpose_a) continue;
    }
    // the quantization's side
    int t_q = 0, t1 = 0, axis = -1;
    std::string q_mode, m_mode = "SCALED";
    const std::string *qt = q.FindAttr("T"), *mt = m.FindAttr("T1"), *qm = q.FindAttr("mode");
    if (!qt || !mt || !graph::AttrType(*qt, &t_q) || !graph::AttrType(*mt, &t1) || t_q != t1 || dev_types[0] != t1) continue;
    if (!qm || !graph::AttrString(*qm, &q_mode)) continue;
    if (const std::string* mm = m.FindAttr("input_quant_mode")) {
      if (!graph::AttrString(*mm, &m_mode)) continue;
    }
    if (q_mode != m_mode || (q_mode != "SCALED" && !(q_mode == "MIN_FIRST" && t_q == kDtQuint8))) continue;
    if (const std::string* ax = q.FindAttr("axis")) {
      if (!ax->empty() && (!graph::AttrInt(*ax, &axis) || axis != -1)) continue;
    }
    const std::vector<std::string> q_data = DataInputs(q);
    if (q_data.size() != 1) continue;
    // ---- rewrite
    std::vector<std::string> inputs = {q_data[0], data[1], data[2]};
    for (size_t k = 5; k < data.size(); ++k) inputs.push_back(data[k]);
    for (const graph::Node* from : {static_cast<const graph::Node*>(&m), &q})
      for (const std::string& in : from->inputs)
        if (!in.empty() && in[0] == '^' && std::find(inputs.begin(), inputs.end(), in) == inputs.end()) inputs.push_back(in);
    dev_types[0] = kDtFloat;
    host_types.erase(host_types.begin(), host_types.begin() + 2);
    if (const std::string* emr = q.FindAttr("ensure_minimum_range")) m.SetAttr("ensure_minimum_range", *emr);
    m.SetAttr("Tdevice_inputs", graph::MakeAttrTypeList(dev_types));
    m.SetAttr("Thost_inputs", graph::MakeAttrTypeList(host_types));
    m.inputs = inputs;
    m.op = "_ITEXQuantizedMatMulDynamicInput";
    dead[qi->second] = true;
    ++fused;
  }
  if (fused) {
    std::vector<graph::Node> kept;
    for (size_t i = 0; i < g->nodes.size(); ++i)
      if (!dead[i]) kept.push_back(std::move(g->nodes[i]));
    g->nodes.swap(kept);
  }
  return fused;
}

struct Optimizer {
  std::string device_type;
};

void* Create() { return new Optimizer{DeviceType()}; }
void Destroy(void* o) { delete static_cast<Optimizer*>(o); }

void FreeBuffer(void* data, size_t) { std::free(data); }

// names the session fetches or asked to keep (itex/core/graph/utils/grappler_item.cc:23-68); a fetch may name a port
std::set<std::string> NamesToKeep(const TF_GrapplerItem* item) {
  std::set<std::string> keep;
  if (item == nullptr) return keep;
  using SizeFn = void (*)(const TF_GrapplerItem*, int*, size_t*, TF_Status*);
  using ListFn = void (*)(const TF_GrapplerItem*, char**, size_t*, int, void*, size_t, TF_Status*);
  const std::pair<SizeFn, ListFn> lists[2] = {{TF_GetNodesToPreserveListSize, TF_GetNodesToPreserveList},
                                              {TF_GetFetchNodesListSize, TF_GetFetchNodesList}};
  TF_Status* st = TF_NewStatus();
  for (const auto& fn : lists) {
    int count = 0;
    size_t storage_size = 0;
    fn.first(item, &count, &storage_size, st);
    if (TF_GetCode(st) != TF_OK || count <= 0) continue;
    std::vector<char*> values(count);
    std::vector<size_t> lengths(count);
    std::vector<char> storage(storage_size + 1);
    fn.second(item, values.data(), lengths.data(), count, storage.data(), storage_size, st);
    if (TF_GetCode(st) != TF_OK) continue;
    for (int i = 0; i < count; ++i) {
      std::string name(values[i], lengths[i]);
      const size_t colon = name.find(':');
      if (colon != std::string::npos) name.resize(colon);
      if (!name.empty() && name[0] == '^') name.erase(0, 1);
      keep.insert(name);
    }
  }
  TF_DeleteStatus(st);
  return keep;
}

void Optimize(void* opt, const TF_Buffer* in, const TF_GrapplerItem* item, TF_Buffer* out, TF_Status* status) {
  const Optimizer* self = static_cast<const Optimizer*>(opt);
  graph::Graph g;
  if (!graph::Parse(in->data, in->length, &g)) {
    TF_SetStatus(status, TF_INVALID_ARGUMENT, "itex_amd graph optimizer: the GraphDef could not be parsed");
    return;
  }
  const char* sw = std::getenv("ITEX_AMD_NATIVE_FORMAT");
  const bool enabled = !(sw && std::strcmp(sw, "0") == 0);

  // consumers of output 0 of every node, by op name (for CopyAttrsQuantize)
  std::map<std::string, std::vector<const graph::Node*>> fanout0;
  for (const graph::Node& n : g.nodes)
    for (const std::string& in_name : n.inputs) {
      std::string producer;
      int port = 0;
      if (SplitInput(in_name, &producer, &port) && port == 0) fanout0[producer].push_back(&n);
    }
  std::map<std::string, const graph::Node*> by_name;
  for (const graph::Node& n : g.nodes) by_name[n.name] = &n;
  const char* dsw = std::getenv("ITEX_AMD_FUSE_DYNAMIC_RANGE");
  const bool fuse_dynamic = !(dsw && std::strcmp(dsw, "0") == 0);
  // decisions first, on the unmodified graph: a QuantizeV2's consumers are looked up by their original op
  std::vector<const Rename*> plan(g.nodes.size(), nullptr);
  std::vector<bool> classic(g.nodes.size(), false), dynamic(g.nodes.size(), false);
  for (size_t i = 0; enabled && i < g.nodes.size(); ++i) {
    const graph::Node& n = g.nodes[i];
    // NodeIsOnDevice (utils.cc:262-265): the node carries a device string naming this device type
    if (n.device.empty() || n.device.find(self->device_type) == std::string::npos) continue;
    if (!SupportedType(n)) continue;
    for (const Rename& r : kTable) {
      if (n.op != r.from) continue;
      if (r.rule == Rule::kQuantize && !RewriteQuantize(n)) break;
      if (r.rule == Rule::kQint8Only) {
        int t = 0;
        const std::string* a = n.FindAttr("T");
        if (!a || !graph::AttrType(*a, &t) || t != kDtQint8) break;
      }
      plan[i] = &r;
      if (r.copy == Copy::kQuantize) {  // layout_utils.cc:530-541
        bool all_dequantize = true;
        for (const graph::Node* c : fanout0[n.name]) all_dequantize = all_dequantize && c->op == "Dequantize";
        classic[i] = all_dequantize;
        dynamic[i] = fuse_dynamic && n.op == "QuantizeV2" && MatchDynamicRange(n, by_name);
      }
      break;
    }
  }
  for (size_t i = 0; i < g.nodes.size(); ++i) {
    if (!plan[i]) continue;
    graph::Node& n = g.nodes[i];  // name, inputs (control inputs included), device and attributes stay (RewriteNode :411-441)
    n.op = plan[i]->to;
    if (plan[i]->copy == Copy::kQuantize) {
      if (!n.FindAttr("dtype")) n.SetAttr("dtype", graph::MakeAttrType(kDtFloat));
      n.SetAttr("classic_asymmetric_algorithm", graph::MakeAttrBool(classic[i]));
      if (dynamic[i]) {  // the range inputs go; Min, Max and Reshape stay for whoever else reads them (else they are pruned)
        n.op = "_ITEXQuantizeV2DynamicRange";
        std::vector<std::string> kept;
        int data = 0;
        for (const std::string& in_name : n.inputs)
          if ((!in_name.empty() && in_name[0] == '^') || data++ == 0) kept.push_back(in_name);
        n.inputs = kept;
      }
    }
    if (plan[i]->copy == Copy::kQuantizedConv2D) n.SetAttr("data_format", graph::MakeAttrString("NHWC"));  // :471-495
    // CopyAttrsQuantizedMatMul (:497-515) copies every attribute and then Tbias once more: nothing to add
  }

  const char* msw = std::getenv("ITEX_AMD_FUSE_QUANTIZE_MATMUL");
  if (enabled && fuse_dynamic && !(msw && std::strcmp(msw, "0") == 0)) FuseDynamicQuantizeIntoMatMul(&g, NamesToKeep(item));

  const std::string bytes = graph::Serialize(g);
  void* mem = std::malloc(bytes.size() ? bytes.size() : 1);
  if (!mem) {
    TF_SetStatus(status, TF_INTERNAL, "itex_amd graph optimizer: out of memory");
    return;
  }
  std::memcpy(mem, bytes.data(), bytes.size());
  out->data = mem;
  out->length = bytes.size();
  out->data_deallocator = FreeBuffer;
  TF_SetStatus(status, TF_OK, "");
}

}  // namespace
}  // namespace itex_amd

// itex/core/graph/xpu_graph.cc:137-176
extern "C" void TF_InitGraph(TP_OptimizerRegistrationParams* params, TF_Status* status) {
  params->struct_size = TP_OPTIMIZER_REGISTRATION_PARAMS_STRUCT_SIZE;
  params->optimizer_configs->struct_size = TP_OPTIMIZER_CONFIGS_STRUCT_SIZE;
  params->optimizer->struct_size = TP_OPTIMIZER_STRUCT_SIZE;
  params->major_version = GO_MAJOR;
  params->minor_version = GO_MINOR;
  params->patch_version = GO_PATCH;
  // TensorFlow's own remapper and layout optimizer stay off while a plugin optimizer is registered, as the
  // reference sets them (:146-148); this pass does not depend on the others
  params->optimizer_configs->remapping = TF_TriState_Off;
  params->optimizer_configs->layout_optimizer = TF_TriState_Off;
  static std::string device_type;  // must outlive the call
  device_type = itex_amd::DeviceType();
  params->device_type = device_type.c_str();
  params->optimizer->create_func = itex_amd::Create;
  params->optimizer->optimize_func = itex_amd::Optimize;
  params->optimizer->destroy_func = itex_amd::Destroy;
  TF_SetStatus(status, TF_OK, "");
}
