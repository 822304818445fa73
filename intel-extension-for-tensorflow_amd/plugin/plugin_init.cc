// Plugin entry point.  TensorFlow calls TF_InitKernel() once after dlopen()ing the library
// (itex/core/wrapper/itex_cpu_wrapper.cc:99-112 -> itex/core/kernels/xpu_kernel.cc:39-118): register
// the op definitions stock TensorFlow lacks, then every kernel of the INT8 path.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <set>
#include <string>
#include <vector>

#include "op_kernel.h"

namespace itex_amd {
namespace {

// ---- names of the ops TensorFlow already knows: a walk over the serialized OpList
// (OpList { repeated OpDef op = 1; }  OpDef { string name = 1; ... }), itex/core/ops/op_init.cc:31-59
bool ReadVarint(const uint8_t*& p, const uint8_t* end, uint64_t* v) {
  *v = 0;
  for (int shift = 0; p < end && shift < 64; shift += 7) {
    const uint8_t b = *p++;
    *v |= static_cast<uint64_t>(b & 0x7f) << shift;
    if (!(b & 0x80)) return true;
  }
  return false;
}
bool SkipField(const uint8_t*& p, const uint8_t* end, uint32_t wire) {
  uint64_t v;
  switch (wire) {
    case 0: return ReadVarint(p, end, &v);
    case 1: if (end - p < 8) return false; p += 8; return true;
    case 2: if (!ReadVarint(p, end, &v) || static_cast<uint64_t>(end - p) < v) return false; p += v; return true;
    case 5: if (end - p < 4) return false; p += 4; return true;
    default: return false;
  }
}
std::set<std::string> KnownOps() {
  std::set<std::string> names;
  TF_Buffer* buf = TF_GetAllOpList();
  if (buf == nullptr) return names;
  const uint8_t* p = static_cast<const uint8_t*>(buf->data);
  const uint8_t* end = p + buf->length;
  while (p < end) {
    uint64_t tag, len;
    if (!ReadVarint(p, end, &tag)) break;
    if ((tag >> 3) == 1 && (tag & 7) == 2) {  // one OpDef
      if (!ReadVarint(p, end, &len) || static_cast<uint64_t>(end - p) < len) break;
      const uint8_t* q = p;
      const uint8_t* qend = p + len;
      while (q < qend) {
        uint64_t t2, l2;
        if (!ReadVarint(q, qend, &t2)) break;
        if ((t2 >> 3) == 1 && (t2 & 7) == 2) {
          if (!ReadVarint(q, qend, &l2) || static_cast<uint64_t>(qend - q) < l2) break;
          names.emplace(reinterpret_cast<const char*>(q), static_cast<size_t>(l2));
          break;
        }
        if (!SkipField(q, qend, static_cast<uint32_t>(t2 & 7))) break;
      }
      p = qend;
    } else if (!SkipField(p, end, static_cast<uint32_t>(tag & 7))) {
      break;
    }
  }
  TF_DeleteBuffer(buf);
  return names;
}

void UnknownShape(TF_ShapeInferenceContext* ctx, TF_Status* status) { TF_ShapeInferenceContextSetUnknownShape(ctx, status); }

struct OpSpec {
  const char* name;
  std::vector<const char*> inputs, outputs, attrs;
};

// Signatures as defined by the reference: itex/core/ops/nn_ops.cc:379-495 (V1 fused MatMul),
// :1070-1127 (_ITEXQuantizeV2 / _ITEXDequantize), :4451-4573 (_QuantizedMatMul, _ITEXQuantizedMatMul).
std::vector<OpSpec> OpSpecs() {
  std::vector<OpSpec> v;
  v.push_back({"_ITEXQuantizeV2",
               {"input: dtype", "min_range: float", "max_range: float"},
               {"output: T", "output_min: float", "output_max: float"},
               {"T: quantizedtype", "mode: {'MIN_COMBINED', 'MIN_FIRST', 'SCALED'} = 'SCALED'",
                "round_mode: {'HALF_AWAY_FROM_ZERO', 'HALF_TO_EVEN'} = 'HALF_AWAY_FROM_ZERO'",
                "narrow_range: bool = false", "axis: int = -1", "ensure_minimum_range: float = 0.01",
                "dtype: {bfloat16, float} = DT_FLOAT", "classic_asymmetric_algorithm: bool = false"}});
  // made by this plugin's graph pass from QuantizeV2 fed by Min / Max of its own input: no range inputs
  v.push_back({"_ITEXQuantizeV2DynamicRange",
               {"input: dtype"},
               {"output: T", "output_min: float", "output_max: float"},
               {"T: quantizedtype", "mode: {'MIN_COMBINED', 'MIN_FIRST', 'SCALED'} = 'SCALED'",
                "round_mode: {'HALF_AWAY_FROM_ZERO', 'HALF_TO_EVEN'} = 'HALF_AWAY_FROM_ZERO'",
                "narrow_range: bool = false", "axis: int = -1", "ensure_minimum_range: float = 0.01",
                "dtype: {float} = DT_FLOAT", "classic_asymmetric_algorithm: bool = false"}});
  v.push_back({"_ITEXDequantize",
               {"input: T", "min_range: float", "max_range: float"},
               {"output: dtype"},
               {"T: quantizedtype", "mode: {'MIN_COMBINED', 'MIN_FIRST', 'SCALED'} = 'SCALED'",
                "narrow_range: bool = false", "axis: int = -1", "dtype: {bfloat16, float} = DT_FLOAT"}});
  for (const char* name : {"_QuantizedMatMul", "_ITEXQuantizedMatMul", "_ITEXQuantizedMatMulDynamicInput"}) {
    v.push_back({name,
                 {"device_inputs: Tdevice_inputs", "host_inputs: Thost_inputs"},
                 {"device_outputs: Tdevice_outputs", "host_outputs: Thost_outputs"},
                 {"Tdevice_inputs: list(type) >= 0 = []", "Thost_inputs: list(type) >= 0 = []",
                  "Tdevice_outputs: list(type) >= 0 = []", "Thost_outputs: list(type) >= 0 = []",
                  "T1: quantizedtype", "T2: quantizedtype", "Tbias: {bfloat16, float, quantizedtype} = DT_FLOAT",
                  "U: {bfloat16, float, quantizedtype} = DT_FLOAT", "Tout: {bfloat16, float, quantizedtype} = DT_FLOAT",
                  "transpose_a: bool = false", "transpose_b: bool = false", "is_weight_const: bool = true",
                  "is_bias_const: bool = true", "fused_ops: list(string) = []",
                  "input_quant_mode: {'MIN_FIRST', 'SCALED'} = 'SCALED'",
                  "output_quant_mode: {'MIN_FIRST', 'SCALED'} = 'SCALED'", "leakyrelu_alpha: float = 0.2"}});
    // the last name is made by this plugin's graph pass from _ITEXQuantizeV2DynamicRange -> _ITEXQuantizedMatMul:
    // device_inputs[0] is the float tensor, host_inputs start at min_b, and the quantization's range floor comes along
    if (std::strcmp(name, "_ITEXQuantizedMatMulDynamicInput") == 0) v.back().attrs.push_back("ensure_minimum_range: float = 0.01");
  }
  const std::vector<const char*> v1_attrs = {
      "T1: quantizedtype", "T2: quantizedtype", "num_args: int >= 0", "Targs: {float, bfloat16, half, quantizedtype}",
      "transpose_a: bool = false", "transpose_b: bool = false", "fused_ops: list(string) = []",
      "is_filter_const: bool = true", "is_bias_const: bool = true", "epsilon: float = 0.0001",
      "leakyrelu_alpha: float = 0.2", "input_quant_mode: {'MIN_FIRST', 'SCALED'} = 'SCALED'"};
  for (const char* prefix : {"_", "_ITEX"}) {
    static std::vector<std::string> keep;  // the table stores pointers
    auto nm = [&](const char* tail) { keep.push_back(std::string(prefix) + tail); return keep.back().c_str(); };
    OpSpec plain{nm("QuantizedFusedMatMul"),
                 {"a: T1", "b: T2", "args: num_args * Targs", "min_a: float", "max_a: float", "min_b: float", "max_b: float"},
                 {"product: Toutput", "min_product: float", "max_product: float"}, v1_attrs};
    plain.attrs.push_back("Toutput: quantizedtype");
    OpSpec req{nm("QuantizedFusedMatMulAndRequantize"),
               {"a: T1", "b: T2", "args: num_args * Targs", "min_a: float", "max_a: float", "min_b: float", "max_b: float",
                "min_freezed_output: float", "max_freezed_output: float"},
               {"product: Toutput", "min_product: float", "max_product: float"}, v1_attrs};
    req.attrs.push_back("Toutput: quantizedtype");
    OpSpec deq{nm("QuantizedFusedMatMulAndDequantize"),
               {"a: T1", "b: T2", "args: num_args * Targs", "min_a: float", "max_a: float", "min_b: float", "max_b: float"},
               {"product: Toutput"}, v1_attrs};
    deq.attrs.push_back("Toutput: {float, bfloat16, half} = DT_FLOAT");
    v.push_back(plain);
    v.push_back(req);
    v.push_back(deq);
    // quantized BatchMatMul, nn_ops.cc:497-560 and :3881-3945
    const std::vector<const char*> bmm_attrs = {"T1: quantizedtype", "T2: quantizedtype",
                                                "Toutput: {bfloat16, half, float} = DT_FLOAT", "adj_x: bool = false",
                                                "adj_y: bool = false", "is_filter_const: bool = false"};
    OpSpec bmm{nm("QuantizedBatchMatMulV2AndDequantize"),
               {"x: T1", "y: T2", "min_x: float", "max_x: float", "min_y: float", "max_y: float"},
               {"output: Toutput"}, bmm_attrs};
    OpSpec fbmm{nm("QuantizedFusedBatchMatMulV2AndDequantize"),
                {"x: T1", "y: T2", "args: num_args * T", "min_x: float", "max_x: float", "min_y: float", "max_y: float"},
                {"output: Toutput"}, bmm_attrs};
    fbmm.attrs.push_back("T: {bfloat16, half, float} = DT_FLOAT");
    fbmm.attrs.push_back("num_args: int >= 0");
    fbmm.attrs.push_back("fused_ops: list(string) = []");
    v.push_back(bmm);
    v.push_back(fbmm);
  }
  // the _ITEX twins of TensorFlow's QuantizedMatMulWithBias* ops, nn_ops.cc:1600-1770
  {
    const std::vector<const char*> in7 = {"a: T1", "b: T2", "bias: Tbias", "min_a: float", "max_a: float", "min_b: float",
                                          "max_b: float"};
    std::vector<const char*> in9 = in7;
    in9.push_back("min_freezed_output: float");
    in9.push_back("max_freezed_output: float");
    const std::vector<const char*> out3 = {"out: Toutput", "min_out: float", "max_out: float"};
    auto attrs = [](const char* tbias, const char* toutput) {
      std::vector<const char*> a = {"T1: quantizedtype", "T2: quantizedtype"};
      if (tbias) a.push_back(tbias);
      a.push_back(toutput);
      for (const char* x : {"transpose_a: bool = false", "transpose_b: bool = false",
                            "input_quant_mode: {'MIN_FIRST', 'SCALED'} = 'MIN_FIRST'", "is_weight_const: bool = true"})
        a.push_back(x);
      return a;
    };
    v.push_back({"_ITEXQuantizedMatMulWithBias", in7, out3, attrs("Tbias: {float, qint32}", "Toutput: quantizedtype = DT_QINT32")});
    std::vector<const char*> in7f = in7;
    in7f[2] = "bias: float";
    v.push_back({"_ITEXQuantizedMatMulWithBiasAndRelu", in7f, out3, attrs(nullptr, "Toutput: quantizedtype = DT_QINT32")});
    v.push_back({"_ITEXQuantizedMatMulWithBiasAndRequantize", in9, out3,
                 attrs("Tbias: {float, qint32}", "Toutput: quantizedtype = DT_QUINT8")});
    v.push_back({"_ITEXQuantizedMatMulWithBiasAndReluAndRequantize", in9, out3,
                 attrs("Tbias: {float, qint32}", "Toutput: quantizedtype = DT_QUINT8")});
    v.push_back({"_ITEXQuantizedMatMulWithBiasAndDequantize", in9, {"out: Toutput"},
                 attrs("Tbias: {float, bfloat16, qint32}", "Toutput: {float, bfloat16}")});
  }
  // quantized Conv2D and depthwise Conv2D: the list-attribute form (nn_ops.cc:585-700, 752-860) and the _ITEX twins of
  // TensorFlow's QuantizedConv2D* / QuantizedDepthwiseConv2D* ops
  for (const char* name : {"_QuantizedConv2D", "_ITEXQuantizedConv2DV2", "_QuantizedDepthwiseConv2D", "_ITEXQuantizedDepthwiseConv2DV2"})
    v.push_back({name,
                 {"device_inputs: Tdevice_inputs", "host_inputs: Thost_inputs"},
                 {"device_outputs: Tdevice_outputs", "host_outputs: Thost_outputs"},
                 {"Tinput: quantizedtype = DT_QUINT8", "Tfilter: quantizedtype = DT_QINT8", "Tbias: {float, qint32} = DT_QINT32",
                  "Tsummand: {float, quint8, qint8, qint32, bfloat16}", "out_type: {qint8, quint8, qint32, float, bfloat16}",
                  "Tdevice_inputs: list(type) >= 0 = []", "Thost_inputs: list(type) >= 0", "Tdevice_outputs: list(type) >= 0 = []",
                  "Thost_outputs: list(type) >= 0", "data_format: string = 'NHWC'", "strides: list(int)",
                  "is_filter_const: bool = true", "is_bias_const: bool = true", "padding: {'SAME', 'VALID', 'EXPLICIT'}",
                  "explicit_paddings: list(int) = []", "dilations: list(int) = [1, 1, 1, 1]", "fused_ops: list(string) = []",
                  "alpha: float = 0.0"}});
  {
    const std::vector<const char*> base_attrs = {"Tinput: quantizedtype", "Tfilter: quantizedtype", "strides: list(int)",
                                                 "padding: {'SAME', 'VALID'}", "dilations: list(int) = [1, 1, 1, 1]",
                                                 "padding_list: list(int) = []", "is_filter_const: bool = true"};
    struct Twin { const char* name; bool bias, req; const char* out_default; bool sum = false; };
    for (const Twin& t : {Twin{"_ITEXQuantizedConv2D", false, false, "out_type: quantizedtype = DT_QINT32"},
                          Twin{"_ITEXQuantizedConv2DPerChannel", false, false, "out_type: quantizedtype = DT_QINT32"},
                          Twin{"_ITEXQuantizedConv2DWithBias", true, false, "out_type: quantizedtype = DT_QINT32"},
                          Twin{"_ITEXQuantizedConv2DWithBiasAndRelu", true, false, "out_type: quantizedtype = DT_QINT32"},
                          Twin{"_ITEXQuantizedConv2DAndRelu", false, false, "out_type: quantizedtype = DT_QINT32"},
                          Twin{"_ITEXQuantizedConv2DAndRequantize", false, true, "out_type: quantizedtype = DT_QINT8"},
                          Twin{"_ITEXQuantizedConv2DAndReluAndRequantize", false, true, "out_type: quantizedtype = DT_QUINT8"},
                          Twin{"_ITEXQuantizedConv2DWithBiasAndRequantize", true, true, "out_type: quantizedtype = DT_QINT8"},
                          Twin{"_ITEXQuantizedConv2DWithBiasAndReluAndRequantize", true, true, "out_type: quantizedtype = DT_QUINT8"},
                          Twin{"_ITEXQuantizedDepthwiseConv2D", false, false, "out_type: quantizedtype = DT_QINT32"},
                          Twin{"_ITEXQuantizedDepthwiseConv2DWithBias", true, false, "out_type: quantizedtype = DT_QINT32"},
                          Twin{"_ITEXQuantizedDepthwiseConv2DWithBiasAndRelu", true, false, "out_type: quantizedtype = DT_QINT32"},
                          Twin{"_ITEXQuantizedDepthwiseConv2DWithBiasAndReluAndRequantize", true, true,
                               "out_type: quantizedtype = DT_QUINT8"},
                          Twin{"_ITEXQuantizedConv2DWithBiasSumAndReluAndRequantize", true, true, "out_type: quantizedtype = DT_QUINT8", true},
                          Twin{"_ITEXQuantizedConv2DWithBiasSignedSumAndReluAndRequantize", true, true,
                               "out_type: quantizedtype = DT_QUINT8", true}}) {
      OpSpec s{t.name, {"input: Tinput", "filter: Tfilter"}, {"output: out_type", "min_output: float", "max_output: float"}, base_attrs};
      if (t.bias) s.inputs.push_back(t.req ? "bias: Tbias" : "bias: float");
      for (const char* in : {"min_input: float", "max_input: float", "min_filter: float", "max_filter: float"}) s.inputs.push_back(in);
      if (t.req) {
        s.inputs.push_back("min_freezed_output: float");
        s.inputs.push_back("max_freezed_output: float");
        if (t.bias) s.attrs.push_back("Tbias: {float, qint32}");
      }
      if (t.sum) {  // nn_ops.cc of TensorFlow: ..., summand, min_summand, max_summand
        for (const char* in : {"summand: Tsummand", "min_summand: float", "max_summand: float"}) s.inputs.push_back(in);
        s.attrs.push_back("Tsummand: quantizedtype");
      }
      s.attrs.push_back(t.out_default);
      v.push_back(s);
    }
  }
  // nn_ops.cc:562-585 (_QuantizedTranspose), :3266-3290 (_ITEXQuantizedReshape)
  for (const char* name : {"_QuantizedTranspose", "_ITEXQuantizedTranspose"})
    v.push_back({name,
                 {"x: T", "perm: Tperm", "min_x: float", "max_x: float"},
                 {"y: T", "min_y: float", "max_y: float"},
                 {"T: quantizedtype", "Tperm: {int32, int64} = DT_INT32"}});
  v.push_back({"_ITEXQuantizedReshape",
               {"tensor: T", "shape: Tshape", "input_min: float", "input_max: float"},
               {"output: T", "output_min: float", "output_max: float"},
               {"T: type", "Tshape: {int32, int64} = DT_INT32"}});
  // nn_ops.cc:4636-4691
  for (const char* name : {"_QuantizedBatchMatMul", "_ITEXQuantizedBatchMatMul"})
    v.push_back({name,
                 {"device_inputs: Tdevice_inputs", "host_inputs: Thost_inputs"},
                 {"device_outputs: Tdevice_outputs", "host_outputs: Thost_outputs"},
                 {"Tdevice_inputs: list(type) >= 0 = []", "Thost_inputs: list(type) >= 0 = []",
                  "Tdevice_outputs: list(type) >= 0 = []", "Thost_outputs: list(type) >= 0 = []",
                  "T1: quantizedtype", "T2: quantizedtype", "U: {bfloat16, float, quantizedtype} = DT_FLOAT",
                  "Tout: {bfloat16, float, quantizedtype} = DT_FLOAT", "adj_x: bool = false", "adj_y: bool = false",
                  "fused_ops: list(string) = []", "input_quant_mode: {'MIN_FIRST', 'SCALED'} = 'SCALED'",
                  "output_quant_mode: {'MIN_FIRST', 'SCALED'} = 'SCALED'"}});
  return v;
}

}  // namespace

void RegisterOps() {
  static std::vector<OpSpec> specs = OpSpecs();
  const std::set<std::string> known = KnownOps();
  for (const OpSpec& s : specs) {
    if (known.count(s.name)) continue;  // TensorFlow (or another plugin) already defines it
    TF_OpDefinitionBuilder* b = TF_NewOpDefinitionBuilder(s.name);
    for (const char* i : s.inputs) TF_OpDefinitionBuilderAddInput(b, i);
    for (const char* o : s.outputs) TF_OpDefinitionBuilderAddOutput(b, o);
    for (const char* a : s.attrs) TF_OpDefinitionBuilderAddAttr(b, a);
    TF_OpDefinitionBuilderSetShapeInferenceFunction(b, &UnknownShape);
    TF_Status* st = TF_NewStatus();
    TF_RegisterOpDefinition(b, st);
    if (TF_GetCode(st) != TF_OK) std::fprintf(stderr, "itex_amd: %s op registration failed: %s\n", s.name, TF_Message(st));
    TF_DeleteStatus(st);
  }
}

}  // namespace itex_amd

extern "C" void TF_InitKernel(void) {
  static std::once_flag once;
  std::call_once(once, [] {
    using namespace itex_amd;
    RegisterOps();
    AddQuantizeKernels();
    AddDequantizeKernels();
    AddQuantizedMatMulKernels();
    AddQuantizedBatchMatMulKernels();
    AddQuantizedShapeKernels();
    AddQuantizedConvKernels();
    AddRequantizeKernels();
    // the device type the kernels attach to: ITEX's own PluggableDevice type by default, so that graphs
    // placed by ITEX's passes keep their device strings
    const char* dev = std::getenv("ITEX_AMD_DEVICE_TYPE");
    RegisterKernels(dev && dev[0] ? dev : "XPU");
  });
}
