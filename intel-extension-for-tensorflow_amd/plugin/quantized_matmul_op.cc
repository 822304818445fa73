// Quantized MatMul op kernels: _QuantizedMatMul / _ITEXQuantizedMatMul (V2),
// _QuantizedFusedMatMul{,AndRequantize,AndDequantize} (V1) and the legacy
// QuantizedMatMulWithBias{,AndRelu,AndRequantize,AndReluAndRequantize,AndDequantize}.
//
// Mirrors LegacyQuantizedMatMulOpBase and its three subclasses
// (itex/core/kernels/common/quantized_matmul_common.h:48-736, 1412-1909): attribute parsing, input
// index conventions, one Compute at a time per node, cached weight preparation, host-memory min/max
// outputs.  Where the reference builds a oneDNN inner-product primitive, reorders the weight and
// prepares scales / bias on the host, this kernel prepacks the weight once on the device
// (itexhip_qgemm_prepack_b, which also yields the column sums the MIN_FIRST compensation needs),
// lets a small device kernel derive the per-channel scale and bias vectors from the current ranges
// (itexhip_qmatmul_prepare: no host wait when the activation range changes) and launches
// itexhip_qgemm.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "device_vector_cache.h"
#include "itexhip.h"
#include "op_kernel.h"
#include "qparams.h"

namespace itex_amd {
namespace {

enum class Api { V2 = ITEXHIP_API_V2, V1 = ITEXHIP_API_V1, LEGACY = ITEXHIP_API_LEGACY };

struct Variant {
  Api api;
  TF_DataType t_in, t_out;
  bool legacy_relu;  // QuantizedMatMulReluOp
  // _ITEXQuantizedMatMulDynamicInput (made by this plugin's graph pass; no counterpart in the reference): input 0 is
  // the float tensor, quantized here against its own range, and the min_a / max_a inputs are gone
  bool dynamic_input = false;
};

int ActivationFromName(const std::string& n) {
  if (n == "Relu") return ITEXHIP_ACT_RELU;
  if (n == "Relu6") return ITEXHIP_ACT_RELU6;
  if (n == "LeakyRelu") return ITEXHIP_ACT_LEAKYRELU;
  if (n == "GeluApproximate") return ITEXHIP_ACT_GELU_APPROX;
  if (n == "GeluExact") return ITEXHIP_ACT_GELU_EXACT;
  if (n == "Elu") return ITEXHIP_ACT_ELU;
  if (n == "Sigmoid") return ITEXHIP_ACT_SIGMOID;
  if (n == "Tanh") return ITEXHIP_ACT_TANH;
  if (n == "_ITEXSwish") return ITEXHIP_ACT_SWISH;
  if (n == "_ITEXMish") return ITEXHIP_ACT_MISH;
  return -1;
}

class QuantizedMatMulOp : public OpKernel {
 public:
  QuantizedMatMulOp(OpKernelConstruction* ctx, const Variant& v) : v_(v) {
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("transpose_a", &transpose_a_));
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("transpose_b", &transpose_b_));
    std::string mode_string;
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("input_quant_mode", &mode_string));
    ITEX_REQUIRES(ctx, mode_string == "MIN_FIRST" || mode_string == "SCALED", TF_INVALID_ARGUMENT,
                  "Quantization mode must be either MIN_FIRST or SCALED, but received " + mode_string);
    p_.input_mode = mode_string == "MIN_FIRST" ? ITEXHIP_MIN_FIRST : ITEXHIP_SCALED;
    p_.api = static_cast<int>(v.api);
    p_.t_in = v.t_in;
    p_.t_out = v.t_out;
    p_.leakyrelu_alpha = 0.2f;

    std::vector<std::string> fused_ops;
    if (v.api == Api::LEGACY) {  // :1418-1465, :1516-1523
      if (ctx->HasAttr("is_weight_const")) ITEX_REQUIRES_OK(ctx, ctx->GetAttr("is_weight_const", &is_weight_const_));
      is_bias_const_ = true;
      if (v.legacy_relu) p_.activation = ITEXHIP_ACT_RELU;
      min_a_idx_ = 3;
      min_out_idx_ = 7;
    } else if (v.api == Api::V1) {  // :1545-1603
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("is_filter_const", &is_weight_const_));
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("is_bias_const", &is_bias_const_));
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("fused_ops", &fused_ops));
      ITEX_REQUIRES(ctx, fused_ops.size() <= 2, TF_INVALID_ARGUMENT, "_QuantizedFusedMatMul supports maximum 2 post ops");
      ITEX_REQUIRES(ctx, fused_ops.empty() || fused_ops[0] == "BiasAdd", TF_INVALID_ARGUMENT,
                    "_QuantizedFusedMatMul first post op must be BiasAdd");
      p_.n_fused_ops = static_cast<int>(fused_ops.size());
      for (size_t i = 1; i < fused_ops.size(); ++i) {
        if (fused_ops[i] == "Add") {  // the addend follows the bias in `args` and shifts every min/max input (:1593-1602)
          p_.add_position = p_.activation == ITEXHIP_ACT_NONE ? 1 : 2;
          continue;
        }
        const int act = ActivationFromName(fused_ops[i]);
        ITEX_REQUIRES(ctx, act >= 0, TF_INVALID_ARGUMENT, "Found unsupported fusion in _QuantizedFusedMatMul.");
        p_.activation = act;
      }
      min_a_idx_ = 3 + (p_.add_position != 0);
      min_out_idx_ = 7 + (p_.add_position != 0);
    } else {  // V2 :1725-1795
      std::string out_mode;
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("output_quant_mode", &out_mode));
      p_.out_min_first = out_mode == "MIN_FIRST";
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("is_weight_const", &is_weight_const_));
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("is_bias_const", &is_bias_const_));
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("fused_ops", &fused_ops));
      for (const std::string& f : fused_ops) {
        if (f == "BiasAdd" || f == "Quantized") continue;
        if (f == "Requantize") { p_.has_requantize = 1; continue; }
        if (f == "Dequantize") { p_.has_dequantize = 1; continue; }
        if (f == "Add") {
          ITEX_REQUIRES(ctx, v.t_out == TF_FLOAT || v.t_out == TF_BFLOAT16 || v.t_out == TF_HALF, TF_UNIMPLEMENTED,
                        "Quantized addend tensor is not implemented yet.");
          p_.add_position = p_.activation == ITEXHIP_ACT_NONE ? 1 : 2;
          continue;
        }
        const int act = ActivationFromName(f);
        ITEX_REQUIRES(ctx, act >= 0, TF_INVALID_ARGUMENT, "Found unsupported fusion in _QuantizedMatMul.");
        p_.activation = act;
      }
      p_.n_fused_ops = static_cast<int>(fused_ops.size());
      min_a_idx_ = 3 + (p_.add_position != 0);  // the addend precedes all min/max tensors (:1775-1780)
      min_out_idx_ = 7;  // fixed, as in the reference (:1784-1785)
      if (v.dynamic_input) {
        ITEX_REQUIRES(ctx, p_.add_position == 0 && (p_.has_requantize || p_.has_dequantize), TF_INVALID_ARGUMENT,
                      "_ITEXQuantizedMatMulDynamicInput takes no addend and needs Requantize or Dequantize in fused_ops");
        ITEX_REQUIRES(ctx, p_.input_mode == ITEXHIP_SCALED || v.t_in == TF_QUINT8, TF_INVALID_ARGUMENT,
                      "MIN_FIRST input quantization gives quint8");
        if (ctx->HasAttr("ensure_minimum_range")) ITEX_REQUIRES_OK(ctx, ctx->GetAttr("ensure_minimum_range", &ensure_minimum_range_));
        min_out_idx_ = 5;
      }
    }
    if (p_.activation == ITEXHIP_ACT_LEAKYRELU) ITEX_REQUIRES_OK(ctx, ctx->GetAttr("leakyrelu_alpha", &p_.leakyrelu_alpha));
    // the bias type attribute is "Targs" for the V1 ops (:1533-1537), "Tbias" elsewhere
    const char* bias_attr = v.api == Api::V1 ? "Targs" : "Tbias";
    if (ctx->HasAttr(bias_attr)) {
      TF_DataType tb = TF_FLOAT;
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr(bias_attr, &tb));
      ITEX_REQUIRES(ctx, tb == TF_FLOAT || tb == TF_QINT32 || tb == TF_BFLOAT16 || tb == TF_HALF || tb == TF_QINT8 || tb == TF_QUINT8,
                    TF_UNIMPLEMENTED, "the bias type must be float, bfloat16, half, qint32, qint8 or quint8");
      // 8-bit biases are registered, as the reference registers them for a device (kernels/gpu/quantized_matmul.cc:
      // 123-133), so that a graph naming them is placed; Compute refuses them (see there)
      eight_bit_bias_ = tb == TF_QINT8 || tb == TF_QUINT8;
      p_.t_bias = eight_bit_bias_ ? 0 : tb;
    }
    if (p_.add_position != 0) {
      ITEX_REQUIRES(ctx, v.t_out == TF_FLOAT || v.t_out == TF_BFLOAT16 || v.t_out == TF_HALF, TF_UNIMPLEMENTED,
                    "Quantized addend tensor is not implemented yet.");
      // the V1 ops pass bias and addend in one `args` list of type Targs, and the addend has the output's type
      // (:341-389): Targs must be that type
      const TF_DataType targs = p_.t_bias == 0 ? TF_FLOAT : static_cast<TF_DataType>(p_.t_bias);
      ITEX_REQUIRES(ctx, v.api != Api::V1 || targs == v.t_out, TF_INVALID_ARGUMENT,
                    "the Add fusion of _QuantizedFusedMatMul needs args of the output's type");
    }
  }

  void Compute(OpKernelContext* ctx) override {
    std::lock_guard<std::mutex> lock(mu_);  // one Compute at a time per node (:62)
    Tensor a = ctx->input(0);
    Tensor w = ctx->input(1);
    Tensor bias = ctx->input(2);
    const bool dyn = v_.dynamic_input;
    const int min_b_idx = dyn ? min_a_idx_ : min_a_idx_ + 2;
    Tensor min_a_t, max_a_t;
    if (!dyn) {
      min_a_t = ctx->input(min_a_idx_);
      max_a_t = ctx->input(min_a_idx_ + 1);
    }
    Tensor min_b_t = ctx->input(min_b_idx), max_b_t = ctx->input(min_b_idx + 1);
    if (!ctx->ok()) return;
    // The reference's generic GetScaledBias stores the adjusted bias back in Tbias with a C conversion from float
    // (quantized_matmul_common.h:578-599: truncation, undefined outside the 8-bit range) or a saturating oneDNN reorder
    // (:602-634) depending on the input mode; nothing in its tests runs an 8-bit bias, so there is no defined result to
    // reproduce.
    ITEX_REQUIRES(ctx, !eight_bit_bias_, TF_UNIMPLEMENTED,
                  "quantized MatMul with Tbias / Targs = qint8 or quint8 is registered but not computed on this device: the "
                  "reference narrows the adjusted fp32 bias back to 8 bits, which is undefined for most values");
    ITEX_REQUIRES(ctx, a.dims() == 2 && w.dims() == 2, TF_INVALID_ARGUMENT, "quantized MatMul operands must be matrices");
    const TF_DataType bias_type = p_.t_bias == 0 ? TF_FLOAT : static_cast<TF_DataType>(p_.t_bias);
    ITEX_REQUIRES(ctx, a.dtype() == (dyn ? TF_FLOAT : v_.t_in) && w.dtype() == TF_QINT8 && bias.dtype() == bias_type, TF_INVALID_ARGUMENT,
                  "quantized MatMul operand types do not match the kernel");
    // transpose_a: the reference swaps the two dimensions but still describes the buffer as a row-major [batch, k]
    // matrix (:183-198, format_tag::nc), so nothing is transposed - the [k, batch] tensor is read as [batch, k].
    // Reproduced as written.
    const int64_t M = a.dim_size(transpose_a_ ? 1 : 0), K = a.dim_size(transpose_a_ ? 0 : 1);
    const int64_t N = transpose_b_ ? w.dim_size(0) : w.dim_size(1);
    ITEX_REQUIRES(ctx, (transpose_b_ ? w.dim_size(1) : w.dim_size(0)) == K, TF_INVALID_ARGUMENT,
                  "Matrix size-incompatible: In[0] inner dimension " + std::to_string(K) + " vs In[1]");
    ITEX_REQUIRES(ctx, bias.NumElements() == N, TF_INVALID_ARGUMENT, "bias must have one entry per output channel");
    // the reference's zero-point compensation indexes the weight as [K, N] whatever transpose_b says
    // (:569-573); that combination is refused instead of reproduced
    ITEX_REQUIRES(ctx, !(transpose_b_ && p_.input_mode == ITEXHIP_MIN_FIRST), TF_UNIMPLEMENTED,
                  "transpose_b with MIN_FIRST input quantization is not supported");
    const int64_t nb = min_b_t.NumElements();
    ITEX_REQUIRES(ctx, max_b_t.NumElements() == nb && (nb == 1 || nb == N), TF_INVALID_ARGUMENT,
                  "min_b / max_b must be scalars or hold one entry per output channel");
    ITEX_REQUIRES(ctx, v_.api != Api::LEGACY || nb == 1, TF_INVALID_ARGUMENT,
                  "QuantizedMatMulWithBias takes per-tensor weight ranges");

    itexhip_matmul_params p = p_;
    if (!dyn) {
      p.min_a = min_a_t.flat<float>()[0];
      p.max_a = max_a_t.flat<float>()[0];
    }
    const bool out_q8 = v_.t_out == TF_QINT8 || v_.t_out == TF_QUINT8;
    const bool needs_freezed =
        out_q8 || (v_.api == Api::LEGACY && (v_.t_out == TF_FLOAT || v_.t_out == TF_BFLOAT16 || v_.t_out == TF_HALF));
    if (needs_freezed) {
      ITEX_REQUIRES(ctx, ctx->num_inputs() > min_out_idx_ + 1, TF_INVALID_ARGUMENT,
                    "min_freezed_output / max_freezed_output inputs are missing");
      Tensor mo = ctx->input(min_out_idx_), xo = ctx->input(min_out_idx_ + 1);
      if (!ctx->ok()) return;
      p.min_out = mo.flat<float>()[0];
      p.max_out = xo.flat<float>()[0];
    }
    itexhip_epilogue ep;
    int st = itexhip_qmatmul_epilogue_desc(&p, nb, &ep);
    ITEX_REQUIRES(ctx, st == ITEXHIP_OK, static_cast<TF_Code>(st), itexhip_last_error());

    void* stream = ctx->stream();
    // ---- weight: prepacked once when constant, else every call (:238-275)
    const bool packed_path = K % 16 == 0 && K > 0;
    const bool repack = !packed_.valid() || !is_weight_const_ || packed_src_ != w.data() || packed_k_ != K || packed_n_ != N;
    if (packed_path && repack) {
      const int64_t bytes = itexhip_qgemm_packed_bytes(K, N);
      packed_ = ctx->allocate_temp(TF_QINT8, {std::max<int64_t>(bytes, 16)});
      colsum_ = ctx->allocate_temp(TF_INT32, {std::max<int64_t>(N, 1)});
      if (!ctx->ok()) return;
      st = itexhip_qgemm_prepack_b(w.flat<int8_t>(), transpose_b_ ? 1 : 0, K, N, packed_.flat<int8_t>(),
                                   colsum_.flat<int32_t>(), stream);
      ITEX_REQUIRES(ctx, st == ITEXHIP_OK, TF_ABORTED, std::string("Operation received an exception: ") + itexhip_last_error());
      packed_src_ = w.data();
      packed_k_ = K;
      packed_n_ = N;
    }
    // ---- the weight ranges on the device (uploaded when they change)
    float* min_b_dev = min_b_cache_.Get(ctx, min_b_t.flat<float>(), nb, TF_FLOAT);
    float* max_b_dev = max_b_cache_.Get(ctx, max_b_t.flat<float>(), nb, TF_FLOAT);
    if (min_b_dev == nullptr || max_b_dev == nullptr) return;
    // ---- product: one launch, the MatMul kernel derives each channel's output scale and compensated
    // bias itself, so a new activation range costs nothing extra.  K a multiple of 16: MFMA kernels on
    // the prepacked weight; other K: the reference-shaped kernel on the unpacked weight.
    // "Add": the addend (of the output's type: float, bfloat16 or half) is input 3 (:352-389 adds it in place into the forwarded output buffer; here the
    // kernel reads it and writes a fresh output, same values)
    const void* addend = nullptr;
    Tensor addend_t;
    if (p_.add_position != 0) {
      addend_t = ctx->input(3);
      if (!ctx->ok()) return;
      ITEX_REQUIRES(ctx, addend_t.dtype() == v_.t_out && addend_t.dims() == 2 && addend_t.dim_size(0) == M &&
                             addend_t.dim_size(1) == N,
                    TF_INVALID_ARGUMENT, "the addend must be a tensor of the output's type and shape");
      addend = addend_t.data();
    }
    Tensor out = ctx->allocate_output(0, v_.t_out, {M, N});
    if (!ctx->ok()) return;
    if (dyn && M * K > 0) {
      // range reduction, parameter math and quantization of the float tensor, then the product reading the range
      // from device memory: nothing waits on the host.  K not a multiple of 16 (no MFMA kernel): the range is
      // fetched once for the reference-shaped kernel.
      Tensor aq = ctx->allocate_temp(v_.t_in, {M, K});
      Tensor state = ctx->allocate_temp(TF_FLOAT, {ITEXHIP_DYNAMIC_STATE_FLOATS});
      if (!ctx->ok()) return;
      st = itexhip_quantize_dynamic(a.flat<float>(), aq.data(), M * K, v_.t_in, p_.input_mode, ensure_minimum_range_,
                                    state.flat<float>(), stream);
      if (st == ITEXHIP_OK && packed_path) {
        st = itexhip_qmatmul_device_range(&p, aq.data(), packed_.flat<int8_t>(), colsum_.flat<int32_t>(), M, K, N,
                                          state.flat<float>() + 2, min_b_dev, max_b_dev, nb, bias.data(), nullptr,
                                          out.data(), stream);
      } else if (st == ITEXHIP_OK) {
        float range[2] = {0.0f, 0.0f};
        st = itexhip_memcpy_d2h(range, state.flat<float>() + 2, sizeof(range), stream);
        p.min_a = range[0];
        p.max_a = range[1];
        if (st == ITEXHIP_OK)
          st = itexhip_qmatmul_unpacked(&p, aq.data(), w.flat<int8_t>(), transpose_b_ ? 1 : 0, M, K, N, min_b_dev, max_b_dev,
                                        nb, bias.data(), nullptr, out.data(), stream);
      }
    } else if (dyn) {  // no elements to take a range from: the bias (K == 0) or nothing (M == 0)
      float mn = 0.0f, mx = 0.0f;  // what _ITEXQuantizeV2DynamicRange reports for an empty tensor
      qparams::AdjustRange(0.0f, 0.0f, ensure_minimum_range_, &mn, &mx);
      if (p_.input_mode == ITEXHIP_SCALED) {
        const float r = std::max(std::fabs(mn), std::fabs(mx));
        mx = r;
        mn = v_.t_in == TF_QUINT8 ? 0.0f : -r;
      }
      p.min_a = mn;
      p.max_a = mx;
      st = itexhip_qmatmul_unpacked(&p, a.data(), w.flat<int8_t>(), transpose_b_ ? 1 : 0, M, K, N, min_b_dev, max_b_dev, nb,
                                    bias.data(), nullptr, out.data(), stream);
    } else if (packed_path) {
      st = itexhip_qmatmul(&p, a.data(), packed_.flat<int8_t>(), colsum_.flat<int32_t>(), M, K, N, min_b_dev, max_b_dev,
                           nb, bias.data(), addend, out.data(), stream);
    } else {
      st = itexhip_qmatmul_unpacked(&p, a.data(), w.flat<int8_t>(), transpose_b_ ? 1 : 0, M, K, N, min_b_dev, max_b_dev, nb,
                                    bias.data(), addend, out.data(), stream);
    }
    ITEX_REQUIRES(ctx, st == ITEXHIP_OK, st == ITEXHIP_INVALID_ARGUMENT ? TF_INVALID_ARGUMENT : TF_ABORTED,
                  std::string("Operation received an exception: ") + itexhip_last_error());

    // ---- output ranges in host memory (AllocateNativeOutputMinMax,
    // itex/core/kernels/onednn/block/quantized_ops.h:142-203)
    if (out_q8) {
      Tensor omin = ctx->allocate_output(1, TF_FLOAT, {});
      Tensor omax = ctx->allocate_output(2, TF_FLOAT, {});
      if (!ctx->ok()) return;
      omin.flat<float>()[0] = p.min_out;
      omax.flat<float>()[0] = p.max_out;
    } else if (v_.t_out == TF_QINT32) {
      const bool scalar = min_b_t.dims() == 0;
      const std::vector<int64_t> shp = scalar ? std::vector<int64_t>{} : std::vector<int64_t>{nb};
      Tensor omin = ctx->allocate_output(1, TF_FLOAT, shp);
      Tensor omax = ctx->allocate_output(2, TF_FLOAT, shp);
      if (!ctx->ok()) return;
      for (int64_t i = 0; i < (scalar ? 1 : nb); ++i)
        qparams::RangeForMultiplication(v_.t_in, TF_QINT8, p.min_a, p.max_a, min_b_t.flat<float>()[i],
                                        max_b_t.flat<float>()[i], &omin.flat<float>()[i], &omax.flat<float>()[i]);
    }
  }

 private:
  Variant v_;
  itexhip_matmul_params p_{};
  bool transpose_a_ = false, transpose_b_ = false;
  bool is_weight_const_ = true, is_bias_const_ = true;
  int min_a_idx_ = 3, min_out_idx_ = 7;
  float ensure_minimum_range_ = 0.01f;
  std::mutex mu_;
  bool eight_bit_bias_ = false;
  // persistent device state of the node
  Tensor packed_, colsum_;
  const void* packed_src_ = nullptr;
  int64_t packed_k_ = -1, packed_n_ = -1;
  DeviceVectorCache<float> min_b_cache_, max_b_cache_;
};

template <int API, int TIN, int TOUT, bool RELU>
struct MatMulKernel : QuantizedMatMulOp {
  explicit MatMulKernel(OpKernelConstruction* c)
      : QuantizedMatMulOp(c, Variant{static_cast<Api>(API), static_cast<TF_DataType>(TIN), static_cast<TF_DataType>(TOUT), RELU}) {}
};

template <int TIN, int TOUT>
struct DynamicInputMatMulKernel : QuantizedMatMulOp {
  explicit DynamicInputMatMulKernel(OpKernelConstruction* c)
      : QuantizedMatMulOp(c, Variant{Api::V2, static_cast<TF_DataType>(TIN), static_cast<TF_DataType>(TOUT), false, true}) {}
};

template <int TIN, int TOUT>
void RegDynamicInput() {
  for (TF_DataType tb : {TF_FLOAT, TF_QINT32, TF_BFLOAT16, TF_HALF}) {
    KernelDefBuilder b("_ITEXQuantizedMatMulDynamicInput", "QuantizedMatMulOp");
    b.TypeConstraint("T1", static_cast<TF_DataType>(TIN)).TypeConstraint("T2", TF_QINT8);
    b.TypeConstraint("Tbias", tb).TypeConstraint("Tout", static_cast<TF_DataType>(TOUT));
    b.HostMemory("host_inputs").HostMemory("host_outputs");
    b.Register<DynamicInputMatMulKernel<TIN, TOUT>>();
  }
}

template <int API, int TIN, int TOUT, bool RELU>
void Reg(const char* op, const char* out_attr, const char* bias_attr, std::initializer_list<const char*> host_args) {
  KernelDefBuilder b(op, "QuantizedMatMulOp");
  b.TypeConstraint("T1", static_cast<TF_DataType>(TIN)).TypeConstraint("T2", TF_QINT8);
  if (bias_attr) b.TypeConstraint(bias_attr, TF_FLOAT);
  b.TypeConstraint(out_attr, static_cast<TF_DataType>(TOUT));
  for (const char* h : host_args) b.HostMemory(h);
  b.Register<MatMulKernel<API, TIN, TOUT, RELU>>();
  if (bias_attr) {  // the same kernel with a qint32 bias and, for the V1 / V2 ops, a bfloat16 / half bias
    for (TF_DataType tb : {TF_QINT32, TF_BFLOAT16, TF_HALF, TF_QINT8, TF_QUINT8}) {
      if (tb != TF_QINT32 && API == ITEXHIP_API_LEGACY) continue;
      KernelDefBuilder q(op, "QuantizedMatMulOp");
      q.TypeConstraint("T1", static_cast<TF_DataType>(TIN)).TypeConstraint("T2", TF_QINT8);
      q.TypeConstraint(bias_attr, tb).TypeConstraint(out_attr, static_cast<TF_DataType>(TOUT));
      for (const char* h : host_args) q.HostMemory(h);
      q.Register<MatMulKernel<API, TIN, TOUT, RELU>>();
    }
  }
}

template <int API, int TOUT>
void RegBothInputs(const char* op, const char* out_attr, const char* bias_attr, std::initializer_list<const char*> host_args) {
  Reg<API, TF_QUINT8, TOUT, false>(op, out_attr, bias_attr, host_args);
  Reg<API, TF_QINT8, TOUT, false>(op, out_attr, bias_attr, host_args);
}

}  // namespace

// Names, type constraints and host-memory arguments as registered by the reference for a device
// (itex/core/kernels/gpu/quantized_matmul.cc:35-201); the _ITEX names are the CPU-side renames
// (itex/core/kernels/cpu/quantized_matmul.cc:97-163), registered as well.
void AddQuantizedMatMulKernels() {
  constexpr int V2 = ITEXHIP_API_V2, V1 = ITEXHIP_API_V1, LG = ITEXHIP_API_LEGACY;
  // legacy ops: quint8 x qint8
  for (const char* op : {"QuantizedMatMulWithBiasAndRelu", "_ITEXQuantizedMatMulWithBiasAndRelu"})
    Reg<LG, TF_QUINT8, TF_QINT32, true>(op, "Toutput", nullptr, {"min_a", "max_a", "min_b", "max_b", "min_out", "max_out"});
  for (const char* op : {"QuantizedMatMulWithBias", "_ITEXQuantizedMatMulWithBias"})
    Reg<LG, TF_QUINT8, TF_QINT32, false>(op, "Toutput", "Tbias", {"min_a", "max_a", "min_b", "max_b", "min_out", "max_out"});
  for (const char* op : {"QuantizedMatMulWithBiasAndReluAndRequantize", "_ITEXQuantizedMatMulWithBiasAndReluAndRequantize"})
    Reg<LG, TF_QUINT8, TF_QUINT8, true>(op, "Toutput", "Tbias",
                                        {"min_a", "max_a", "min_b", "max_b", "min_freezed_output", "max_freezed_output",
                                         "min_out", "max_out"});
  for (const char* op : {"QuantizedMatMulWithBiasAndRequantize", "_ITEXQuantizedMatMulWithBiasAndRequantize"})
    Reg<LG, TF_QUINT8, TF_QUINT8, false>(op, "Toutput", "Tbias",
                                         {"min_a", "max_a", "min_b", "max_b", "min_freezed_output", "max_freezed_output",
                                          "min_out", "max_out"});
  for (const char* op : {"QuantizedMatMulWithBiasAndDequantize", "_ITEXQuantizedMatMulWithBiasAndDequantize"})
    Reg<LG, TF_QUINT8, TF_FLOAT, false>(op, "Toutput", "Tbias",
                                        {"min_a", "max_a", "min_b", "max_b", "min_freezed_output", "max_freezed_output"});
  for (const char* op : {"QuantizedMatMulWithBiasAndDequantize", "_ITEXQuantizedMatMulWithBiasAndDequantize"}) {
    Reg<LG, TF_QUINT8, TF_BFLOAT16, false>(op, "Toutput", "Tbias",
                                           {"min_a", "max_a", "min_b", "max_b", "min_freezed_output", "max_freezed_output"});
    Reg<LG, TF_QUINT8, TF_HALF, false>(op, "Toutput", "Tbias",
                                       {"min_a", "max_a", "min_b", "max_b", "min_freezed_output", "max_freezed_output"});
  }
  // V1
  for (const char* op : {"_QuantizedFusedMatMul", "_ITEXQuantizedFusedMatMul"})
    RegBothInputs<V1, TF_QINT32>(op, "Toutput", "Targs", {"min_a", "max_a", "min_b", "max_b", "min_product", "max_product"});
  for (const char* op : {"_QuantizedFusedMatMulAndDequantize", "_ITEXQuantizedFusedMatMulAndDequantize"})
    RegBothInputs<V1, TF_FLOAT>(op, "Toutput", "Targs", {"min_a", "max_a", "min_b", "max_b"});
  for (const char* op : {"_QuantizedFusedMatMulAndDequantize", "_ITEXQuantizedFusedMatMulAndDequantize"}) {
    RegBothInputs<V1, TF_BFLOAT16>(op, "Toutput", "Targs", {"min_a", "max_a", "min_b", "max_b"});
    RegBothInputs<V1, TF_HALF>(op, "Toutput", "Targs", {"min_a", "max_a", "min_b", "max_b"});
  }
  for (const char* op : {"_QuantizedFusedMatMulAndRequantize", "_ITEXQuantizedFusedMatMulAndRequantize"}) {
    RegBothInputs<V1, TF_QUINT8>(op, "Toutput", "Targs", {"min_a", "max_a", "min_b", "max_b", "min_freezed_output",
                                                          "max_freezed_output", "min_product", "max_product"});
    RegBothInputs<V1, TF_QINT8>(op, "Toutput", "Targs", {"min_a", "max_a", "min_b", "max_b", "min_freezed_output",
                                                         "max_freezed_output", "min_product", "max_product"});
  }
  // V2
  for (const char* op : {"_QuantizedMatMul", "_ITEXQuantizedMatMul"}) {
    RegBothInputs<V2, TF_QINT32>(op, "Tout", "Tbias", {"host_inputs", "host_outputs"});
    RegBothInputs<V2, TF_FLOAT>(op, "Tout", "Tbias", {"host_inputs", "host_outputs"});
    RegBothInputs<V2, TF_BFLOAT16>(op, "Tout", "Tbias", {"host_inputs", "host_outputs"});
    RegBothInputs<V2, TF_QINT8>(op, "Tout", "Tbias", {"host_inputs", "host_outputs"});
    RegBothInputs<V2, TF_QUINT8>(op, "Tout", "Tbias", {"host_inputs", "host_outputs"});
  }
  // the fused node of this plugin's graph pass (float activations, quantized here against their own range)
  RegDynamicInput<TF_QUINT8, TF_FLOAT>();
  RegDynamicInput<TF_QINT8, TF_FLOAT>();
  RegDynamicInput<TF_QUINT8, TF_BFLOAT16>();
  RegDynamicInput<TF_QINT8, TF_BFLOAT16>();
  RegDynamicInput<TF_QUINT8, TF_QINT8>();
  RegDynamicInput<TF_QINT8, TF_QINT8>();
  RegDynamicInput<TF_QUINT8, TF_QUINT8>();
  RegDynamicInput<TF_QINT8, TF_QUINT8>();
}

}  // namespace itex_amd
