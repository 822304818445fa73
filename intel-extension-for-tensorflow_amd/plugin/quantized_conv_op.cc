// Quantized Conv2D op kernels: QuantizedConv2D, ...PerChannel, ...WithBias, ...AndRelu, ...AndRequantize and
// their combinations, and the list-attribute form _QuantizedConv2D / _ITEXQuantizedConv2DV2
// (itex/core/kernels/common/quantized_conv_ops.h:63-597 over conv_ops.h:615-1150; device registrations in
// itex/core/kernels/gpu/quantized_conv_ops.cc).  Host half as in the reference: attribute and fusion
// parsing, input indices, geometry, output scales and bias factors; the convolution itself runs on the filter
// prepacked as a [KH*KW*C, O] matrix: as an implicit GEMM (itexhip_qconv2d) where the input channels are a multiple
// of 16, on a channel- and window-padded copy (itexhip_pad_nhwc8) where they are at most 8, as a plain GEMM for 1x1
// windows, else as itexhip_im2col8 + itexhip_qgemm; depthwise windows have a kernel of their own.
// Not carried over: Swish / HardSwish fusions, 3-D variants, NCHW.
#include <mutex>
#include <algorithm>
#include <cmath>
#include <cstring>
#include <string>
#include <vector>

#include "device_vector_cache.h"
#include "itexhip.h"
#include "op_kernel.h"
#include "qparams.h"

namespace itex_amd {
namespace {

// fusions of the ops without a fused_ops attribute (quantized_conv_ops.h:44-60)
std::vector<std::string> LegacyFusions(const std::string& op) {
  std::string name = op;
  if (name.rfind("_ITEX", 0) == 0) name = name.substr(5);
  if (name == "QuantizedConv2D" || name == "QuantizedConv2DPerChannel" || name == "QuantizedDepthwiseConv2D") return {};
  if (name == "QuantizedDepthwiseConv2DWithBias") return {"BiasAdd"};
  if (name == "QuantizedDepthwiseConv2DWithBiasAndRelu") return {"BiasAdd", "Relu"};
  if (name == "QuantizedDepthwiseConv2DWithBiasAndReluAndRequantize") return {"BiasAdd", "Relu", "Requantize"};
  if (name == "QuantizedConv2DWithBias") return {"BiasAdd"};
  if (name == "QuantizedConv2DWithBiasAndRelu") return {"BiasAdd", "Relu"};
  if (name == "QuantizedConv2DAndRelu") return {"Relu"};
  if (name == "QuantizedConv2DAndRequantize") return {"Requantize"};
  if (name == "QuantizedConv2DAndReluAndRequantize") return {"Relu", "Requantize"};
  if (name == "QuantizedConv2DWithBiasAndRequantize") return {"BiasAdd", "Requantize"};
  if (name == "QuantizedConv2DWithBiasAndReluAndRequantize") return {"BiasAdd", "Relu", "Requantize"};
  if (name == "QuantizedConv2DWithBiasSumAndReluAndRequantize" || name == "QuantizedConv2DWithBiasSignedSumAndReluAndRequantize")
    return {"BiasAdd", "Sum", "Relu", "Requantize"};
  return {};
}

// TensorFlow's GetWindowedOutputSizeVerbose
bool OutDim(int64_t in, int64_t k, int64_t stride, int64_t dil, const std::string& padding, int64_t before, int64_t after,
            int64_t* out, int64_t* lead) {
  const int64_t eff = (k - 1) * dil + 1;
  if (padding == "VALID") {
    *out = (in - eff + stride) / stride;
    *lead = 0;
  } else if (padding == "SAME") {
    *out = (in + stride - 1) / stride;
    *lead = std::max<int64_t>((*out - 1) * stride + eff - in, 0) / 2;
  } else {
    *out = (in + before + after - eff + stride) / stride;
    *lead = before;
  }
  return *out >= 0;
}

class QuantizedConv2DOp : public OpKernel {
 public:
  QuantizedConv2DOp(OpKernelConstruction* ctx, const std::string& op, bool new_api, TF_DataType t_in, TF_DataType t_out)
      : t_in_(t_in), t_out_(t_out), depthwise_(op.find("Depthwise") != std::string::npos) {
    std::vector<int64_t> strides, dilations;
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("dilations", &dilations));
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("strides", &strides));
    ITEX_REQUIRES(ctx, strides.size() == 4, TF_INVALID_ARGUMENT, "Sliding window strides field must specify 4 dimensions");
    ITEX_REQUIRES(ctx, dilations.size() == 4, TF_INVALID_ARGUMENT, "Sliding window dilations field must specify 4 dimensions");
    if (ctx->HasAttr("data_format")) {
      std::string fmt;
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("data_format", &fmt));
      ITEX_REQUIRES(ctx, fmt == "NHWC" || fmt == "NCHW", TF_INVALID_ARGUMENT, "Invalid data format");
      ITEX_REQUIRES(ctx, fmt == "NHWC", TF_UNIMPLEMENTED, "the quantized Conv2D on this device takes NHWC tensors");
    }
    ITEX_REQUIRES(ctx, strides[0] == 1 && strides[3] == 1, TF_UNIMPLEMENTED,
                  "Current implementation does not yet support strides in the batch and depth dimensions.");
    ITEX_REQUIRES(ctx, dilations[0] == 1 && dilations[3] == 1, TF_INVALID_ARGUMENT,
                  "Current implementation does not yet support dilations in the batch and depth dimensions.");
    ITEX_REQUIRES(ctx, strides[1] > 0 && strides[2] > 0, TF_INVALID_ARGUMENT, "Row and column strides should be larger than 0.");
    ITEX_REQUIRES(ctx, dilations[1] > 0 && dilations[2] > 0, TF_INVALID_ARGUMENT, "Dilated rates should be larger than 0.");
    stride_h_ = strides[1]; stride_w_ = strides[2]; dil_h_ = dilations[1]; dil_w_ = dilations[2];
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("padding", &padding_));
    ITEX_REQUIRES(ctx, padding_ == "SAME" || padding_ == "VALID" || padding_ == "EXPLICIT", TF_INVALID_ARGUMENT,
                  "padding must be SAME, VALID or EXPLICIT");
    for (const char* attr : {"explicit_paddings", "padding_list"})  // the second is the legacy spelling (:121-124)
      if (ctx->HasAttr(attr)) {
        std::vector<int64_t> p;
        ITEX_REQUIRES_OK(ctx, ctx->GetAttr(attr, &p));
        if (!p.empty()) explicit_ = p;
      }
    if (!explicit_.empty()) {  // conv_ops.h:412-427: explicit paddings win when present
      ITEX_REQUIRES(ctx, explicit_.size() == 8, TF_INVALID_ARGUMENT, "explicit paddings must hold 8 values for a 2-D convolution");
      ITEX_REQUIRES(ctx, explicit_[0] == 0 && explicit_[1] == 0 && explicit_[6] == 0 && explicit_[7] == 0, TF_INVALID_ARGUMENT,
                    "explicit padding of the batch and depth dimensions must be 0");
      padding_ = "EXPLICIT";
    }
    ITEX_REQUIRES(ctx, padding_ != "EXPLICIT" || explicit_.size() == 8, TF_INVALID_ARGUMENT, "EXPLICIT padding without paddings");

    std::vector<std::string> fused;
    if (ctx->HasAttr("fused_ops")) ITEX_REQUIRES_OK(ctx, ctx->GetAttr("fused_ops", &fused));
    const std::vector<std::string> legacy = LegacyFusions(op);
    ITEX_REQUIRES(ctx, !(fused.size() > 0 && legacy.size() > 0), TF_INVALID_ARGUMENT,
                  "QuantizedConv fused ops should be only availabe through either new API or old API, got both.");
    if (fused.empty()) fused = legacy;
    for (const std::string& f : fused) {
      if (f == "BiasAdd") fuse_bias_ = true;
      else if (f == "Requantize") fuse_requantize_ = true;
      else if (f == "Dequantize") fuse_dequantize_ = true;
      else if (f == "Relu") { activation_ = ITEXHIP_ELT_RELU; if (sum_position_ == 0) sum_position_ = -1; }
      else if (f == "LeakyRelu") { activation_ = ITEXHIP_ELT_RELU; leaky_ = true; if (sum_position_ == 0) sum_position_ = -1; }
      // quantized_conv_ops.h:83, 86, 100, 103 with the table's alpha = 1 (onednn_post_op_util.cc:38, 59-60)
      else if (f == "Elu") { activation_ = ITEXHIP_ELT_ELU; transcendental_ = true; }
      else if (f == "Sigmoid") { activation_ = ITEXHIP_ELT_LOGISTIC; transcendental_ = true; }
      else if (f == "Sum") sum_position_ = sum_position_ == -1 ? 2 : 1;  // after / before the activation
      else
        ITEX_REQUIRES(ctx, false, TF_UNIMPLEMENTED, "the " + f + " fusion of the quantized Conv2D is not implemented on this device");
    }
    if (sum_position_ < 0) sum_position_ = 0;
    if (leaky_) ITEX_REQUIRES_OK(ctx, ctx->GetAttr("alpha", &alpha_));
    ITEX_REQUIRES(ctx, !(depthwise_ && sum_position_ != 0), TF_UNIMPLEMENTED, "the depthwise convolution has no Sum fusion on this device");
    ITEX_REQUIRES(ctx, !(transcendental_ && (depthwise_ || sum_position_ != 0)), TF_UNIMPLEMENTED,
                  "Elu / Sigmoid are fused into the plain quantized Conv2D only (no Sum, not depthwise) on this device");
    if (sum_position_ != 0) {
      // quantized_conv_ops.h:202-218, 398-433: an 8-bit summand under an 8-bit output; the qint32 output with a float
      // summand (the graph before Requantize is fused) is not built
      ITEX_REQUIRES(ctx, fuse_requantize_, TF_UNIMPLEMENTED,
                    "the Sum fusion of the quantized Conv2D is implemented together with Requantize only");
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("Tsummand", &t_summand_));
      ITEX_REQUIRES(ctx, t_summand_ == TF_QINT8 || t_summand_ == TF_QUINT8, TF_UNIMPLEMENTED,
                    "the Sum fusion of the quantized Conv2D takes a qint8 or quint8 summand on this device");
      ITEX_REQUIRES(ctx, !(t_summand_ == TF_QUINT8 && t_out == TF_QINT8), TF_INVALID_ARGUMENT,
                    "Current fusion requires summand has same dtype as output if output is qint8");
    }
    if (fuse_requantize_)
      ITEX_REQUIRES(ctx, t_out == TF_QINT8 || t_out == TF_QUINT8, TF_INVALID_ARGUMENT,
                    "QuantizedConv: unsupported output type when Requantize is fused.");
    if (fuse_dequantize_)
      ITEX_REQUIRES(ctx, t_out == TF_FLOAT || t_out == TF_BFLOAT16, TF_INVALID_ARGUMENT,
                    "QuantizedConv: unsupported output type when Dequantize is fused.");
    if (fuse_bias_ && ctx->HasAttr("Tbias")) {
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("Tbias", &t_bias_));
      ITEX_REQUIRES(ctx, t_bias_ == TF_FLOAT || t_bias_ == TF_QINT32, TF_UNIMPLEMENTED,
                    "the quantized Conv2D takes a float or qint32 bias on this device");
    }
    if (ctx->HasAttr("is_filter_const")) ITEX_REQUIRES_OK(ctx, ctx->GetAttr("is_filter_const", &is_filter_const_));
    if (ctx->HasAttr("is_bias_const")) ITEX_REQUIRES_OK(ctx, ctx->GetAttr("is_bias_const", &is_bias_const_));

    // input positions (:246-317)
    const int bias_off = fuse_bias_ ? 1 : 0;
    src_min_idx_ = 2 + bias_off;
    filter_min_idx_ = src_min_idx_ + 2;
    freezed_idx_ = 6 + bias_off;  // both spellings, without a summand and with a float / qint32 bias
    if (sum_position_ != 0) {
      if (new_api) {  // input, filter, {bias}, summand, min/max input, min/max filter, min/max summand, min/max freezed output
        summand_idx_ = 2 + bias_off;
        src_min_idx_ = 3 + bias_off;
        filter_min_idx_ = src_min_idx_ + 2;
        summand_min_idx_ = 6 + bias_off + 1;
        freezed_idx_ = summand_min_idx_ + 2;
      } else {        // ..., min/max freezed output, summand, min/max summand
        summand_idx_ = 8 + bias_off;
        summand_min_idx_ = 9 + bias_off;
      }
    }
  }

  void Compute(OpKernelContext* ctx) override {
    // one Compute at a time per node: the cached device vectors below are reassigned in place, and TensorFlow may run
    // one node from several threads (the reference serialises its kernels the same way, conv_ops.h:786,
    // quantized_matmul_common.h:62)
    std::lock_guard<std::mutex> lock(mu_);
    Tensor x = ctx->input(0);
    Tensor filter = ctx->input(1);
    if (!ctx->ok()) return;
    ITEX_REQUIRES(ctx, ctx->num_inputs() >= filter_min_idx_ + 2 && (!fuse_requantize_ || ctx->num_inputs() >= freezed_idx_ + 2) &&
                           (sum_position_ == 0 || ctx->num_inputs() >= summand_min_idx_ + 2),
                  TF_INVALID_ARGUMENT, "the min / max inputs are missing");
    Tensor min_in_t = ctx->input(src_min_idx_), max_in_t = ctx->input(src_min_idx_ + 1);
    Tensor min_f_t = ctx->input(filter_min_idx_), max_f_t = ctx->input(filter_min_idx_ + 1);
    if (!ctx->ok()) return;
    ITEX_REQUIRES(ctx, x.dims() == 4 && filter.dims() == 4, TF_INVALID_ARGUMENT, "input and filter must be 4-dimensional");
    ITEX_REQUIRES(ctx, x.dtype() == t_in_ && filter.dtype() == TF_QINT8, TF_INVALID_ARGUMENT,
                  "quantized Conv2D operand types do not match the kernel");
    const int64_t B = x.dim_size(0), H = x.dim_size(1), W = x.dim_size(2), C = x.dim_size(3);
    // depthwise: the filter is [KH, KW, C, multiplier] and the output has C * multiplier channels (conv_ops.h:395-397)
    const int64_t KH = filter.dim_size(0), KW = filter.dim_size(1);
    const int64_t O = depthwise_ ? filter.dim_size(2) * filter.dim_size(3) : filter.dim_size(3);
    ITEX_REQUIRES(ctx, filter.dim_size(2) == C, TF_INVALID_ARGUMENT,
                  "input depth " + std::to_string(C) + " vs. filter input depth " + std::to_string(filter.dim_size(2)));
    ITEX_REQUIRES(ctx, KH > 0 && KW > 0, TF_INVALID_ARGUMENT, "empty filter window");
    const int64_t depth = min_f_t.NumElements();
    ITEX_REQUIRES(ctx, max_f_t.NumElements() == depth && (depth == 1 || depth == O), TF_INVALID_ARGUMENT,
                  "min_filter / max_filter must be scalars or hold one entry per output channel");

    itexhip_conv_geometry g{};
    g.batch = B; g.in_h = H; g.in_w = W; g.in_c = C; g.k_h = KH; g.k_w = KW;
    g.stride_h = static_cast<int>(stride_h_); g.stride_w = static_cast<int>(stride_w_);
    g.dil_h = static_cast<int>(dil_h_); g.dil_w = static_cast<int>(dil_w_);
    const int64_t pt = explicit_.empty() ? 0 : explicit_[2], pb = explicit_.empty() ? 0 : explicit_[3];
    const int64_t pl = explicit_.empty() ? 0 : explicit_[4], pr = explicit_.empty() ? 0 : explicit_[5];
    ITEX_REQUIRES(ctx, OutDim(H, KH, stride_h_, dil_h_, padding_, pt, pb, &g.out_h, &g.pad_top) &&
                           OutDim(W, KW, stride_w_, dil_w_, padding_, pl, pr, &g.out_w, &g.pad_left),
                  TF_INVALID_ARGUMENT, "Computed output size would be negative");
    const int64_t M = B * g.out_h * g.out_w, K = KH * KW * C, Kp = (K + 15) / 16 * 16;

    // ---- output scales and bias factors (ExtendInt8PostOps :329-393, GetBiasHandle :448-597), fp32 on the host
    const float min_in = min_in_t.flat<float>()[0], max_in = max_in_t.flat<float>()[0];
    const float* min_f = min_f_t.flat<float>();
    const float* max_f = max_f_t.flat<float>();
    const bool out_q8 = t_out_ == TF_QINT8 || t_out_ == TF_QUINT8;
    const bool out_f = t_out_ == TF_FLOAT || t_out_ == TF_BFLOAT16;
    float min_out = 0.0f, max_out = 0.0f;
    if (out_q8) {
      ITEX_REQUIRES(ctx, fuse_requantize_, TF_INVALID_ARGUMENT, "an 8-bit output needs the Requantize fusion");
      Tensor mo = ctx->input(freezed_idx_), xo = ctx->input(freezed_idx_ + 1);
      if (!ctx->ok()) return;
      min_out = mo.flat<float>()[0];
      max_out = xo.flat<float>()[0];
    }
    std::vector<float> scales(depth, 1.0f), factors(depth, 1.0f);
    const float in_range = std::max(std::abs(min_in), std::abs(max_in));
    const float int_const_scale_limit = (t_in_ == TF_QUINT8) ? static_cast<float>(255.0 * 127.0) : static_cast<float>(127.0 * 127.0);
    if (out_f) {
      const float int_input_limit = (t_in_ == TF_QUINT8) ? 255.0f : 127.0f;
      const float src_qscale_f32 = in_range / int_input_limit;
      for (int64_t i = 0; i < depth; ++i) {
        const float wei_qscale_f32 = std::max(std::abs(min_f[i]), std::abs(max_f[i])) / 127.0f;
        scales[i] = src_qscale_f32 * wei_qscale_f32;
      }
    } else if (out_q8) {
      const float int_output_limit = (t_out_ == TF_QUINT8) ? 255.0f : 127.0f;
      const float float_output_range = std::max(std::abs(min_out), std::abs(max_out));
      for (int64_t i = 0; i < depth; ++i) {
        const float float_filter_range = std::max(std::abs(min_f[i]), std::abs(max_f[i]));
        scales[i] = int_output_limit * in_range * float_filter_range / (int_const_scale_limit * float_output_range);
      }
    }
    if (fuse_bias_) {
      for (int64_t i = 0; i < depth; ++i) {
        const float filt_range = std::max(std::abs(max_f[i]), std::abs(min_f[i]));
        if (t_bias_ == TF_QINT32) {
          factors[i] = t_out_ == TF_QINT32 ? 1.0f : out_f ? (in_range * filt_range) / int_const_scale_limit : scales[i];
        } else {
          const float tmp_scale = int_const_scale_limit / (in_range * filt_range);
          factors[i] = tmp_scale * scales[i];
        }
      }
    }

    void* stream = ctx->stream();
    // ---- fewer than 16 input channels (the first layer of a vision network): the patch rows have no 16-byte piece that
    // lies inside one pixel.  Instead of writing the patch matrix out, the input is copied once with 4 or 8 channels and
    // with the windows' spatial padding in place, the filter is padded to the same channel count and to a window row of
    // a multiple of 16 bytes, and the tile kernel gathers runs of whole pixels from that copy.  All padding bytes are
    // zero on both sides: the integer sums are unchanged.
    itexhip_conv_geometry gn = g;
    bool narrow = false;
    const int64_t Cn = C <= 4 ? 4 : 8, KWn = (KW * Cn + 15) / 16 * 16 / Cn;
    if (!depthwise_ && C > 0 && C <= 8 && dil_w_ == 1 && !transcendental_ && sum_position_ == 0 && M > 0 && O > 0 && O % 4 == 0) {
      gn.in_c = Cn;
      gn.k_w = KWn;
      gn.in_h = std::max<int64_t>(g.pad_top + H, (g.out_h - 1) * stride_h_ + (KH - 1) * dil_h_ + 1);
      gn.in_w = std::max<int64_t>(g.pad_left + W, (g.out_w - 1) * stride_w_ + KWn);
      gn.in_w = (gn.in_w + 16 / Cn - 1) / (16 / Cn) * (16 / Cn);  // rows of whole 16-byte vectors: the copy writes one per thread
      gn.pad_top = gn.pad_left = 0;
      // legality without the buffers (they come 16-byte aligned from the allocator)
      const void* aligned16 = reinterpret_cast<const void*>(static_cast<uintptr_t>(64));
      narrow = itexhip_qconv2d_implicit_ok(&gn, aligned16, O, t_out_, aligned16) != 0;
    }
    const int64_t Kn = KH * KWn * Cn;
    // ---- filter: packed once when constant (the HWIO tensor read as a [K, O] matrix)
    const int64_t pack_k = narrow ? Kn : K;
    const bool repack = !depthwise_ &&
                        (!packed_.valid() || !is_filter_const_ || packed_src_ != filter.data() || packed_k_ != pack_k || packed_n_ != O);
    if (repack && O > 0) {
      packed_ = ctx->allocate_temp(TF_QINT8, {std::max<int64_t>(itexhip_qgemm_packed_bytes(narrow ? Kn : Kp, O), 16)});
      colsum_ = ctx->allocate_temp(TF_INT32, {O});
      if (!ctx->ok()) return;
      const int8_t* w = filter.flat<int8_t>();
      Tensor padded_filter;
      if (narrow) {  // [KH, KW, C, O] -> [KH, KWn, Cn, O]
        padded_filter = ctx->allocate_temp(TF_QINT8, {KH, KWn, Cn, O});
        if (!ctx->ok()) return;
        const int st = itexhip_pad_nhwc8(w, KH, KW, C, O, 0, 0, KWn, Cn, O, padded_filter.data(), stream);
        ITEX_REQUIRES(ctx, st == ITEXHIP_OK, TF_ABORTED, std::string("Operation received an exception: ") + itexhip_last_error());
        w = padded_filter.flat<int8_t>();
      }
      const int st = itexhip_qgemm_prepack_b(w, 0, pack_k, O, packed_.flat<int8_t>(), colsum_.flat<int32_t>(), stream);
      ITEX_REQUIRES(ctx, st == ITEXHIP_OK, TF_ABORTED, std::string("Operation received an exception: ") + itexhip_last_error());
      packed_src_ = filter.data();
      packed_k_ = pack_k;
      packed_n_ = O;
    }
    std::vector<float> both(scales);
    both.insert(both.end(), factors.begin(), factors.end());
    float* params = params_.Get(ctx, both.data(), both.size(), TF_FLOAT);
    if (params == nullptr) return;

    Tensor out = ctx->allocate_output(0, t_out_, {B, g.out_h, g.out_w, O});
    if (!ctx->ok()) return;
    if (M > 0 && O > 0) {
      // ---- bias in the epilogue's units
      // A constant bias (is_bias_const, quantized_conv_ops.h:168-174, 448-455: the reference caches the scaled bias too) is
      // scaled once and kept while its buffer and the factors stay the same; likewise the zero vector of a node without
      // bias (the MFMA kernels' vector epilogue wants a bias vector).
      const float* bias_dev = nullptr;
      const void* bias_src = nullptr;
      if (fuse_bias_) {
        Tensor bias = ctx->input(2);
        if (!ctx->ok()) return;
        ITEX_REQUIRES(ctx, bias.dtype() == t_bias_ && bias.NumElements() == O, TF_INVALID_ARGUMENT,
                      "bias must have one entry per output channel and the type of Tbias");
        bias_src = bias.data();
      }
      const bool reuse = sbias_.valid() && sbias_n_ == O && sbias_src_ == bias_src && sbias_factors_ == factors &&
                         (!fuse_bias_ || is_bias_const_);
      if (!reuse) {
        sbias_ = ctx->allocate_temp(TF_FLOAT, {O});
        if (!ctx->ok()) return;
        const int st = fuse_bias_ ? itexhip_scale_vector(bias_src, t_bias_, params + depth, depth, O, sbias_.flat<float>(), stream)
                                  : itexhip_memset32_async(sbias_.data(), 0, static_cast<size_t>(O) * sizeof(float), stream);
        ITEX_REQUIRES(ctx, st == ITEXHIP_OK, TF_ABORTED, std::string("Operation received an exception: ") + itexhip_last_error());
        sbias_n_ = O;
        sbias_src_ = bias_src;
        sbias_factors_ = factors;
      }
      bias_dev = sbias_.flat<float>();
      itexhip_epilogue dep{};
      if (depthwise_) {  // no matrix product in it: a kernel of its own on the filter as TensorFlow stores it
        dep.n_scales = static_cast<int>(depth);
        if (activation_ != 0) dep.elt[dep.n_eltwise++] = {activation_, leaky_ ? alpha_ : 0.0f, 0.0f};
        const int st = itexhip_qdepthwise_conv2d(x.data(), t_in_, &g, filter.dim_size(3), filter.flat<int8_t>(), params, bias_dev, &dep,
                                                 t_out_, out.data(), stream);
        ITEX_REQUIRES(ctx, st == ITEXHIP_OK, st == ITEXHIP_INVALID_ARGUMENT ? TF_INVALID_ARGUMENT : TF_ABORTED,
                      std::string("Operation received an exception: ") + itexhip_last_error());
      }
      if (!depthwise_) {
      // ---- summand of the Sum fusion
      const void* summand_dev = nullptr;
      int summand_type = 0;
      float sum_scale = 0.0f;
      if (sum_position_ != 0) {
        Tensor summand = ctx->input(summand_idx_);
        Tensor min_s = ctx->input(summand_min_idx_), max_s = ctx->input(summand_min_idx_ + 1);
        if (!ctx->ok()) return;
        ITEX_REQUIRES(ctx, (summand.dtype() == TF_QINT8 || summand.dtype() == TF_QUINT8) && summand.NumElements() == M * O,
                      TF_INVALID_ARGUMENT, "the summand must be a qint8 / quint8 tensor of the output's shape");
        // :398-433; the destination's previous contents are read as the output type (:622-626 bit-casts a qint8 summand)
        const float scale_output = std::max(std::abs(min_out), std::abs(max_out));
        const float scale_summand = std::max(std::abs(min_s.flat<float>()[0]), std::abs(max_s.flat<float>()[0]));
        if (t_out_ == TF_QUINT8 && summand.dtype() == TF_QINT8) sum_scale = 255.0f * scale_summand / (scale_output * 127.0f);
        else sum_scale = scale_summand / scale_output;
        summand_dev = summand.data();
        summand_type = t_out_;
      }
      // ---- patches, then the quantized GEMM
      const void* a = x.data();
      Tensor cols, x_narrow;
      if (narrow) {
        x_narrow = ctx->allocate_temp(t_in_, {B, gn.in_h, gn.in_w, Cn});
        if (!ctx->ok()) return;
        int st = itexhip_pad_nhwc8(x.data(), B, H, W, C, g.pad_top, g.pad_left, gn.in_h, gn.in_w, Cn, x_narrow.data(), stream);
        ITEX_REQUIRES(ctx, st == ITEXHIP_OK, TF_ABORTED, std::string("Operation received an exception: ") + itexhip_last_error());
        ITEX_REQUIRES(ctx, itexhip_qconv2d_implicit_ok(&gn, x_narrow.data(), O, t_out_, out.data()) != 0, TF_INTERNAL,
                      "the padded input or the output is not 16-byte aligned");
        itexhip_epilogue epn{};
        epn.n_scales = static_cast<int>(depth);
        if (activation_ != 0) epn.elt[epn.n_eltwise++] = {activation_, leaky_ ? alpha_ : 0.0f, 0.0f};
        st = itexhip_qconv2d(x_narrow.data(), t_in_, &gn, packed_.flat<int8_t>(), colsum_.flat<int32_t>(), O, params, bias_dev, &epn,
                             t_out_, out.data(), stream);
        ITEX_REQUIRES(ctx, st == ITEXHIP_OK, st == ITEXHIP_INVALID_ARGUMENT ? TF_INVALID_ARGUMENT : TF_ABORTED,
                      std::string("Operation received an exception: ") + itexhip_last_error());
      }
      if (!narrow) {
      const bool pointwise = KH == 1 && KW == 1 && stride_h_ == 1 && stride_w_ == 1 && g.pad_top == 0 && g.pad_left == 0 &&
                             g.out_h == H && g.out_w == W && K == Kp;
      // windows the tile kernel can gather by itself (input channels a multiple of 16, ...) need no patch matrix
      // (the implicit-GEMM kernels carry the cheap post-op chains only: Elu / Sigmoid go through the patch matrix)
      const bool implicit = !pointwise && !transcendental_ && itexhip_qconv2d_implicit_ok(&g, x.data(), O, t_out_, out.data()) != 0 &&
                            (reinterpret_cast<uintptr_t>(summand_dev) & 3) == 0;
      if (!pointwise && !implicit) {
        cols = ctx->allocate_temp(t_in_, {M, Kp});
        if (!ctx->ok()) return;
        const int st = itexhip_im2col8(x.data(), &g, Kp, cols.data(), stream);
        ITEX_REQUIRES(ctx, st == ITEXHIP_OK, TF_ABORTED, std::string("Operation received an exception: ") + itexhip_last_error());
        a = cols.data();
      }
      itexhip_epilogue ep{};
      ep.n_scales = static_cast<int>(depth);
      if (sum_position_ == 1) ep.elt[ep.n_eltwise++] = {ITEXHIP_ELT_SUM, sum_scale, 0.0f};
      if (activation_ != 0) ep.elt[ep.n_eltwise++] = {activation_, transcendental_ ? 1.0f : leaky_ ? alpha_ : 0.0f, 0.0f};
      if (sum_position_ == 2) ep.elt[ep.n_eltwise++] = {ITEXHIP_ELT_SUM, sum_scale, 0.0f};
      int st;
      if (summand_dev != nullptr) {
        st = implicit ? itexhip_qconv2d_sum(x.data(), t_in_, &g, packed_.flat<int8_t>(), colsum_.flat<int32_t>(), O, params,
                                            bias_dev, &ep, summand_dev, summand_type, t_out_, out.data(), stream)
                      : itexhip_qgemm_sum(a, t_in_, packed_.flat<int8_t>(), colsum_.flat<int32_t>(), M, Kp, O, params, bias_dev,
                                          &ep, summand_dev, summand_type, t_out_, out.data(), stream);
      } else {
        st = implicit ? itexhip_qconv2d(x.data(), t_in_, &g, packed_.flat<int8_t>(), colsum_.flat<int32_t>(), O, params,
                                        bias_dev, &ep, t_out_, out.data(), stream)
                      : itexhip_qgemm(a, t_in_, packed_.flat<int8_t>(), colsum_.flat<int32_t>(), M, Kp, O, params, bias_dev,
                                      &ep, t_out_, out.data(), stream);
      }
      ITEX_REQUIRES(ctx, st == ITEXHIP_OK, st == ITEXHIP_INVALID_ARGUMENT ? TF_INVALID_ARGUMENT : TF_ABORTED,
                    std::string("Operation received an exception: ") + itexhip_last_error());
      }  // !narrow
      }  // !depthwise_
    }

    // ---- output ranges in host memory (AllocateNativeOutputMinMax, quantized_ops.h:142-203)
    if (out_q8) {
      Tensor omin = ctx->allocate_output(1, TF_FLOAT, {});
      Tensor omax = ctx->allocate_output(2, TF_FLOAT, {});
      if (!ctx->ok()) return;
      omin.flat<float>()[0] = min_out;
      omax.flat<float>()[0] = max_out;
    } else if (t_out_ == TF_QINT32) {
      const bool scalar = min_f_t.dims() == 0;
      const std::vector<int64_t> shp = scalar ? std::vector<int64_t>{} : std::vector<int64_t>{depth};
      Tensor omin = ctx->allocate_output(1, TF_FLOAT, shp);
      Tensor omax = ctx->allocate_output(2, TF_FLOAT, shp);
      if (!ctx->ok()) return;
      for (int64_t i = 0; i < (scalar ? 1 : depth); ++i)
        qparams::RangeForMultiplication(t_in_, TF_QINT8, min_in, max_in, min_f[i], max_f[i], &omin.flat<float>()[i],
                                        &omax.flat<float>()[i]);
    }
  }

 private:
  TF_DataType t_in_, t_out_, t_bias_ = TF_FLOAT;
  bool depthwise_ = false;
  TF_DataType t_summand_ = TF_QUINT8;
  int sum_position_ = 0;  // 0 none, 1 before the activation, 2 after it
  int summand_idx_ = -1, summand_min_idx_ = -1;
  int64_t stride_h_ = 1, stride_w_ = 1, dil_h_ = 1, dil_w_ = 1;
  std::string padding_;
  std::vector<int64_t> explicit_;
  bool fuse_bias_ = false, fuse_requantize_ = false, fuse_dequantize_ = false, leaky_ = false, transcendental_ = false;
  int activation_ = 0;
  float alpha_ = 0.0f;
  bool is_filter_const_ = true;
  bool is_bias_const_ = true;   // the legacy ops have no such attribute: their bias is taken as constant (:168-174)
  Tensor sbias_;
  const void* sbias_src_ = nullptr;
  int64_t sbias_n_ = -1;
  std::vector<float> sbias_factors_;
  int src_min_idx_ = 2, filter_min_idx_ = 4, freezed_idx_ = 6;
  Tensor packed_, colsum_;
  const void* packed_src_ = nullptr;
  int64_t packed_k_ = -1, packed_n_ = -1;
  std::mutex mu_;
  DeviceVectorCache<float> params_;
};

// the op name is needed at construction (legacy fusions), so each registration carries it as a template value
template <int NAME, bool NEW_API, int TIN, int TOUT>
struct ConvKernel;

const char* const kLegacyNames[] = {"QuantizedConv2D", "QuantizedConv2DPerChannel", "QuantizedConv2DWithBias",
                                    "QuantizedConv2DWithBiasAndRelu", "QuantizedConv2DAndRelu", "QuantizedConv2DAndRequantize",
                                    "QuantizedConv2DAndReluAndRequantize", "QuantizedConv2DWithBiasAndRequantize",
                                    "QuantizedConv2DWithBiasAndReluAndRequantize",
                                    "QuantizedConv2DWithBiasSumAndReluAndRequantize",
                                    "QuantizedConv2DWithBiasSignedSumAndReluAndRequantize",
                                    "QuantizedDepthwiseConv2D", "QuantizedDepthwiseConv2DWithBias",
                                    "QuantizedDepthwiseConv2DWithBiasAndRelu",
                                    "QuantizedDepthwiseConv2DWithBiasAndReluAndRequantize"};

// NAME < 0 with NEW_API: the depthwise op
template <int NAME, bool NEW_API, int TIN, int TOUT>
struct ConvKernel : QuantizedConv2DOp {
  explicit ConvKernel(OpKernelConstruction* c)
      : QuantizedConv2DOp(c, NEW_API ? (NAME < 0 ? "_QuantizedDepthwiseConv2D" : "_QuantizedConv2D") : kLegacyNames[NAME < 0 ? 0 : NAME],
                          NEW_API, static_cast<TF_DataType>(TIN), static_cast<TF_DataType>(TOUT)) {}
};

template <int NAME, int TIN, int TOUT>
void RegLegacy(bool with_bias_types, std::initializer_list<const char*> host_args, int t_summand = 0) {
  for (const char* prefix : {"", "_ITEX"}) {
    const std::string op = std::string(prefix) + kLegacyNames[NAME];
    for (TF_DataType tb : {TF_FLOAT, TF_QINT32}) {
      if (!with_bias_types && tb != TF_FLOAT) continue;
      KernelDefBuilder b(op.c_str(), "QuantizedConvOp");
      b.TypeConstraint("Tinput", static_cast<TF_DataType>(TIN)).TypeConstraint("Tfilter", TF_QINT8);
      if (with_bias_types) b.TypeConstraint("Tbias", tb);
      if (t_summand != 0) b.TypeConstraint("Tsummand", static_cast<TF_DataType>(t_summand));
      b.TypeConstraint("out_type", static_cast<TF_DataType>(TOUT));
      for (const char* h : host_args) b.HostMemory(h);
      b.Register<ConvKernel<NAME, false, TIN, TOUT>>();
    }
  }
}

// Tsummand as the reference constrains it (quantized_conv_ops.cc:168-262): either 8-bit type under an 8-bit output, the
// output's own type otherwise
template <int TIN, int TOUT>
void RegNewApi() {
  const bool out_q8 = TOUT == TF_QINT8 || TOUT == TF_QUINT8;
  const std::vector<TF_DataType> summands = out_q8 ? std::vector<TF_DataType>{TF_QINT8, TF_QUINT8}
                                                   : std::vector<TF_DataType>{static_cast<TF_DataType>(TOUT)};
  static const char* const kNames[2][2] = {{"_QuantizedConv2D", "_ITEXQuantizedConv2DV2"},
                                           {"_QuantizedDepthwiseConv2D", "_ITEXQuantizedDepthwiseConv2DV2"}};
  for (const bool depthwise : {false, true})
    for (const char* op : kNames[depthwise ? 1 : 0])
      for (TF_DataType tb : {TF_FLOAT, TF_QINT32})
        for (TF_DataType ts : summands) {
          KernelDefBuilder b(op, "QuantizedConvOp");
          b.TypeConstraint("Tinput", static_cast<TF_DataType>(TIN)).TypeConstraint("Tfilter", TF_QINT8).TypeConstraint("Tbias", tb);
          b.TypeConstraint("Tsummand", ts).TypeConstraint("out_type", static_cast<TF_DataType>(TOUT));
          b.HostMemory("host_inputs").HostMemory("host_outputs");
          if (depthwise) b.Register<ConvKernel<-1, true, TIN, TOUT>>();
          else b.Register<ConvKernel<0, true, TIN, TOUT>>();
        }
}

}  // namespace

// Names, type constraints and host-memory arguments as registered by the reference for a device
// (itex/core/kernels/gpu/quantized_conv_ops.cc:77-310); the _ITEX names are the CPU-side renames
// (itex/core/graph/native_layout/native_layout.cc:118-145, 178-179).
void AddQuantizedConvKernels() {
  const std::initializer_list<const char*> plain = {"min_input", "max_input", "min_filter", "max_filter", "min_output", "max_output"};
  const std::initializer_list<const char*> req = {"min_input", "max_input", "min_filter", "max_filter", "min_freezed_output",
                                                  "max_freezed_output", "min_output", "max_output"};
  RegLegacy<0, TF_QINT8, TF_QINT32>(false, plain);  RegLegacy<0, TF_QUINT8, TF_QINT32>(false, plain);
  RegLegacy<1, TF_QINT8, TF_QINT32>(false, plain);  RegLegacy<1, TF_QUINT8, TF_QINT32>(false, plain);
  RegLegacy<2, TF_QINT8, TF_QINT32>(false, plain);  RegLegacy<2, TF_QUINT8, TF_QINT32>(false, plain);
  RegLegacy<3, TF_QINT8, TF_QINT32>(false, plain);  RegLegacy<3, TF_QUINT8, TF_QINT32>(false, plain);
  RegLegacy<4, TF_QUINT8, TF_QINT32>(false, plain);
  RegLegacy<5, TF_QINT8, TF_QINT8>(false, req);     RegLegacy<5, TF_QUINT8, TF_QINT8>(false, req);
  RegLegacy<6, TF_QUINT8, TF_QUINT8>(false, req);
  RegLegacy<7, TF_QINT8, TF_QINT8>(true, req);      RegLegacy<7, TF_QUINT8, TF_QINT8>(true, req);
  RegLegacy<8, TF_QINT8, TF_QUINT8>(true, req);     RegLegacy<8, TF_QUINT8, TF_QUINT8>(true, req);
  const std::initializer_list<const char*> sum = {"min_input", "max_input", "min_filter", "max_filter", "min_freezed_output",
                                                  "max_freezed_output", "min_summand", "max_summand", "min_output", "max_output"};
  RegLegacy<9, TF_QUINT8, TF_QUINT8>(true, sum, TF_QUINT8);
  RegLegacy<10, TF_QUINT8, TF_QUINT8>(true, sum, TF_QINT8);
  // depthwise, legacy spellings (:92-99, 126-129): quint8 input only
  RegLegacy<11, TF_QUINT8, TF_QINT32>(false, plain);
  RegLegacy<12, TF_QUINT8, TF_QINT32>(false, plain);
  RegLegacy<13, TF_QUINT8, TF_QINT32>(false, plain);
  RegLegacy<14, TF_QUINT8, TF_QUINT8>(true, req);
  RegNewApi<TF_QINT8, TF_QINT8>();   RegNewApi<TF_QUINT8, TF_QINT8>();
  RegNewApi<TF_QINT8, TF_QUINT8>();  RegNewApi<TF_QUINT8, TF_QUINT8>();
  RegNewApi<TF_QINT8, TF_FLOAT>();   RegNewApi<TF_QUINT8, TF_FLOAT>();
  RegNewApi<TF_QINT8, TF_BFLOAT16>(); RegNewApi<TF_QUINT8, TF_BFLOAT16>();
  RegNewApi<TF_QINT8, TF_QINT32>();  RegNewApi<TF_QUINT8, TF_QINT32>();
}

}  // namespace itex_amd
