// Parameter preparation of the quantized MatMul ops: the epilogue descriptor (host) and the
// per-channel output scales + scaled / zero-point-compensated bias (one small device kernel, so that
// a change of the activation range between calls costs no host-device synchronisation).
//
// Follows, operation by operation and in fp32:
//   ExtendInt8PostOps  itex/core/kernels/common/quantized_matmul_common.h:1472-1508 (legacy),
//                      :1610-1702 (V1), :1809-1908 (V2)
//   GetScaledBias      quantized_matmul_common.h:466-660 (fp32 bias)
//   PostOpUtil         itex/core/utils/onednn/onednn_post_op_util.cc:73-128, 237-273
#include "qmatmul_params.hpp"

namespace itexhip {
namespace {

__global__ void qmatmul_prepare_kernel(PrepArgs p, const float* __restrict__ min_b,
                                       const float* __restrict__ max_b, int64_t nb,
                                       const void* __restrict__ bias, const int32_t* __restrict__ colsum,
                                       int64_t N, float* __restrict__ scales_out,
                                       float* __restrict__ bias_out) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (j >= N) return;
  const ChannelScaleBias c = channel_scale_bias(p, min_b, max_b, nb, bias, colsum, N, j);
  if (p.n_scales > 1) scales_out[j] = c.scale;
  else if (p.n_scales == 1 && j == 0) scales_out[0] = c.scale;
  bias_out[j] = c.bias;
}

int eltwise_from_activation(int act, itexhip_eltwise* e) {
  switch (act) {
    case ITEXHIP_ACT_RELU: *e = {ITEXHIP_ELT_RELU, 0.0f, 0.0f}; return 1;
    case ITEXHIP_ACT_RELU6: *e = {ITEXHIP_ELT_CLIP, 0.0f, 6.0f}; return 1;
    case ITEXHIP_ACT_LEAKYRELU: *e = {ITEXHIP_ELT_RELU, 0.0f, 0.0f}; return 1;
    case ITEXHIP_ACT_GELU_APPROX: *e = {ITEXHIP_ELT_GELU_TANH, 0.0f, 0.0f}; return 1;
    case ITEXHIP_ACT_GELU_EXACT: *e = {ITEXHIP_ELT_GELU_ERF, 0.0f, 0.0f}; return 1;
    case ITEXHIP_ACT_ELU: *e = {ITEXHIP_ELT_ELU, 1.0f, 0.0f}; return 1;
    case ITEXHIP_ACT_SIGMOID: *e = {ITEXHIP_ELT_LOGISTIC, 1.0f, 0.0f}; return 1;
    case ITEXHIP_ACT_TANH: *e = {ITEXHIP_ELT_TANH, 0.0f, 0.0f}; return 1;
    case ITEXHIP_ACT_SWISH: *e = {ITEXHIP_ELT_SWISH, 1.0f, 0.0f}; return 1;
    case ITEXHIP_ACT_MISH: *e = {ITEXHIP_ELT_MISH, 0.0f, 0.0f}; return 1;
    default: return 0;
  }
}

int validate(const itexhip_matmul_params* p, int64_t nb) {
  ITEXHIP_REQUIRE(p != nullptr, "qmatmul: null params");
  ITEXHIP_REQUIRE(p->api == ITEXHIP_API_V2 || p->api == ITEXHIP_API_V1 || p->api == ITEXHIP_API_LEGACY,
                  "qmatmul: unknown api %d", p->api);
  ITEXHIP_REQUIRE(p->t_in == ITEXHIP_QUINT8 || p->t_in == ITEXHIP_QINT8, "qmatmul: T1 must be quint8 or qint8");
  ITEXHIP_REQUIRE(p->t_out == ITEXHIP_QINT32 || p->t_out == ITEXHIP_QINT8 || p->t_out == ITEXHIP_QUINT8 ||
                      is_float_out(p->t_out),
                  "qmatmul: unsupported output type %d", p->t_out);
  ITEXHIP_REQUIRE(p->input_mode == ITEXHIP_MIN_FIRST || p->input_mode == ITEXHIP_SCALED,
                  "Quantization mode must be either MIN_FIRST or SCALED");
  ITEXHIP_REQUIRE(nb >= 1, "qmatmul: empty weight range");
  ITEXHIP_REQUIRE(p->t_bias == 0 || p->t_bias == ITEXHIP_FLOAT || p->t_bias == ITEXHIP_QINT32 || is_float16_type(p->t_bias),
                  "qmatmul: Tbias must be float, bfloat16, half or qint32");
  ITEXHIP_REQUIRE(p->add_position >= 0 && p->add_position <= 2, "qmatmul: bad add_position");
  // the addend has the output's type (the sum post-op reads the destination, quantized_matmul_common.h:341-389): float,
  // bfloat16 or half; a quantized one is refused upstream as well
  if (p->add_position != 0 && !is_float_out(p->t_out)) {
    set_error("Quantized addend tensor is not implemented yet.");
    return ITEXHIP_UNIMPLEMENTED;
  }
  return ITEXHIP_OK;
}

}  // namespace
}  // namespace itexhip

using namespace itexhip;

extern "C" int itexhip_qmatmul_epilogue_desc(const itexhip_matmul_params* p, int64_t nb,
                                             itexhip_epilogue* ep) {
  if (int st = validate(p, nb)) return st;
  ITEXHIP_REQUIRE(ep != nullptr, "qmatmul: null epilogue");
  *ep = itexhip_epilogue{};
  const bool out_q8 = p->t_out == ITEXHIP_QINT8 || p->t_out == ITEXHIP_QUINT8;
  const float max_int8_output = (p->t_out == ITEXHIP_QUINT8) ? 255.0f : 127.0f;

  bool has_linear = false;
  const bool has_leaky = p->activation == ITEXHIP_ACT_LEAKYRELU;
  // post-ops in fused_ops order; "Add" is a sum post-op with scale 1 and no activation
  if (p->add_position == 1) ep->elt[ep->n_eltwise++] = {ITEXHIP_ELT_SUM, 1.0f, 0.0f};
  if (eltwise_from_activation(p->activation, &ep->elt[ep->n_eltwise])) ep->n_eltwise++;
  if (p->add_position == 2) ep->elt[ep->n_eltwise++] = {ITEXHIP_ELT_SUM, 1.0f, 0.0f};
  if (p->api == ITEXHIP_API_V2 && p->has_requantize && p->out_min_first) {
    ep->elt[ep->n_eltwise++] = {ITEXHIP_ELT_LINEAR, 1.0f, 0.0f};
    has_linear = true;
  }
  float linear_alpha = 0.0f, linear_beta = 0.0f;
  if (p->api == ITEXHIP_API_V2) {
    if (p->has_requantize || p->has_dequantize) ep->n_scales = static_cast<int>(nb);
    if (has_linear) {
      const float range_output = p->max_out - p->min_out;
      linear_alpha = max_int8_output / range_output;
      linear_beta = -p->min_out * max_int8_output / range_output;
    }
  } else if (p->api == ITEXHIP_API_V1) {
    ep->n_scales = (p->t_out == ITEXHIP_QINT32) ? 1 : static_cast<int>(nb);
  } else {
    ep->n_scales = (p->t_out == ITEXHIP_QINT32) ? 0 : 1;
  }
  for (int e = 0; e < ep->n_eltwise; ++e) {
    if (ep->elt[e].alg == ITEXHIP_ELT_SUM) continue;
    if (has_leaky) ep->elt[e].alpha = p->leakyrelu_alpha;
    if (has_linear) {
      ep->elt[e].alpha = linear_alpha;
      ep->elt[e].beta = linear_beta;
    }
  }
  // GetScaledBias indexes the output scales for an 8-bit output; without any the reference reads
  // out of bounds, so refuse.
  ITEXHIP_REQUIRE(!(out_q8 && p->input_mode == ITEXHIP_MIN_FIRST && ep->n_scales == 0),
                  "qmatmul: 8-bit output with MIN_FIRST input needs Requantize in fused_ops");
  return ITEXHIP_OK;
}

extern "C" int itexhip_qmatmul_prepare(const itexhip_matmul_params* p, const float* min_b,
                                       const float* max_b, int64_t nb, const void* bias,
                                       const int32_t* colsum, int64_t N, float* scales_out,
                                       float* bias_out, void* stream) {
  itexhip_epilogue ep;
  if (int st = itexhip_qmatmul_epilogue_desc(p, nb, &ep)) return st;
  ITEXHIP_REQUIRE(N >= 0, "qmatmul_prepare: negative N");
  ITEXHIP_REQUIRE(nb == 1 || nb == N, "qmatmul_prepare: %lld weight ranges for %lld channels",
                  static_cast<long long>(nb), static_cast<long long>(N));
  if (N == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(min_b && max_b && bias_out, "qmatmul_prepare: null buffer");
  ITEXHIP_REQUIRE(ep.n_scales == 0 || scales_out, "qmatmul_prepare: null scales_out");
  ITEXHIP_REQUIRE(p->input_mode != ITEXHIP_MIN_FIRST || colsum, "qmatmul_prepare: MIN_FIRST needs colsum");

  const PrepArgs a = make_prep_args(p, ep);
  const unsigned grid = static_cast<unsigned>((N + 255) / 256);
  qmatmul_prepare_kernel<<<grid, 256, 0, as_stream(stream)>>>(a, min_b, max_b, nb, bias, colsum, N,
                                                              scales_out, bias_out);
  ITEXHIP_CHECK_LAUNCH("itexhip_qmatmul_prepare");
  return ITEXHIP_OK;
}
