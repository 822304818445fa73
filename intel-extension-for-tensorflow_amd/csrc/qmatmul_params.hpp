// Per-channel epilogue parameters of the quantized MatMul ops, shared by the parameter kernel and by
// the MatMul kernels that derive them on the fly (one launch for the whole op).
//
// Follows, operation by operation and in fp32:
//   ExtendInt8PostOps  itex/core/kernels/common/quantized_matmul_common.h:1472-1508 (legacy),
//                      :1610-1702 (V1), :1809-1908 (V2)
//   GetScaledBias      quantized_matmul_common.h:466-660 (fp32 bias)
#ifndef ITEXHIP_QMATMUL_PARAMS_HPP_
#define ITEXHIP_QMATMUL_PARAMS_HPP_

#include "common.hpp"

namespace itexhip {

struct PrepArgs {
  int api, t_in, t_out, input_mode;
  int n_scales;        // from the epilogue descriptor
  int mul_requant;     // multiply the output scale by (max_int8_output / range_output)
  int legacy_kind;     // 1: u8 out, 2: s8 out, 3: fp32 out (legacy api only)
  int bias_s32;        // Tbias = qint32: the bias vector holds int32 (quantized_matmul_common.h:1153-1334)
  int bias_16;         // Tbias = bfloat16 / half (the type, else 0): widened to fp32, the fp32 arithmetic, and the
                       // adjusted bias rounded to Tbias again, as the generic-in-Tbias code stores it (:578-599, 609-617)
  float min_a, max_a, min_out, max_out;
};

// entry j of the op's bias vector: the raw bits first (a load that nothing waits for), the fp32 value later
// (the qint32 bias is cast, :1165-1167); 0 without a bias
__device__ __forceinline__ uint32_t bias_bits(const PrepArgs& p, const void* bias, int64_t j) {
  if (bias == nullptr) return 0u;
  if (p.bias_s32) return static_cast<uint32_t>(static_cast<const int32_t*>(bias)[j]);
  if (p.bias_16 != 0) return static_cast<const uint16_t*>(bias)[j];
  return static_cast<const uint32_t*>(bias)[j];
}
__device__ __forceinline__ float bias_from_bits(const PrepArgs& p, uint32_t b) {
  if (p.bias_s32) return static_cast<float>(static_cast<int32_t>(b));
  if (p.bias_16 == ITEXHIP_BFLOAT16) return bf16_bits_to_f32(b);
  if (p.bias_16 == ITEXHIP_HALF) return f16_bits_to_f32(b);
  return __uint_as_float(b);
}
__device__ __forceinline__ float bias_entry(const PrepArgs& p, const void* bias, int64_t j) {
  return bias_from_bits(p, bias_bits(p, bias, j));
}

struct ChannelScaleBias {
  float scale;  // output scale of the channel (the single scale when the node has one; 1 when none)
  float bias;   // scaled / zero-point-compensated bias
};

__device__ __forceinline__ float absmax(float a, float b) { return fmaxf(fabsf(a), fabsf(b)); }

// Value form: the weight range of the channel (min_bj, max_bj), the first weight range (min_b0, max_b0;
// the legacy ops and the SCALED-input bias use it for every channel), the channel's raw bias and
// weight column sum.
__device__ __forceinline__ ChannelScaleBias channel_scale_bias(const PrepArgs& p, float min_bj, float max_bj,
                                                               float min_b0, float max_b0, float b, int colsum_j) {
  const float max_int8_input = (p.t_in == ITEXHIP_QUINT8) ? 255.0f : 127.0f;
  const float max_int8_weight = 127.0f;
  const float max_int8_output = (p.t_out == ITEXHIP_QUINT8) ? 255.0f : 127.0f;
  const float range_input =
      (p.input_mode == ITEXHIP_MIN_FIRST) ? p.max_a - p.min_a : absmax(p.min_a, p.max_a);
  const float range_weight = absmax(min_bj, max_bj);

  // ---- output scale of the channel (or the single per-tensor scale) ----------------------------
  float os = 1.0f;
  if (p.api == ITEXHIP_API_LEGACY) {
    if (p.legacy_kind != 0) {
      const float a_level = (p.max_a - p.min_a) / 255.0f;
      const float b_level = (max_b0 - min_b0) / 254.0f;
      const float c_level = a_level * b_level;
      const float scale_int32 = absmax(c_level * -2147483648.0f, c_level * 2147483648.0f);
      const float scale_eightbit = absmax(p.min_out, p.max_out);
      if (p.legacy_kind == 1) os = scale_int32 / scale_eightbit / 8388608.0f;
      else if (p.legacy_kind == 2) os = scale_int32 / scale_eightbit / 16777216.0f;
      else os = scale_int32 / 2147483648.0f;
    }
  } else if (p.api == ITEXHIP_API_V1 && p.t_out == ITEXHIP_QINT32) {
    os = 1.0f;
  } else if (p.n_scales > 0) {
    os = (range_input * range_weight) / (max_int8_input * max_int8_weight);
    if (p.mul_requant) {
      const float range_output = absmax(p.min_out, p.max_out);
      os = os * (max_int8_output / range_output);
    }
  }

  // ---- bias -----------------------------------------------------------------------------------
  if (p.bias_s32) {
    // qint32 bias: scaled by the inverse of the fp32 path's factor, no zero-point compensation (:1204-1271)
    const float sj = (range_input * range_weight) / (max_int8_input * max_int8_weight);
    float out;
    if (p.input_mode != ITEXHIP_MIN_FIRST || is_float_out(p.t_out)) out = b * sj;
    else if (p.t_out == ITEXHIP_QINT8 || p.t_out == ITEXHIP_QUINT8) out = b * os;
    else out = b;
    return ChannelScaleBias{os, out};
  }
  const float bias_scale = (max_int8_input * max_int8_weight) / (range_input * range_weight);
  float out;
  if (p.input_mode == ITEXHIP_MIN_FIRST) {
    const float q_min_input = max_int8_input * p.min_a / range_input;
    const float sum = static_cast<float>(colsum_j);
    if (is_float_out(p.t_out)) {
      out = b + (sum * q_min_input / bias_scale);
    } else if (p.t_out == ITEXHIP_QINT8 || p.t_out == ITEXHIP_QUINT8) {
      // os is this channel's output scale, or the single scale when n_scales == 1
      out = b * bias_scale * os + (sum * q_min_input * os);
    } else {
      out = b * bias_scale + (sum * q_min_input);
    }
  } else {
    // SCALED input: the bias is scaled by the FIRST weight's bias scale for every channel
    const float bs0 = (max_int8_input * max_int8_weight) / (range_input * absmax(min_b0, max_b0));
    out = b * bs0;
  }
  if (p.bias_16 == ITEXHIP_BFLOAT16) out = bf16_bits_to_f32(f32_to_bf16_bits(out));
  if (p.bias_16 == ITEXHIP_HALF) out = f16_bits_to_f32(f32_to_f16_bits(out));
  return ChannelScaleBias{os, out};
}

// Pointer form: channel j of N; nb = number of weight ranges (1 or N); colsum is only read for
// MIN_FIRST input.
__device__ __forceinline__ ChannelScaleBias channel_scale_bias(const PrepArgs& p, const float* __restrict__ min_b,
                                                               const float* __restrict__ max_b, int64_t nb,
                                                               const void* __restrict__ bias,
                                                               const int32_t* __restrict__ colsum, int64_t N,
                                                               int64_t j) {
  const int64_t jb = (nb == N) ? j : 0;
  return channel_scale_bias(p, min_b[jb], max_b[jb], min_b[0], max_b[0], bias_entry(p, bias, j),
                            p.input_mode == ITEXHIP_MIN_FIRST ? colsum[j] : 0);
}

// host: fills PrepArgs from the op parameters and its epilogue descriptor
inline PrepArgs make_prep_args(const itexhip_matmul_params* p, const itexhip_epilogue& ep) {
  PrepArgs a{};
  a.api = p->api; a.t_in = p->t_in; a.t_out = p->t_out; a.input_mode = p->input_mode;
  a.n_scales = ep.n_scales;
  a.bias_s32 = p->t_bias == ITEXHIP_QINT32;
  a.bias_16 = is_float16_type(p->t_bias) ? p->t_bias : 0;
  a.min_a = p->min_a; a.max_a = p->max_a; a.min_out = p->min_out; a.max_out = p->max_out;
  const bool out_q8 = p->t_out == ITEXHIP_QINT8 || p->t_out == ITEXHIP_QUINT8;
  if (p->api == ITEXHIP_API_V2) {
    // requantize factor folded into the output scale only without any eltwise post-op
    int n_act = 0;
    for (int k = 0; k < ep.n_eltwise; ++k) n_act += ep.elt[k].alg != ITEXHIP_ELT_SUM;
    a.mul_requant = p->has_requantize && n_act == 0;
  } else if (p->api == ITEXHIP_API_V1) {
    a.mul_requant = out_q8 && p->n_fused_ops == 1;
  } else {
    a.legacy_kind = p->t_out == ITEXHIP_QUINT8 ? 1 : p->t_out == ITEXHIP_QINT8 ? 2
                    : is_float_out(p->t_out) ? 3 : 0;
  }
  return a;
}

}  // namespace itexhip
#endif  // ITEXHIP_QMATMUL_PARAMS_HPP_
