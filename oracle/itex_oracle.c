/*
 * CPU oracle (test infrastructure; see itex_oracle.h for the full header comment, the list of
 * parity pins and of the parts whose parity is unpinned).
 *
 * Build with contraction off: every fp32 operation below must round on its own
 * (gcc -O2 -ffp-contract=off -fno-fast-math).
 */
#include "itex_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* Eigen::NumTraits<T>::highest() / lowest() for the quantized types
 * (used at itex/core/utils/quantization_util.h:58-59). */
static int64_t q_highest(int T) {
  switch (T) {
    case ORC_QINT8: return 127;
    case ORC_QUINT8: return 255;
    case ORC_QINT32: return 2147483647LL;
    default: return 0;
  }
}
static int64_t q_lowest(int T) {
  switch (T) {
    case ORC_QINT8: return -128;
    case ORC_QUINT8: return 0;
    case ORC_QINT32: return -2147483648LL;
    default: return 0;
  }
}

/* oneDNN destination conversion: clamp in fp32 to the destination range, then convert with
 * round-to-nearest-even.  NaN maps to the lower bound here (parity unpinned). */
static inline float sat_rne(float y, float lo, float hi) {
  y = fmaxf(y, lo);
  y = fminf(y, hi);
  return rintf(y);
}
static inline void sat_bounds(int T, float* lo, float* hi) {
  if (T == ORC_QINT8) { *lo = -128.0f; *hi = 127.0f; }
  else if (T == ORC_QUINT8) { *lo = 0.0f; *hi = 255.0f; }
  else { *lo = -2147483648.0f; *hi = 2147483520.0f; } /* largest fp32 below 2^31 */
}
static inline void store_q(void* q, int64_t i, int T, float r) {
  if (T == ORC_QINT8) ((int8_t*)q)[i] = (int8_t)(int32_t)r;
  else if (T == ORC_QUINT8) ((uint8_t*)q)[i] = (uint8_t)(int32_t)r;
  else ((int32_t*)q)[i] = (int32_t)r;
}

/* QuantizeV2Op::AdjustInputMinMaxRange, itex/core/kernels/common/quantize_op.h:130-152 */
int orc_adjust_input_range(float in_min, float in_max, float ensure_minimum_range, float* adj_min,
                           float* adj_max) {
  if (!(in_max >= in_min)) return ORC_INVALID_ARGUMENT; /* :133-135 */
  *adj_min = fminf(0.0f, in_min);                        /* :137 */
  const float epsilon = fmaxf(1.0f, fmaxf(fabsf(in_min), fabsf(in_max))) * ensure_minimum_range;
  *adj_max = fmaxf(0.0f, fmaxf(in_max, *adj_min + epsilon)); /* :150-151 */
  return ORC_OK;
}

/* GetScaleAndZeropointAndAlignMinMax<T>, itex/core/utils/quantization_util.h:54-84.
 * int64 operands are converted to float before the fp32 division / subtraction, exactly as the
 * usual arithmetic conversions do in the reference expression. */
int orc_scale_zeropoint_align(int T, int mode, int dequantize, float* min_data, float* max_data,
                              int length, float* scales, int32_t* zero_points) {
  const float max_int = (float)q_highest(T);
  const float span = (float)(q_highest(T) - q_lowest(T));
  if (mode == ORC_SCALED) {
    for (int i = 0; i < length; ++i) {
      float abs_range = fmaxf(fabsf(min_data[i]), fabsf(max_data[i]));
      max_data[i] = abs_range;
      min_data[i] = -abs_range;
      scales[i] = dequantize ? (abs_range / max_int) : (max_int / abs_range);
      zero_points[i] = 0;
    }
  } else if (mode == ORC_MIN_FIRST) {
    for (int i = 0; i < length; ++i) {
      scales[i] = dequantize ? ((max_data[i] - min_data[i]) / span)
                             : (span / (max_data[i] - min_data[i]));
      /* std::round: half away from zero */
      zero_points[i] = dequantize ? (int32_t)roundf(max_int - max_data[i] / scales[i])
                                  : (int32_t)roundf(max_int - max_data[i] * scales[i]);
    }
  } else {
    return ORC_INVALID_ARGUMENT;
  }
  return ORC_OK;
}

/* Legacy MIN_FIRST scale, quantize_op.h:204-214: (number_of_steps - 1.0) is a double, so the
 * division is carried out in double and rounded once to float on assignment. */
float orc_legacy_min_first_scale(int T, float adj_min, float adj_max) {
  const int number_of_bits = (T == ORC_QINT32) ? 32 : 8;
  const int64_t number_of_steps = (int64_t)1 << number_of_bits;
  return (float)(((double)number_of_steps - 1.0) / (double)(adj_max - adj_min));
}

/* QuantizeV2Op::Compute, quantize_op.h:154-408.  The tensor is viewed as [outer, slices, inner]
 * with `slices` the size of `axis` (1 for per-tensor). */
int orc_quantize_v2(const float* x, int64_t outer, int64_t slices, int64_t inner, int T, int mode,
                    int classic_asymmetric, float ensure_minimum_range, const float* in_min,
                    const float* in_max, void* q, float* out_min, float* out_max) {
  if (T != ORC_QINT8 && T != ORC_QUINT8) return ORC_INVALID_ARGUMENT;
  if (mode != ORC_SCALED && mode != ORC_MIN_FIRST) return ORC_INVALID_ARGUMENT; /* :94-97 */
  float* mn = (float*)malloc(sizeof(float) * (size_t)slices);
  float* mx = (float*)malloc(sizeof(float) * (size_t)slices);
  float* scale = (float*)malloc(sizeof(float) * (size_t)slices);
  int32_t* zp = (int32_t*)malloc(sizeof(int32_t) * (size_t)slices);
  int st = ORC_OK;
  for (int64_t s = 0; s < slices && st == ORC_OK; ++s)
    st = orc_adjust_input_range(in_min[s], in_max[s], ensure_minimum_range, &mn[s], &mx[s]);
  if (st != ORC_OK) goto done;

  const int legacy = (mode == ORC_MIN_FIRST && !classic_asymmetric);
  if (!legacy) {
    orc_scale_zeropoint_align(T, mode, 0, mn, mx, (int)slices, scale, zp); /* :198-202 */
  } else {
    for (int64_t s = 0; s < slices; ++s) {
      scale[s] = orc_legacy_min_first_scale(T, mn[s], mx[s]);
      zp[s] = 0;
    }
  }
  float lo, hi;
  sat_bounds(T, &lo, &hi);
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t o = 0; o < outer; ++o) {
    for (int64_t s = 0; s < slices; ++s) {
      const float sc = scale[s];
      const int64_t base = (o * slices + s) * inner;
      if (mode == ORC_SCALED) {
        /* reorder with a source scale (:256-275): q = sat(rne(x * scale)) */
        for (int64_t i = 0; i < inner; ++i) store_q(q, base + i, T, sat_rne(x[base + i] * sc, lo, hi));
      } else if (!legacy) {
        /* reorder with source scale and destination zero point (:276-291):
         * q = sat(rne(x * scale + zp)), the zero point is added in fp32 before the conversion */
        const float zpf = (float)zp[s];
        for (int64_t i = 0; i < inner; ++i)
          store_q(q, base + i, T, sat_rne(x[base + i] * sc + zpf, lo, hi));
      } else {
        /* binary_add of x and shift=-min', both sources scaled by `scale` (:292-314, 383-391):
         * three separately rounded fp32 operations */
        const float shift = -mn[s]; /* :244-245 */
        const float t1 = shift * sc;
        for (int64_t i = 0; i < inner; ++i) {
          const float t0 = x[base + i] * sc;
          store_q(q, base + i, T, sat_rne(t0 + t1, lo, hi));
        }
      }
    }
  }
  /* output ranges, :397-408 */
  for (int64_t s = 0; s < slices; ++s) {
    if (T == ORC_QUINT8 && mode == ORC_SCALED) { out_min[s] = 0.0f; out_max[s] = mx[s]; }
    else { out_min[s] = mn[s]; out_max[s] = mx[s]; }
  }
done:
  free(mn); free(mx); free(scale); free(zp);
  return st;
}

/* DequantizeOp::Compute, itex/core/kernels/common/dequantize_op.h:67-178: reorder with a source
 * scale and (MIN_FIRST) a source zero point: y = ((float)q - zp) * scale. */
int orc_dequantize(const void* q, int64_t outer, int64_t slices, int64_t inner, int T, int mode,
                   const float* in_min, const float* in_max, float* y) {
  if (T != ORC_QINT8 && T != ORC_QUINT8) return ORC_INVALID_ARGUMENT;
  if (mode != ORC_SCALED && mode != ORC_MIN_FIRST) return ORC_INVALID_ARGUMENT;
  float* mn = (float*)malloc(sizeof(float) * (size_t)slices);
  float* mx = (float*)malloc(sizeof(float) * (size_t)slices);
  float* scale = (float*)malloc(sizeof(float) * (size_t)slices);
  int32_t* zp = (int32_t*)malloc(sizeof(int32_t) * (size_t)slices);
  memcpy(mn, in_min, sizeof(float) * (size_t)slices);
  memcpy(mx, in_max, sizeof(float) * (size_t)slices);
  orc_scale_zeropoint_align(T, mode, 1, mn, mx, (int)slices, scale, zp); /* :101-103 */
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t o = 0; o < outer; ++o) {
    for (int64_t s = 0; s < slices; ++s) {
      const float sc = scale[s];
      const float zpf = (mode == ORC_MIN_FIRST) ? (float)zp[s] : 0.0f;
      const int64_t base = (o * slices + s) * inner;
      for (int64_t i = 0; i < inner; ++i) {
        const float v = (T == ORC_QINT8) ? (float)((const int8_t*)q)[base + i]
                                         : (float)((const uint8_t*)q)[base + i];
        y[base + i] = (v - zpf) * sc;
      }
    }
  }
  free(mn); free(mx); free(scale); free(zp);
  return ORC_OK;
}

/* OneDnnRequantizePerChannelOp::Compute,
 * itex/core/kernels/onednn/block/requantize_per_channel_op.cc:44-159.  Channel = last dimension. */
int orc_requantize_per_channel(const int32_t* x, int64_t rows, int64_t depth, const float* in_min,
                               const float* in_max, float req_min, float req_max, int out_type,
                               void* q, float* out_min, float* out_max) {
  if (out_type != ORC_QINT8 && out_type != ORC_QUINT8) return ORC_INVALID_ARGUMENT; /* :40-42 */
  const float factor = (out_type == ORC_QINT8) ? 127.0f : 255.0f;                     /* :82 */
  const float requested_min_max = fmaxf(fabsf(req_min), fabsf(req_max));              /* :83-85 */
  float* scales = (float*)malloc(sizeof(float) * (size_t)depth);
  for (int64_t i = 0; i < depth; ++i) {
    const float mm = fmaxf(fabsf(in_min[i]), fabsf(in_max[i]));
    scales[i] = factor * (mm / requested_min_max / 2147483648.0f); /* :91-95 */
  }
  float lo, hi;
  sat_bounds(out_type, &lo, &hi);
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < depth; ++c)
      store_q(q, r * depth + c, out_type, sat_rne((float)x[r * depth + c] * scales[c], lo, hi));
  *out_min = req_min; /* :149-150 */
  *out_max = req_max;
  free(scales);
  return ORC_OK;
}

/* OneDnnRequantizationRangePerChannelOp::Compute,
 * itex/core/kernels/onednn/block/requantization_range_per_channel_op.cc:41-159. */
int orc_requantization_range_per_channel(const int32_t* x, int64_t rows, int64_t depth,
                                         const float* in_min, const float* in_max,
                                         float clip_value_max, float* out_min, float* out_max) {
  float out_min_max = FLT_MIN; /* std::numeric_limits<float>::min(), :78 */
  int is_non_negative = 1;
  for (int64_t c = 0; c < depth; ++c) {
    int32_t mn = INT32_MAX, mx = INT32_MIN;
    for (int64_t r = 0; r < rows; ++r) {
      const int32_t v = x[r * depth + c];
      if (v < mn) mn = v;
      if (v > mx) mx = v;
    }
    /* std::abs(int32) wraps for INT32_MIN upstream (undefined behaviour; parity unpinned) */
    const int32_t amn = (mn == INT32_MIN) ? INT32_MIN : (mn < 0 ? -mn : mn);
    const int32_t amx = (mx == INT32_MIN) ? INT32_MIN : (mx < 0 ? -mx : mx);
    const int32_t abs_max = amn > amx ? amn : amx;                       /* :133-134 */
    const float scale = fmaxf(fabsf(in_min[c]), fabsf(in_max[c]));       /* :135-136 */
    const float range = scale * (float)abs_max / 2147483648.0f;          /* :137-138 */
    if (mn < 0) is_non_negative = 0;                                     /* :139 */
    out_min_max = fmaxf(out_min_max, range);                             /* :142 */
  }
  if (out_min_max > clip_value_max) out_min_max = clip_value_max;        /* :150 */
  *out_min = is_non_negative ? 0.0f : -out_min_max;                      /* :158-159 */
  *out_max = out_min_max;
  return ORC_OK;
}

/* Exact int32 accumulation of a[M,K] (u8 or s8, row-major) times w (s8; TF layout [K,N] row-major,
 * or [N,K] when transpose_b), quantized_matmul_common.h:183-226 (inner_product_forward). */
void orc_int_gemm(const void* a, int a_type, const int8_t* w, int transpose_b, int64_t M, int64_t K,
                  int64_t N, int32_t* acc) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    int32_t* row = acc + m * N;
    for (int64_t n = 0; n < N; ++n) row[n] = 0;
    if (!transpose_b) {
      for (int64_t k = 0; k < K; ++k) {
        const int32_t av = (a_type == ORC_QUINT8) ? (int32_t)((const uint8_t*)a)[m * K + k]
                                                  : (int32_t)((const int8_t*)a)[m * K + k];
        const int8_t* wr = w + k * N;
        for (int64_t n = 0; n < N; ++n) row[n] += av * (int32_t)wr[n];
      }
    } else {
      for (int64_t n = 0; n < N; ++n) {
        const int8_t* wr = w + n * K;
        int32_t s = 0;
        if (a_type == ORC_QUINT8) {
          const uint8_t* ar = (const uint8_t*)a + m * K;
          for (int64_t k = 0; k < K; ++k) s += (int32_t)ar[k] * (int32_t)wr[k];
        } else {
          const int8_t* ar = (const int8_t*)a + m * K;
          for (int64_t k = 0; k < K; ++k) s += (int32_t)ar[k] * (int32_t)wr[k];
        }
        row[n] = s;
      }
    }
  }
}

/* Column sums of the [K,N] weight, quantized_matmul_common.h:569-573. */
void orc_weight_colsum(const int8_t* w, int64_t K, int64_t N, int32_t* colsum) {
  for (int64_t j = 0; j < N; ++j) colsum[j] = 0;
  for (int64_t i = 0; i < K; ++i)
    for (int64_t j = 0; j < N; ++j) colsum[j] += (int32_t)w[i * N + j];
}

static int eltwise_from_activation(int act, orc_eltwise* e) {
  /* table at itex/core/utils/onednn/onednn_post_op_util.cc:34-68 */
  switch (act) {
    case ORC_ACT_RELU: e->alg = ORC_ELT_RELU; e->alpha = 0.0f; e->beta = 0.0f; return 1;
    case ORC_ACT_RELU6: e->alg = ORC_ELT_CLIP; e->alpha = 0.0f; e->beta = 6.0f; return 1;
    case ORC_ACT_LEAKYRELU: e->alg = ORC_ELT_RELU; e->alpha = 0.0f; e->beta = 0.0f; return 1;
    case ORC_ACT_GELU_APPROX: e->alg = ORC_ELT_GELU_TANH; e->alpha = 0.0f; e->beta = 0.0f; return 1;
    case ORC_ACT_GELU_EXACT: e->alg = ORC_ELT_GELU_ERF; e->alpha = 0.0f; e->beta = 0.0f; return 1;
    case ORC_ACT_ELU: e->alg = ORC_ELT_ELU; e->alpha = 1.0f; e->beta = 0.0f; return 1;          /* "Elu", kAlphaOne */
    case ORC_ACT_SIGMOID: e->alg = ORC_ELT_LOGISTIC; e->alpha = 1.0f; e->beta = 0.0f; return 1; /* "Sigmoid", kAlphaOne */
    case ORC_ACT_TANH: e->alg = ORC_ELT_TANH; e->alpha = 0.0f; e->beta = 0.0f; return 1;        /* "Tanh" */
    case ORC_ACT_SWISH: e->alg = ORC_ELT_SWISH; e->alpha = 1.0f; e->beta = 0.0f; return 1;      /* "_ITEXSwish", kAlphaOne */
    case ORC_ACT_MISH: e->alg = ORC_ELT_MISH; e->alpha = 0.0f; e->beta = 0.0f; return 1;        /* "_ITEXMish" */
    default: return 0;
  }
}

/* fp32 -> bfloat16, round to nearest even (the destination conversion of a bf16 memory descriptor and
 * the float -> Eigen::bfloat16 cast) */
static inline uint16_t f32_to_bf16_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* fp32 -> IEEE half, round to nearest even, overflow to infinity, denormals kept */
static inline uint16_t f32_to_f16_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);          /* NaN */
  if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);         /* >= 65520 rounds to infinity */
  if (a < 0x33000001u) return sign;                                /* <= 2^-25 rounds to zero */
  const int e = (int)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;                        /* 24-bit significand */
  int shift;                                                       /* bits dropped from m */
  uint32_t base;
  if (e < -14) { shift = 13 + (-14 - e); base = 0; }               /* half denormal: value = m * 2^(e-23) / 2^-24 */
  else { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7fffffu; }
  const uint32_t q = m >> shift, rem = m & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
  uint32_t r = base + q;
  if (rem > halfway || (rem == halfway && (r & 1u))) r += 1u;      /* carries into the exponent correctly */
  return (uint16_t)(sign | r);
}

static inline float f16_bits_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
  uint32_t u;
  if (e == 0x1fu) u = sign | 0x7f800000u | (m << 13);
  else if (e != 0) u = sign | ((e + 112u) << 23) | (m << 13);
  else if (m == 0) u = sign;
  else {
    float f = (float)m * 5.9604644775390625e-08f; /* m * 2^-24, exact */
    memcpy(&u, &f, 4);
    u |= sign;
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint16_t f32_to_bits16(int t, float f) { return t == ORC_HALF ? f32_to_f16_bits(f) : f32_to_bf16_bits(f); }
static inline float bits16_to_f32(int t, uint16_t h);

static inline float bf16_bits_to_f32(uint16_t h) {
  const uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline float bits16_to_f32(int t, uint16_t h) { return t == ORC_HALF ? f16_bits_to_f32(h) : bf16_bits_to_f32(h); }

/*
 * Host-side parameter preparation of the quantized MatMul kernels:
 *   output scales  - ExtendInt8PostOps: V2 quantized_matmul_common.h:1809-1908,
 *                    V1 :1610-1702, legacy :1472-1508 (+ :1526-1530 for the ReLU variant)
 *   scaled bias    - GetScaledBias (fp32 bias), :466-660
 *   post-op chain  - PostOpUtil::AddOps / SetPostOp, onednn_post_op_util.cc:73-128, 237-273
 * `scales` must hold max(nb,1) floats, `bias_out` N floats.  `colsum` (N int32, column sums of the
 * [K,N] weight) is only read for input_mode == MIN_FIRST.
 */
int orc_qmatmul_prepare(const orc_matmul_attrs* at, int64_t N, const int32_t* colsum, float min_a,
                        float max_a, const float* min_b, const float* max_b, int64_t nb,
                        float min_out, float max_out, const void* bias_v, float* scales,
                        float* bias_out, orc_epilogue_desc* ep) {
  const int bias_s32 = (at->t_bias == ORC_QINT32);
  /* Tbias = bfloat16: GetScaledBias is generic in Tbias; every entry is widened with
   * static_cast<float>, the arithmetic is fp32, and the result is stored as Tbias again (:578-599 cast,
   * :609-617 the reorder's bf16 destination), i.e. rounded to bfloat16 before the primitive reads it */
  const int bias_bf16 = (at->t_bias == ORC_BFLOAT16 || at->t_bias == ORC_HALF); /* either 16-bit float type */
  const int32_t* bias_i32 = (const int32_t*)bias_v;
  const int out_q8 = (at->t_out == ORC_QINT8 || at->t_out == ORC_QUINT8);
  /* the float-output branches upstream test Toutput against float, bfloat16 and half alike (:577, 1255-1257) */
  const int out_f32 = (at->t_out == ORC_FLOAT || at->t_out == ORC_BFLOAT16 || at->t_out == ORC_HALF);
  const int out_s32 = (at->t_out == ORC_QINT32);
  if (!out_q8 && !out_f32 && !out_s32) return ORC_INVALID_ARGUMENT;
  if (at->input_mode != ORC_MIN_FIRST && at->input_mode != ORC_SCALED) return ORC_INVALID_ARGUMENT;
  if (nb != 1 && nb != N) return ORC_INVALID_ARGUMENT;

  const float max_int8_input = (at->t_in == ORC_QUINT8) ? 255.0f : 127.0f;  /* :503-506 */
  const float max_int8_weight = 127.0f;
  const float range_input = (at->input_mode == ORC_MIN_FIRST)
                                ? max_a - min_a
                                : fmaxf(fabsf(min_a), fabsf(max_a));          /* :507-510 */
  const float max_int8_output = (at->t_out == ORC_QUINT8) ? 255.0f : 127.0f;

  memset(ep, 0, sizeof(*ep));

  /* ---- post-op chain -------------------------------------------------------------------- */
  int has_linear = 0, has_leaky = 0;
  float linear_alpha = 0.0f, linear_beta = 0.0f;
  /* post-ops are appended in fused_ops order (onednn_post_op_util.cc:73-128, 237-266); "Add" is a sum
   * post-op with scale 1 (:1694-1699, 1902-1906) and does not count as an activation */
  int n_act = 0;
  if (at->add_position == 1) {
    ep->elt[ep->n_eltwise].alg = ORC_ELT_SUM; ep->elt[ep->n_eltwise].alpha = 1.0f; ep->elt[ep->n_eltwise].beta = 0.0f;
    ep->n_eltwise++;
  }
  if (eltwise_from_activation(at->activation, &ep->elt[ep->n_eltwise])) { ep->n_eltwise++; n_act++; }
  if (at->add_position == 2) {
    ep->elt[ep->n_eltwise].alg = ORC_ELT_SUM; ep->elt[ep->n_eltwise].alpha = 1.0f; ep->elt[ep->n_eltwise].beta = 0.0f;
    ep->n_eltwise++;
  }
  /* a quantized addend is not implemented upstream either (:1768-1773).  The addend has the output's type (the sum
   * post-op reads the destination buffer, :341-389); for a bfloat16 / half result the caller passes its values widened
   * to float, which is exact, and the sum is formed in fp32 before the result is rounded to the 16-bit type. */
  if (at->add_position != 0 && at->t_out != ORC_FLOAT && at->t_out != ORC_BFLOAT16 && at->t_out != ORC_HALF)
    return ORC_UNIMPLEMENTED;
  if (at->activation == ORC_ACT_LEAKYRELU) has_leaky = 1;
  if (at->api == ORC_API_V2 && at->has_requantize && at->out_min_first) {
    /* :1753-1757: "Linear" is appended to fused_ops */
    ep->elt[ep->n_eltwise].alg = ORC_ELT_LINEAR;
    ep->elt[ep->n_eltwise].alpha = 1.0f;
    ep->elt[ep->n_eltwise].beta = 0.0f;
    ep->n_eltwise++;
    n_act++;
    has_linear = 1;
  }
  const int has_activation = n_act > 0; /* has_activation_ is set by every eltwise post-op */

  /* ---- output scales ---------------------------------------------------------------------- */
  if (at->api == ORC_API_V2) {
    const int has_output_scales = at->has_requantize || at->has_dequantize;
    if (has_output_scales) { /* :1815-1865 */
      for (int64_t i = 0; i < nb; ++i) {
        const float range_weight = fmaxf(fabsf(min_b[i]), fabsf(max_b[i]));
        scales[i] = (range_input * range_weight) / (max_int8_input * max_int8_weight);
      }
      if (at->has_requantize && !has_activation && !has_linear) {
        const float range_output = fmaxf(fabsf(min_out), fabsf(max_out));
        for (int64_t i = 0; i < nb; ++i) scales[i] = scales[i] * (max_int8_output / range_output);
      }
      ep->n_scales = (int)nb;
    }
    /* :1867-1885: the activation's post-op scale is stored but never reaches oneDNN
     * (onednn_post_op_util.cc:248-263 appends eltwise(alg, alpha, beta) only) */
    if (has_linear) { /* :1887-1900 */
      const float range_output = max_out - min_out;
      linear_alpha = max_int8_output / range_output;
      linear_beta = -min_out * max_int8_output / range_output;
    }
  } else if (at->api == ORC_API_V1) {
    if (out_s32) { /* :1611-1614 */
      scales[0] = 1.0f;
      ep->n_scales = 1;
    } else { /* :1615-1701 */
      for (int64_t i = 0; i < nb; ++i) {
        const float range_weight = fmaxf(fabsf(min_b[i]), fabsf(max_b[i]));
        scales[i] = (range_input * range_weight) / (max_int8_input * max_int8_weight);
      }
      if (out_q8) {
        const float range_output = fmaxf(fabsf(min_out), fabsf(max_out));
        if (at->n_fused_ops == 1) {
          const float f = (at->t_out == ORC_QINT8) ? 127.0f : 255.0f;
          for (int64_t i = 0; i < nb; ++i) scales[i] = scales[i] * (f / range_output);
        } /* else: folded into the activation's post-op scale, which is dropped */
      }
      ep->n_scales = (int)nb;
    }
  } else if (at->api == ORC_API_LEGACY) { /* :1472-1508, per-tensor weights only */
    if (!out_s32) {
      /* ComputeOutputRangeForInt32 (:409-421) with <quint8, qint8, qint32> */
      const float a_level = (max_a - min_a) / 255.0f;
      const float b_level = (max_b[0] - min_b[0]) / 254.0f;
      const float c_level = a_level * b_level;
      const float min_o = c_level * -2147483648.0f;
      const float max_o = c_level * 2147483648.0f; /* (float)INT32_MAX */
      const float scale_int32 = fmaxf(fabsf(min_o), fabsf(max_o));
      const float scale_eightbit = fmaxf(fabsf(min_out), fabsf(max_out));
      float scale;
      if (at->t_out == ORC_QUINT8) scale = scale_int32 / scale_eightbit / 8388608.0f;
      else if (at->t_out == ORC_QINT8) scale = scale_int32 / scale_eightbit / 16777216.0f;
      else scale = scale_int32 / 2147483648.0f; /* float / bfloat16 output */
      scales[0] = scale;
      ep->n_scales = 1;
    }
  } else {
    return ORC_INVALID_ARGUMENT;
  }

  /* alpha / beta overrides applied to EVERY eltwise of the chain, onednn_post_op_util.cc:251-262 */
  for (int e = 0; e < ep->n_eltwise; ++e) {
    if (ep->elt[e].alg == ORC_ELT_SUM) continue;
    if (has_leaky) ep->elt[e].alpha = at->leakyrelu_alpha;
    if (has_linear) { ep->elt[e].alpha = linear_alpha; ep->elt[e].beta = linear_beta; }
  }

  /* ---- scaled bias, GetScaledBias :466-660 ------------------------------------------------ */
  /* bias_scales, :511-519 */
  float* bias_scales = (float*)malloc(sizeof(float) * (size_t)nb);
  for (int64_t i = 0; i < nb; ++i) {
    const float range_weight = fmaxf(fabsf(min_b[i]), fabsf(max_b[i]));
    bias_scales[i] = (max_int8_input * max_int8_weight) / (range_input * range_weight);
  }
  int st = ORC_OK;
  float* bias_wide = NULL;
  if (bias_bf16) {
    bias_wide = (float*)malloc(sizeof(float) * (size_t)(N > 0 ? N : 1));
    for (int64_t j = 0; j < N; ++j) bias_wide[j] = bits16_to_f32(at->t_bias, ((const uint16_t*)bias_v)[j]);
  }
  const float* bias = bias_bf16 ? bias_wide : (const float*)bias_v;
  if (bias_s32) {
    /* Tbias = qint32, :1153-1334: the bias is cast to float (:1165-1167) and scaled by
     * (range_input * range_weight) / (A * 127) (:1204-1211), the inverse of the fp32 path's factor;
     * no zero-point compensation (the column-sum loop is commented out, :1250-1253) */
    for (int64_t j = 0; j < N; ++j) {
      const int64_t jb = (nb != N) ? 0 : j;
      const float range_weight = fmaxf(fabsf(min_b[jb]), fabsf(max_b[jb]));
      const float sj = (range_input * range_weight) / (max_int8_input * max_int8_weight);
      const float bf = (float)bias_i32[j];
      if (at->input_mode == ORC_MIN_FIRST) { /* :1254-1271 */
        if (out_f32) bias_out[j] = bf * sj;
        else if (out_q8) {
          if (ep->n_scales == 0) { st = ORC_INVALID_ARGUMENT; break; }
          bias_out[j] = bf * ((ep->n_scales == 1) ? scales[0] : scales[j]);
        } else bias_out[j] = bf;
      } else { /* :1273-1305: reorder of the 1-D bias with per-entry source scales */
        bias_out[j] = bf * sj;
      }
    }
    free(bias_scales);
    return st;
  }
  if (at->input_mode == ORC_MIN_FIRST) { /* :520-601 */
    const float q_min_input = max_int8_input * min_a / range_input; /* :557 */
    for (int64_t j = 0; j < N; ++j) {
      const float sj = (nb != N) ? bias_scales[0] : bias_scales[j]; /* :561-565 */
      const float sum = (float)colsum[j];                            /* int * float */
      if (out_f32) {
        bias_out[j] = bias[j] + (sum * q_min_input / sj);            /* :578-580 */
      } else if (out_q8) {
        if (ep->n_scales == 0) { st = ORC_INVALID_ARGUMENT; break; } /* out-of-bounds upstream */
        const float os = (ep->n_scales == 1) ? scales[0] : scales[j];
        bias_out[j] = bias[j] * sj * os + (sum * q_min_input * os);  /* :583-595 */
      } else {
        bias_out[j] = bias[j] * sj + (sum * q_min_input);            /* :597-599 */
      }
    }
  } else { /* :602-634: reorder of a {1,N} bias with source scales */
    /* mask 0 for one weight scale; mask 1 otherwise, which selects dimension 0 of extent 1, so a
     * single scale (the first) applies to all N entries.  Parity unpinned for nb > 1. */
    for (int64_t j = 0; j < N; ++j) bias_out[j] = bias[j] * bias_scales[0];
  }
  if (bias_bf16) {
    for (int64_t j = 0; j < N; ++j) bias_out[j] = bits16_to_f32(at->t_bias, f32_to_bits16(at->t_bias, bias_out[j]));
    free(bias_wide);
  }
  free(bias_scales);
  return st;
}

static inline float apply_eltwise(const orc_eltwise* e, float x) {
  switch (e->alg) {
    case ORC_ELT_RELU:  /* eltwise_relu: x > 0 ? x : x * alpha; alpha == 0 is max(x, 0) */
      if (e->alpha == 0.0f) return fmaxf(x, 0.0f);
      return x > 0.0f ? x : x * e->alpha;
    case ORC_ELT_CLIP:  /* eltwise_clip_v2(alpha = low, beta = high) */
      return fminf(fmaxf(x, e->alpha), e->beta);
    case ORC_ELT_LINEAR: /* alpha * x + beta */
      return e->alpha * x + e->beta;
    case ORC_ELT_GELU_TANH: { /* eltwise_gelu_tanh: 0.5 x (1 + tanh(sqrt(2/pi) x (1 + 0.044715 x^2))) */
      const float v = tanhf(0.79788458347320556640625f * x * (1.0f + 0.044715f * x * x));
      return 0.5f * x * (1.0f + v);
    }
    case ORC_ELT_GELU_ERF: /* eltwise_gelu_erf: 0.5 x (1 + erf(x / sqrt(2))) */
      return 0.5f * x * (1.0f + erff(x * 0.707106769084930419921875f));
    /* oneDNN's reference forms of the other transcendental post-ops, in fp32 with libm (its own kernels evaluate
     * them with polynomial approximations: parity unpinned at the last bits, as for the GELUs) */
    case ORC_ELT_ELU: return x > 0.0f ? x : e->alpha * expm1f(x);
    case ORC_ELT_LOGISTIC: return 1.0f / (1.0f + expf(-x));
    case ORC_ELT_TANH: return tanhf(x);
    case ORC_ELT_SWISH: return x / (1.0f + expf(-e->alpha * x));
    case ORC_ELT_MISH: return x * tanhf(log1pf(expf(x)));
    default: return x;
  }
}

/* oneDNN int8 inner-product epilogue (execute at quantized_matmul_common.h:92):
 * y = fl(fl((float)acc * scale[n]) + bias[n]) -> eltwise chain -> destination conversion. */
void orc_qmatmul_epilogue(const int32_t* acc, int64_t M, int64_t N, const orc_epilogue_desc* ep,
                          const float* scales, const float* bias, const float* addend, int t_out,
                          void* out) {
  float lo = 0, hi = 0;
  if (t_out != ORC_FLOAT && t_out != ORC_BFLOAT16 && t_out != ORC_HALF) sat_bounds(t_out, &lo, &hi);
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      float y = (float)acc[m * N + n];
      if (ep->n_scales == 1) y = y * scales[0];
      else if (ep->n_scales > 1) y = y * scales[n];
      y = y + bias[n];
      for (int e = 0; e < ep->n_eltwise; ++e) {
        if (ep->elt[e].alg == ORC_ELT_SUM) y = y + ep->elt[e].alpha * addend[m * N + n]; /* dst = v + scale * dst */
        else y = apply_eltwise(&ep->elt[e], y);
      }
      if (t_out == ORC_FLOAT) ((float*)out)[m * N + n] = y;
      else if (t_out == ORC_BFLOAT16 || t_out == ORC_HALF) ((uint16_t*)out)[m * N + n] = f32_to_bits16(t_out, y);
      else store_q(out, m * N + n, t_out, sat_rne(y, lo, hi));
    }
  }
}

/* OneDnnFloatForOneQuantizedLevel<T>, itex/core/kernels/onednn/block/quantized_ops.h:24-38 */
static float float_for_one_level(int T, float range_min, float range_max) {
  int64_t highest = q_highest(T), lowest = q_lowest(T);
  if (lowest < -highest) ++lowest;
  return (range_max - range_min) / (float)(highest - lowest);
}

/* AllocateNativeOutputMinMax, quantized_ops.h:142-203 (+ :40-83 for the qint32 ranges).
 * n_out receives the number of entries written (0 for fp32 output, which has no min/max). */
int orc_qmatmul_output_minmax(const orc_matmul_attrs* at, float min_a, float max_a,
                              const float* min_b, const float* max_b, int64_t nb, int b_rank,
                              float min_out, float max_out, float* out_min, float* out_max,
                              int64_t* n_out) {
  if (at->t_out == ORC_QINT8 || at->t_out == ORC_QUINT8) {
    out_min[0] = min_out;
    out_max[0] = max_out;
    *n_out = 1;
  } else if (at->t_out == ORC_QINT32) {
    const int64_t cnt = (b_rank == 0) ? 1 : nb;
    for (int64_t n = 0; n < cnt; ++n) {
      const float a_level = float_for_one_level(at->t_in, min_a, max_a);
      const float b_level = float_for_one_level(ORC_QINT8, min_b[n], max_b[n]);
      const float c_level = a_level * b_level;
      out_min[n] = c_level * (float)q_lowest(ORC_QINT32);
      out_max[n] = c_level * (float)q_highest(ORC_QINT32);
    }
    *n_out = cnt;
  } else if (at->t_out == ORC_FLOAT || at->t_out == ORC_BFLOAT16 || at->t_out == ORC_HALF) {
    *n_out = 0;
  } else {
    return ORC_INVALID_ARGUMENT;
  }
  return ORC_OK;
}

/* LegacyQuantizedMatMulOpBase::Compute, quantized_matmul_common.h:61-102 — whole op. */
int orc_qmatmul(const orc_matmul_attrs* at, const void* a, const int8_t* w, int transpose_b,
                int64_t M, int64_t K, int64_t N, const void* bias, const float* addend, float min_a,
                float max_a, const float* min_b, const float* max_b, int64_t nb, float min_out,
                float max_out, void* out) {
  if (at->add_position != 0 && addend == NULL) return ORC_INVALID_ARGUMENT;
  /* the compensation loop indexes the weight as [K,N] regardless of transpose_b (:569-573) */
  if (transpose_b && at->input_mode == ORC_MIN_FIRST) return ORC_UNIMPLEMENTED;
  int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)(M * N));
  int32_t* colsum = (int32_t*)malloc(sizeof(int32_t) * (size_t)N);
  float* scales = (float*)malloc(sizeof(float) * (size_t)(nb > 0 ? nb : 1));
  float* sb = (float*)malloc(sizeof(float) * (size_t)N);
  orc_epilogue_desc ep;
  if (!transpose_b) orc_weight_colsum(w, K, N, colsum);
  else memset(colsum, 0, sizeof(int32_t) * (size_t)N);
  int st = orc_qmatmul_prepare(at, N, colsum, min_a, max_a, min_b, max_b, nb, min_out, max_out,
                               bias, scales, sb, &ep);
  if (st == ORC_OK) {
    orc_int_gemm(a, at->t_in, w, transpose_b, M, K, N, acc);
    orc_qmatmul_epilogue(acc, M, N, &ep, scales, sb, addend, at->t_out, out);
  }
  free(acc); free(colsum); free(scales); free(sb);
  return st;
}


/* ---- quantized BatchMatMul ---------------------------------------------------------------------- */
int orc_qbatch_matmul(const int8_t* x, int x_rank, const int64_t* x_dims, const int8_t* y, int y_rank,
                      const int64_t* y_dims, int adj_x, int adj_y, float min_x, float max_x,
                      float min_y, float max_y, int n_binary, const orc_bmm_binary* bin, int t_out,
                      void* out, int out_rank, const int64_t* out_dims) {
  if (x_rank < 2 || y_rank < 2 || x_rank > 8 || y_rank > 8) return ORC_INVALID_ARGUMENT;
  if (t_out != ORC_FLOAT && t_out != ORC_BFLOAT16 && t_out != ORC_HALF) return ORC_INVALID_ARGUMENT;
  if (n_binary < 0 || n_binary > 2) return ORC_UNIMPLEMENTED; /* kMaxBinaryNum_, :434 */
  /* matrix dimensions, :111-125 */
  int64_t d0 = x_dims[x_rank - 2], d1 = x_dims[x_rank - 1];
  int64_t d2 = y_dims[y_rank - 2], d3 = y_dims[y_rank - 1];
  if (adj_x) { int64_t t = d0; d0 = d1; d1 = t; }
  if (adj_y) { int64_t t = d2; d2 = d3; d3 = t; }
  if (d1 != d2) return ORC_INVALID_ARGUMENT;
  const int64_t M = d0, K = d1, N = d3;
  /* batch broadcast (MatMulBCast, :105-109): right-aligned, equal or 1 */
  const int nbx = x_rank - 2, nby = y_rank - 2, nbo = nbx > nby ? nbx : nby;
  if (out_rank != nbo + 2 || out_dims[nbo] != M || out_dims[nbo + 1] != N) return ORC_INVALID_ARGUMENT;
  int64_t xs[8] = {0}, ys[8] = {0}; /* element strides of the batch dims in x / y, 0 = broadcast */
  {
    int64_t sx = d0 * d1, sy = d2 * d3;
    for (int i = nbo - 1; i >= 0; --i) {
      const int ix = i - (nbo - nbx), iy = i - (nbo - nby);
      const int64_t dx = ix >= 0 ? x_dims[ix] : 1, dy = iy >= 0 ? y_dims[iy] : 1;
      if (dx != dy && dx != 1 && dy != 1) return ORC_INVALID_ARGUMENT;
      if (out_dims[i] != (dx == 1 ? dy : dx)) return ORC_INVALID_ARGUMENT;
      xs[i] = dx == 1 ? 0 : sx;
      ys[i] = dy == 1 ? 0 : sy;
      sx *= dx; sy *= dy;
    }
  }
  /* binary operands: strides per output dimension */
  int64_t bs[2][8] = {{0}};
  for (int b = 0; b < n_binary; ++b) {
    if (bin[b].alg != ORC_BIN_MUL && bin[b].alg != ORC_BIN_ADD) return ORC_UNIMPLEMENTED;
    if (bin[b].rank == 0) continue; /* one element */
    if (bin[b].rank != out_rank) return ORC_INVALID_ARGUMENT;
    int64_t st = 1;
    for (int i = out_rank - 1; i >= 0; --i) {
      if (bin[b].dims[i] != out_dims[i] && bin[b].dims[i] != 1) return ORC_INVALID_ARGUMENT;
      bs[b][i] = bin[b].dims[i] == 1 ? 0 : st;
      st *= bin[b].dims[i];
    }
  }
  /* output scale, :507-514 (mul_value starts at 1) */
  const float range_lhs = fmaxf(fabsf(min_x), fabsf(max_x));
  const float range_rhs = fmaxf(fabsf(min_y), fabsf(max_y));
  const float scale_output = range_lhs * range_rhs / (127.0f * 127.0f);
  const float scale = 1.0f * scale_output;

  int64_t batch = 1;
  for (int i = 0; i < nbo; ++i) batch *= out_dims[i];
  if (batch == 0 || M == 0 || N == 0) return ORC_OK;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t bi = 0; bi < batch; ++bi) {
    for (int64_t m = 0; m < M; ++m) {
      int64_t idx[8], rem = bi, xo = 0, yo = 0, bo[2] = {0, 0};
      for (int i = nbo - 1; i >= 0; --i) { idx[i] = rem % out_dims[i]; rem /= out_dims[i]; }
      for (int i = 0; i < nbo; ++i) {
        xo += idx[i] * xs[i]; yo += idx[i] * ys[i];
        for (int b = 0; b < n_binary; ++b) bo[b] += idx[i] * bs[b][i];
      }
      for (int64_t n = 0; n < N; ++n) {
        int32_t acc = 0;
        for (int64_t k = 0; k < K; ++k) {
          const int32_t xv = adj_x ? x[xo + k * M + m] : x[xo + m * K + k];
          const int32_t yv = adj_y ? y[yo + n * K + k] : y[yo + k * N + n];
          acc += xv * yv;
        }
        float v = (float)acc * scale;
        for (int b = 0; b < n_binary; ++b) {
          const int64_t o = bo[b] + m * bs[b][nbo] + n * bs[b][nbo + 1];
          const float t = t_out == ORC_FLOAT ? ((const float*)bin[b].data)[o]
                                             : bits16_to_f32(t_out, ((const uint16_t*)bin[b].data)[o]);
          v = bin[b].alg == ORC_BIN_MUL ? v * t : v + t;
        }
        const int64_t oo = (bi * M + m) * N + n;
        if (t_out == ORC_FLOAT) ((float*)out)[oo] = v;
        else ((uint16_t*)out)[oo] = f32_to_bits16(t_out, v);
      }
    }
  }
  return ORC_OK;
}


/* ---- quantized Conv2D ---------------------------------------------------------------------------- */
/* TensorFlow's GetWindowedOutputSizeVerbose, which conv_ops.h:405-440 reaches through its shape helper */
int orc_conv_out_dim(int64_t in, int64_t k, int stride, int dil, int padding, int pad_before, int pad_after,
                     int64_t* out, int64_t* pad_lead) {
  const int64_t eff = (k - 1) * dil + 1;
  if (stride <= 0 || dil <= 0) return ORC_INVALID_ARGUMENT;
  if (padding == ORC_PAD_VALID) {
    *out = (in - eff + stride) / stride;
    *pad_lead = 0;
  } else if (padding == ORC_PAD_SAME) {
    *out = (in + stride - 1) / stride;
    int64_t need = (*out - 1) * stride + eff - in;
    if (need < 0) need = 0;
    *pad_lead = need / 2;
  } else {
    *out = (in + pad_before + pad_after - eff + stride) / stride;
    *pad_lead = pad_before;
  }
  return *out < 0 ? ORC_INVALID_ARGUMENT : ORC_OK;
}

void orc_int_conv2d(const void* x, int x_type, const int8_t* w, const orc_conv_geom* g, int64_t out_h,
                    int64_t out_w, int64_t pad_top, int64_t pad_left, int32_t* acc) {
  const uint8_t* xu = (const uint8_t*)x;
  const int8_t* xs = (const int8_t*)x;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t b = 0; b < g->batch; ++b) {
    for (int64_t oh = 0; oh < out_h; ++oh) {
      for (int64_t ow = 0; ow < out_w; ++ow) {
        int32_t* dst = acc + ((b * out_h + oh) * out_w + ow) * g->out_c;
        for (int64_t o = 0; o < g->out_c; ++o) dst[o] = 0;
        for (int64_t kh = 0; kh < g->k_h; ++kh) {
          const int64_t ih = oh * g->stride_h - pad_top + kh * g->dil_h;
          if (ih < 0 || ih >= g->in_h) continue; /* zero padding */
          for (int64_t kw = 0; kw < g->k_w; ++kw) {
            const int64_t iw = ow * g->stride_w - pad_left + kw * g->dil_w;
            if (iw < 0 || iw >= g->in_w) continue;
            const int64_t xo = ((b * g->in_h + ih) * g->in_w + iw) * g->in_c;
            const int8_t* wf = w + (kh * g->k_w + kw) * g->in_c * g->out_c;
            for (int64_t c = 0; c < g->in_c; ++c) {
              const int32_t xv = x_type == ORC_QUINT8 ? (int32_t)xu[xo + c] : (int32_t)xs[xo + c];
              for (int64_t o = 0; o < g->out_c; ++o) dst[o] += xv * (int32_t)wf[c * g->out_c + o];
            }
          }
        }
      }
    }
  }
}

/* Depthwise: one group per input channel (conv_ops.h:238-246: oneDNN filter dims G = in_c, O = multiplier, I = 1), so
 * output channel c * mult + m = sum over the window of x[.., c] * w[kh, kw, c, m]; output depth in_c * mult (:395-397). */
void orc_int_depthwise_conv2d(const void* x, int x_type, const int8_t* w, const orc_conv_geom* g, int64_t mult,
                              int64_t out_h, int64_t out_w, int64_t pad_top, int64_t pad_left, int32_t* acc) {
  const uint8_t* xu = (const uint8_t*)x;
  const int8_t* xs = (const int8_t*)x;
  const int64_t oc = g->in_c * mult;
  for (int64_t b = 0; b < g->batch; ++b)
    for (int64_t oh = 0; oh < out_h; ++oh)
      for (int64_t ow = 0; ow < out_w; ++ow) {
        int32_t* dst = acc + ((b * out_h + oh) * out_w + ow) * oc;
        for (int64_t o = 0; o < oc; ++o) dst[o] = 0;
        for (int64_t kh = 0; kh < g->k_h; ++kh) {
          const int64_t ih = oh * g->stride_h - pad_top + kh * g->dil_h;
          if (ih < 0 || ih >= g->in_h) continue;
          for (int64_t kw = 0; kw < g->k_w; ++kw) {
            const int64_t iw = ow * g->stride_w - pad_left + kw * g->dil_w;
            if (iw < 0 || iw >= g->in_w) continue;
            const int64_t xo = ((b * g->in_h + ih) * g->in_w + iw) * g->in_c;
            const int8_t* wf = w + (kh * g->k_w + kw) * oc;
            for (int64_t c = 0; c < g->in_c; ++c) {
              const int32_t xv = x_type == ORC_QUINT8 ? (int32_t)xu[xo + c] : (int32_t)xs[xo + c];
              for (int64_t m = 0; m < mult; ++m) dst[c * mult + m] += xv * (int32_t)wf[c * mult + m];
            }
          }
        }
      }
}

int orc_qdepthwise_conv2d(const orc_conv_attrs* at, const orc_conv_geom* g, int64_t mult, const void* x, const int8_t* w,
                          const void* bias, float min_in, float max_in, const float* min_f, const float* max_f,
                          int64_t depth, float min_out, float max_out, void* out, int64_t* out_h, int64_t* out_w) {
  int64_t pt = 0, pl = 0;
  if (mult <= 0) return ORC_INVALID_ARGUMENT;
  if (orc_conv_out_dim(g->in_h, g->k_h, g->stride_h, g->dil_h, g->padding, g->pad_top, g->pad_bottom, out_h, &pt) ||
      orc_conv_out_dim(g->in_w, g->k_w, g->stride_w, g->dil_w, g->padding, g->pad_left, g->pad_right, out_w, &pl))
    return ORC_INVALID_ARGUMENT;
  const int64_t M = g->batch * *out_h * *out_w, N = g->in_c * mult;
  if (out == NULL || M == 0 || N == 0) return ORC_OK;
  int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)(M * N));
  float* scales = (float*)malloc(sizeof(float) * (size_t)(depth > 0 ? depth : 1));
  float* sb = (float*)malloc(sizeof(float) * (size_t)N);
  orc_epilogue_desc ep;
  int st = orc_qconv_prepare(at, N, min_in, max_in, min_f, max_f, depth, min_out, max_out, bias, scales, sb, &ep);
  if (st == ORC_OK) {
    orc_int_depthwise_conv2d(x, at->t_in, w, g, mult, *out_h, *out_w, pt, pl, acc);
    orc_qmatmul_epilogue(acc, M, N, &ep, scales, sb, NULL, at->t_out, out);
  }
  free(acc); free(scales); free(sb);
  return st;
}

int orc_qconv_prepare(const orc_conv_attrs* at, int64_t N, float min_in, float max_in, const float* min_f,
                      const float* max_f, int64_t depth, float min_out, float max_out, const void* bias,
                      float* scales, float* bias_out, orc_epilogue_desc* ep) {
  const int out_q8 = at->t_out == ORC_QINT8 || at->t_out == ORC_QUINT8;
  const int out_f = at->t_out == ORC_FLOAT || at->t_out == ORC_BFLOAT16 || at->t_out == ORC_HALF;
  if (!out_q8 && !out_f && at->t_out != ORC_QINT32) return ORC_INVALID_ARGUMENT;
  if (at->t_in != ORC_QUINT8 && at->t_in != ORC_QINT8) return ORC_INVALID_ARGUMENT;
  if (depth != 1 && depth != N) return ORC_INVALID_ARGUMENT;
  memset(ep, 0, sizeof(*ep));
  /* ---- output scales, ExtendInt8PostOps :329-393 ("Quantized" always sets output scales, :76) */
  for (int64_t i = 0; i < depth; ++i) scales[i] = 1.0f;
  if (out_f) {
    const float int_input_limit = (at->t_in == ORC_QUINT8) ? 255.0f : 127.0f;
    const float int_filter_limit = 127.0f;
    const float src_qscale_f32 = fmaxf(fabsf(min_in), fabsf(max_in)) / int_input_limit;
    for (int64_t i = 0; i < depth; ++i) {
      const float wei_qscale_f32 = fmaxf(fabsf(min_f[i]), fabsf(max_f[i])) / int_filter_limit;
      scales[i] = src_qscale_f32 * wei_qscale_f32;
    }
  } else if (out_q8) {
    const float int_output_limit = (at->t_out == ORC_QUINT8) ? 255.0f : 127.0f;
    const float float_input_range = fmaxf(fabsf(min_in), fabsf(max_in));
    const float float_output_range = fmaxf(fabsf(min_out), fabsf(max_out));
    const float int_const_scale_limit = (at->t_in == ORC_QUINT8) ? (float)(255.0 * 127.0) : (float)(127.0 * 127.0);
    for (int64_t i = 0; i < depth; ++i) {
      const float float_filter_range = fmaxf(fabsf(min_f[i]), fabsf(max_f[i]));
      scales[i] = int_output_limit * float_input_range * float_filter_range /
                  (int_const_scale_limit * float_output_range);
    }
  }
  ep->n_scales = (int)depth;
  /* ---- post-ops: one eltwise at most here; its post-op scale is set to 1 (:436-445) */
  if (at->activation == ORC_ACT_RELU) {
    ep->elt[0].alg = ORC_ELT_RELU; ep->elt[0].alpha = 0.0f; ep->elt[0].beta = 0.0f; ep->n_eltwise = 1;
  } else if (at->activation == ORC_ACT_LEAKYRELU) {
    ep->elt[0].alg = ORC_ELT_RELU; ep->elt[0].alpha = at->alpha; ep->elt[0].beta = 0.0f; ep->n_eltwise = 1;
  } else if (at->activation == ORC_ACT_ELU) {      /* table entries of onednn_post_op_util.cc:38, 59-60: alpha 1 */
    ep->elt[0].alg = ORC_ELT_ELU; ep->elt[0].alpha = 1.0f; ep->elt[0].beta = 0.0f; ep->n_eltwise = 1;
  } else if (at->activation == ORC_ACT_SIGMOID) {
    ep->elt[0].alg = ORC_ELT_LOGISTIC; ep->elt[0].alpha = 1.0f; ep->elt[0].beta = 0.0f; ep->n_eltwise = 1;
  } else if (at->activation != ORC_ACT_NONE) {
    /* "_FusedSwish" / "_FusedHardSwish" become "Swish" / "HardSwish" (:135-138); the table has no "Swish", and the
     * result of AddOps is not checked (:225), so that fusion silently drops the activation: not restated */
    return ORC_UNIMPLEMENTED;
  }
  /* ---- bias, GetBiasHandle :448-597 */
  if (at->t_bias == 0) {
    for (int64_t j = 0; j < N; ++j) bias_out[j] = 0.0f;
    return ORC_OK;
  }
  const float int_const_scale_limit = (at->t_in == ORC_QUINT8) ? (float)(255.0 * 127.0) : (float)(127.0 * 127.0);
  const float in_range = fmaxf(fabsf(max_in), fabsf(min_in));
  for (int64_t j = 0; j < N; ++j) {
    const int64_t i = depth == 1 ? 0 : j; /* reorder of the 1-D bias: one scale, or one per element (:573-577) */
    const float filt_range = fmaxf(fabsf(max_f[i]), fabsf(min_f[i]));
    if (at->t_bias == ORC_QINT32) {
      const float bf = (float)((const int32_t*)bias)[j]; /* cast to float, :462-468 */
      if (at->t_out == ORC_QINT32) bias_out[j] = bf;     /* used as is, :450-453 */
      else if (out_f) bias_out[j] = bf * ((in_range * filt_range) / int_const_scale_limit); /* :489-497 */
      else bias_out[j] = bf * scales[i];                 /* :505-509 */
    } else if (at->t_bias == ORC_FLOAT) {
      const float tmp_scale = int_const_scale_limit / (in_range * filt_range); /* :553-557 */
      bias_out[j] = ((const float*)bias)[j] * (tmp_scale * scales[i]);         /* :560, reorder */
    } else {
      return ORC_UNIMPLEMENTED;
    }
  }
  return ORC_OK;
}

int orc_qconv2d(const orc_conv_attrs* at, const orc_conv_geom* g, const void* x, const int8_t* w,
                const void* bias, float min_in, float max_in, const float* min_f, const float* max_f,
                int64_t depth, float min_out, float max_out, void* out, int64_t* out_h, int64_t* out_w) {
  return orc_qconv2d_sum(at, g, x, w, bias, min_in, max_in, min_f, max_f, depth, min_out, max_out, NULL, NULL, out, out_h,
                         out_w);
}

int orc_qconv2d_sum(const orc_conv_attrs* at, const orc_conv_geom* g, const void* x, const int8_t* w,
                    const void* bias, float min_in, float max_in, const float* min_f, const float* max_f,
                    int64_t depth, float min_out, float max_out, const orc_conv_sum* sum, const void* summand,
                    void* out, int64_t* out_h, int64_t* out_w) {
  int64_t pt = 0, pl = 0;
  if (sum != NULL && sum->position != 0) {
    if (at->t_out != ORC_QINT8 && at->t_out != ORC_QUINT8) return ORC_UNIMPLEMENTED; /* qint32 + float summand: not restated */
    if (sum->t_summand != ORC_QINT8 && sum->t_summand != ORC_QUINT8) return ORC_INVALID_ARGUMENT;
    if (sum->t_summand == ORC_QUINT8 && at->t_out == ORC_QINT8) return ORC_INVALID_ARGUMENT; /* :213-218 */
    if (sum->position != 1 && sum->position != 2) return ORC_INVALID_ARGUMENT;
  }
  if (orc_conv_out_dim(g->in_h, g->k_h, g->stride_h, g->dil_h, g->padding, g->pad_top, g->pad_bottom, out_h, &pt) ||
      orc_conv_out_dim(g->in_w, g->k_w, g->stride_w, g->dil_w, g->padding, g->pad_left, g->pad_right, out_w, &pl))
    return ORC_INVALID_ARGUMENT;
  const int64_t M = g->batch * *out_h * *out_w, N = g->out_c;
  if (out == NULL || M == 0 || N == 0) return ORC_OK; /* shape query or empty output */
  int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)(M * N));
  float* scales = (float*)malloc(sizeof(float) * (size_t)(depth > 0 ? depth : 1));
  float* sb = (float*)malloc(sizeof(float) * (size_t)N);
  orc_epilogue_desc ep;
  int st = orc_qconv_prepare(at, N, min_in, max_in, min_f, max_f, depth, min_out, max_out, bias, scales, sb, &ep);
  float* addend = NULL;
  if (st == ORC_OK && sum != NULL && sum->position != 0) {
    /* :398-433 */
    const float scale_output = fmaxf(fabsf(min_out), fabsf(max_out));
    const float scale_summand = fmaxf(fabsf(sum->min_summand), fabsf(sum->max_summand));
    float sum_post_op_scale;
    if (at->t_out == ORC_QUINT8 && sum->t_summand == ORC_QINT8) sum_post_op_scale = 255.0f * scale_summand / (scale_output * 127.0f);
    else sum_post_op_scale = scale_summand / scale_output;
    /* the destination's previous contents as the output type reads them (:622-626: bytes of a qint8 summand are
     * taken as quint8 when the output is quint8) */
    addend = (float*)malloc(sizeof(float) * (size_t)(M * N));
    for (int64_t i = 0; i < M * N; ++i)
      addend[i] = (at->t_out == ORC_QUINT8) ? (float)((const uint8_t*)summand)[i] : (float)((const int8_t*)summand)[i];
    /* place the sum in the chain: before or after the activation */
    orc_eltwise s_elt;
    s_elt.alg = ORC_ELT_SUM; s_elt.alpha = sum_post_op_scale; s_elt.beta = 0.0f;
    if (sum->position == 1 && ep.n_eltwise == 1) { ep.elt[1] = ep.elt[0]; ep.elt[0] = s_elt; ep.n_eltwise = 2; }
    else { ep.elt[ep.n_eltwise++] = s_elt; }
  }
  if (st == ORC_OK) {
    orc_int_conv2d(x, at->t_in, w, g, *out_h, *out_w, pt, pl, acc);
    orc_qmatmul_epilogue(acc, M, N, &ep, scales, sb, addend, at->t_out, out);
  }
  free(acc); free(scales); free(sb); free(addend);
  return st;
}
