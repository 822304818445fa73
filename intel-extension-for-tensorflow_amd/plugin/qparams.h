// Host-side parameter math of the quantization ops: what the op kernels compute from the host-memory
// min/max tensors before a device kernel is launched.  All arithmetic is IEEE fp32 unless a comment
// says otherwise, written expression by expression as the reference evaluates it (this file is built
// with contraction off).
//   AdjustRange          itex/core/kernels/common/quantize_op.h:130-152
//   ScaleZeroPoint       itex/core/utils/quantization_util.h:54-84
//   LegacyMinFirstScale  quantize_op.h:204-214
//   FloatForOneLevel     itex/core/kernels/onednn/block/quantized_ops.h:24-38
#ifndef ITEX_AMD_PLUGIN_QPARAMS_H_
#define ITEX_AMD_PLUGIN_QPARAMS_H_

#include <algorithm>
#include <cmath>
#include <cstdint>

#include "tf_c_api_subset.h"

namespace itex_amd {
namespace qparams {

enum class Mode { MIN_COMBINED = 0, MIN_FIRST = 1, SCALED = 2 };

// numeric limits of the quantized types as 64-bit integers (Eigen::NumTraits<T>::highest/lowest)
inline int64_t Highest(TF_DataType t) { return t == TF_QINT8 ? 127 : t == TF_QUINT8 ? 255 : 2147483647LL; }
inline int64_t Lowest(TF_DataType t) { return t == TF_QINT8 ? -128 : t == TF_QUINT8 ? 0 : -2147483648LL; }

// false when max < min ("input_max_range must be larger than input_min_range.")
inline bool AdjustRange(float in_min, float in_max, float ensure_minimum_range, float* out_min, float* out_max) {
  if (!(in_max >= in_min)) return false;
  const float lo = std::min(0.0f, in_min);
  const float epsilon = std::max(1.0f, std::max(std::fabs(in_min), std::fabs(in_max))) * ensure_minimum_range;
  const float widened = lo + epsilon;
  *out_min = lo;
  *out_max = std::max(0.0f, std::max(in_max, widened));
  return true;
}

// SCALED: symmetric range, zero point 0.  MIN_FIRST: affine, zero point rounded half away from zero.
// `dequantize` selects the direction of the scale.  min/max are updated in place for SCALED.
inline void ScaleZeroPoint(TF_DataType t, Mode mode, bool dequantize, float* mn, float* mx, float* scale,
                           int32_t* zero_point) {
  const float q_high = static_cast<float>(Highest(t));
  const float q_span = static_cast<float>(Highest(t) - Lowest(t));
  if (mode == Mode::SCALED) {
    const float r = std::max(std::fabs(*mn), std::fabs(*mx));
    *mx = r;
    *mn = -r;
    *scale = dequantize ? r / q_high : q_high / r;
    *zero_point = 0;
  } else {
    const float span = *mx - *mn;
    *scale = dequantize ? span / q_span : q_span / span;
    const float scaled_max = dequantize ? *mx / *scale : *mx * *scale;
    *zero_point = static_cast<int32_t>(std::round(q_high - scaled_max));
  }
}

// (2^bits - 1.0) / (max - min): the numerator is a double, so this one division is done in double and
// rounded to float once.
inline float LegacyMinFirstScale(TF_DataType t, float mn, float mx) {
  const int bits = (t == TF_QINT32) ? 32 : 8;
  const double steps = static_cast<double>(static_cast<int64_t>(1) << bits) - 1.0;
  return static_cast<float>(steps / static_cast<double>(mx - mn));
}

inline float FloatForOneLevel(TF_DataType t, float range_min, float range_max) {
  int64_t highest = Highest(t), lowest = Lowest(t);
  if (lowest < -highest) ++lowest;  // symmetric signed range
  return (range_max - range_min) / static_cast<float>(highest - lowest);
}

// range of a qint32 product (quantized_ops.h:40-54)
inline void RangeForMultiplication(TF_DataType t1, TF_DataType t2, float min_a, float max_a, float min_b,
                                   float max_b, float* min_c, float* max_c) {
  const float level = FloatForOneLevel(t1, min_a, max_a) * FloatForOneLevel(t2, min_b, max_b);
  *min_c = level * static_cast<float>(Lowest(TF_QINT32));
  *max_c = level * static_cast<float>(Highest(TF_QINT32));
}

}  // namespace qparams
}  // namespace itex_amd
#endif  // ITEX_AMD_PLUGIN_QPARAMS_H_
