// Shared pieces of the quantized MatMul kernels: operand chunk format, epilogue, compile-time loops.
#ifndef ITEXHIP_QGEMM_COMMON_HPP_
#define ITEXHIP_QGEMM_COMMON_HPP_

#include <algorithm>
#include <type_traits>
#include <utility>

#include "qmatmul_params.hpp"

namespace itexhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

__device__ __forceinline__ bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

constexpr int kChunkRows = 32;     // rows (output channels or activation rows) per operand chunk
constexpr int kChunkK = 32;        // k per operand chunk
constexpr int kChunkBytes = 1024;  // 32 rows x 32 k
constexpr int64_t kMaxK = 1 << 16; // 255 * 128 * 65536 < 2^31

struct EpilogueArgs {
  const float* scales;   // prepared per-channel scales (n_scales of them), unused when `fused`
  const float* bias;     // prepared bias, or the op's raw fp32 bias when `fused`
  const int32_t* colsum;
  int n_scales;
  int comp_mul;  // 128 for u8 activations, 0 for s8
  int n_eltwise;
  itexhip_eltwise elt[2];
  // fused != 0: the kernel derives scale and bias of a channel itself from the op's ranges
  int fused;
  int nb;  // weight ranges (1 or N)
  const float* min_b;
  const float* max_b;
  PrepArgs prep;
};

// scale, bias and zero-point compensation of channel n (n < N), however the call supplied them
__device__ __forceinline__ void resolve_channel(const EpilogueArgs& e, int n, int N, int* comp, float* scale, float* bias) {
  *comp = e.comp_mul ? e.comp_mul * e.colsum[n] : 0;
  if (e.fused) {
    const ChannelScaleBias c = channel_scale_bias(e.prep, e.min_b, e.max_b, e.nb, e.bias, e.colsum, N, n);
    *scale = e.n_scales > 0 ? c.scale : 1.0f;
    *bias = c.bias;
  } else {
    *scale = e.n_scales > 1 ? e.scales[n] : (e.n_scales == 1 ? e.scales[0] : 1.0f);
    *bias = e.bias ? e.bias[n] : 0.0f;
  }
}

// ------------------------------------------------------------------------------------------------
// Fused epilogue.  A 32x32 accumulator tile is held in MFMA layout: lane l, register r (0..15) ->
//   m = m0 + (l % 32), n = n0 + (r / 4) * 8 + (l / 32) * 4 + (r % 4),
// so a lane owns 4 groups of 4 consecutive output channels of one row; epilogue_store handles one group.  The per-channel parameters of those 4
// channels are loaded once (ChannelParams) and reused for every row tile of the same channel tile.
//   y = fl(fl((float)(acc + comp[n]) * scale[n]) + bias[n]);  eltwise chain;  convert.
// ACT selects the eltwise chain at compile time: 0 = none, 1 = relu (alpha 0), 2 = generic chain.
// ------------------------------------------------------------------------------------------------
struct ChannelParams {
  int comp[4];
  float scale[4];
  float bias[4];
};

__device__ __forceinline__ ChannelParams load_channel_params(const EpilogueArgs& e, int n, int N, bool vec_ok) {
  ChannelParams p;
  if (e.fused) {
#pragma unroll
    for (int r = 0; r < 4; ++r) resolve_channel(e, min(n + r, N - 1), N, &p.comp[r], &p.scale[r], &p.bias[r]);
    return p;
  }
  if (vec_ok && n + 3 < N) {
    if (e.comp_mul) {
      const v4i c = *reinterpret_cast<const v4i*>(e.colsum + n);
#pragma unroll
      for (int r = 0; r < 4; ++r) p.comp[r] = e.comp_mul * c[r];
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) p.comp[r] = 0;
    }
    if (e.n_scales > 1) {
      const f4 s = *reinterpret_cast<const f4*>(e.scales + n);
#pragma unroll
      for (int r = 0; r < 4; ++r) p.scale[r] = s[r];
    } else {
      const float s = e.n_scales == 1 ? e.scales[0] : 1.0f;
#pragma unroll
      for (int r = 0; r < 4; ++r) p.scale[r] = s;
    }
    if (e.bias) {
      const f4 b = *reinterpret_cast<const f4*>(e.bias + n);
#pragma unroll
      for (int r = 0; r < 4; ++r) p.bias[r] = b[r];
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) p.bias[r] = 0.0f;
    }
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int nn = min(n + r, N - 1);  // clamped: out-of-range channels are computed but never stored
      p.comp[r] = e.comp_mul ? e.comp_mul * e.colsum[nn] : 0;
      p.scale[r] = e.n_scales > 1 ? e.scales[nn] : (e.n_scales == 1 ? e.scales[0] : 1.0f);
      p.bias[r] = e.bias ? e.bias[nn] : 0.0f;
    }
  }
  return p;
}

// The 4 outputs of one channel group in registers: epilogue arithmetic + conversion, no store.
// 8-bit outputs come back packed in .x; 32-bit outputs as 4 lanes of raw bits.
// 8-bit conversion: after the clamp to [lo, hi] (integers, |.| <= 255) adding 1.5 * 2^23 in fp32
// rounds to nearest even and leaves the integer in the low mantissa bits (two's complement for
// negatives), so the low byte of the sum is the result: one add instead of round + convert.
template <int OUT_T, int ACT>
__device__ __forceinline__ v4i epilogue_convert(const v4i acc, const f4 scale, const f4 bias, const EpilogueArgs& e) {
  float y[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float v = static_cast<float>(acc[r]);  // the zero-point compensation is already part of acc
    v = v * scale[r];
    v = v + bias[r];
    if (ACT == 1) {
      v = fmaxf(v, 0.0f);
    } else if (ACT == 2) {
      for (int k = 0; k < e.n_eltwise; ++k) v = apply_eltwise(e.elt[k], v);
    }
    y[r] = v;
  }
  if constexpr (OUT_T == ITEXHIP_FLOAT) {
    return v4i{__float_as_int(y[0]), __float_as_int(y[1]), __float_as_int(y[2]), __float_as_int(y[3])};
  } else if constexpr (OUT_T == ITEXHIP_QINT32) {
    return v4i{sat_rne<ITEXHIP_QINT32>(y[0]), sat_rne<ITEXHIP_QINT32>(y[1]), sat_rne<ITEXHIP_QINT32>(y[2]),
               sat_rne<ITEXHIP_QINT32>(y[3])};
  } else {
    uint32_t b[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float v = __builtin_amdgcn_fmed3f(y[r], Sat<OUT_T>::lo, Sat<OUT_T>::hi);  // clamp in one instruction
      b[r] = static_cast<uint32_t>(__float_as_int(v + 12582912.0f));
    }
    // bytes: result = {b0.byte0, b1.byte0, b2.byte0, b3.byte0}; v_perm selects from {hi operand bytes 4..7, lo 0..3}
    const uint32_t lo01 = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u);  // [b0.0, b1.0, 0, 0]
    const uint32_t hi23 = __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);  // [0, 0, b2.0, b3.0]
    return v4i{static_cast<int>(lo01 | hi23), 0, 0, 0};
  }
}

template <int OUT_T, int ACT>
__device__ __forceinline__ void epilogue_store(const v4i acc, const ChannelParams& p, int m, int n, int M, int N,
                                               const EpilogueArgs& e, void* __restrict__ out, bool vec_ok) {
  if (m >= M || n >= N) return;
  float y[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float v = static_cast<float>(acc[r] + p.comp[r]);
    v = v * p.scale[r];  // scale 1.0f when the node has no output scale (exact)
    if (e.bias || e.fused) v = v + p.bias[r];
    if (ACT == 1) {
      v = fmaxf(v, 0.0f);
    } else if (ACT == 2) {
      for (int k = 0; k < e.n_eltwise; ++k) v = apply_eltwise(e.elt[k], v);
    }
    y[r] = v;
  }
  const int64_t o = static_cast<int64_t>(m) * N + n;
  const bool full = vec_ok && (n + 3 < N);
  if constexpr (OUT_T == ITEXHIP_FLOAT) {
    float* dst = reinterpret_cast<float*>(out) + o;
    if (full) {
      *reinterpret_cast<f4*>(dst) = f4{y[0], y[1], y[2], y[3]};
    } else {
      for (int r = 0; r < 4 && n + r < N; ++r) dst[r] = y[r];
    }
  } else if constexpr (OUT_T == ITEXHIP_QINT32) {
    int32_t* dst = reinterpret_cast<int32_t*>(out) + o;
    if (full) {
      *reinterpret_cast<v4i*>(dst) = v4i{sat_rne<ITEXHIP_QINT32>(y[0]), sat_rne<ITEXHIP_QINT32>(y[1]),
                                         sat_rne<ITEXHIP_QINT32>(y[2]), sat_rne<ITEXHIP_QINT32>(y[3])};
    } else {
      for (int r = 0; r < 4 && n + r < N; ++r) dst[r] = sat_rne<ITEXHIP_QINT32>(y[r]);
    }
  } else {
    uint8_t* dst = reinterpret_cast<uint8_t*>(out) + o;
    if (full) {
      *reinterpret_cast<uint32_t*>(dst) =
          pack4(sat_rne<OUT_T>(y[0]), sat_rne<OUT_T>(y[1]), sat_rne<OUT_T>(y[2]), sat_rne<OUT_T>(y[3]));
    } else {
      for (int r = 0; r < 4 && n + r < N; ++r) dst[r] = static_cast<uint8_t>(sat_rne<OUT_T>(y[r]));
    }
  }
}

// Compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(<N-1>).  Indices into register arrays
// are constants from the start, so the arrays are split into registers without relying on loop unrolling.
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

}  // namespace itexhip
#endif  // ITEXHIP_QGEMM_COMMON_HPP_
