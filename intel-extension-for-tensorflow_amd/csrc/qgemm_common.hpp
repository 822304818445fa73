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

// A post-op chain of the form [sum] [one activation] [sum] [one linear map], every part optional and at most one sum
// (every chain the MatMul and convolution ops build): resolved once on the host, so that the tile kernels apply it with a few
// wavefront-uniform branches per 32x32 tile instead of a loop over the chain per value.
enum : int { kChainMax0 = 1, kChainLeaky = 2, kChainClip = 4, kChainLinear = 8, kChainGeluTanh = 16, kChainGeluErf = 32,
             kChainSumFirst = 64, kChainSumLast = 128,  // y += sum_scale * addend before / after the activation
             kChainOther = 256 };                       // another transcendental activation: `other`
struct CanonChain {
  int flags;
  float alpha;         // leaky slope
  float lo, hi;        // clip bounds
  float lin_a, lin_b;  // y = lin_a * x + lin_b
  float sum_scale;
  itexhip_eltwise other;  // kChainOther: ELU, logistic, tanh, swish, mish (with its alpha)
};

struct EpilogueArgs {
  const float* scales;   // prepared per-channel scales (n_scales of them), unused when `fused`
  const void* bias;      // prepared fp32 bias, or the op's raw bias (fp32 / int32) when `fused`
  const int32_t* colsum;
  int n_scales;
  int comp_mul;  // 128 for u8 activations, 0 for s8
  int n_eltwise;
  itexhip_eltwise elt[3];
  const void* addend;    // [M, N] tensor of the "Add" / "Sum" fusion (ITEXHIP_ELT_SUM in the chain), else null
  int addend_type;       // ITEXHIP_FLOAT / BFLOAT16 / HALF (the MatMul's "Add": the output's type), or ITEXHIP_QINT8 /
                         // ITEXHIP_QUINT8 (the summand of a quantized convolution)
  // fused != 0: the kernel derives scale and bias of a channel itself from the op's ranges
  int fused;
  int nb;  // weight ranges (1 or N)
  const float* min_b;
  const float* max_b;
  PrepArgs prep;
  // per-row activation ranges (decode batches quantized per token): row m uses row_min_a[m], row_max_a[m]
  // in place of prep.min_a / prep.max_a; null for the reference's per-tensor range
  const float* row_min_a;
  const float* row_max_a;
  // per-tensor activation range in device memory ({min_a, max_a}, written by an earlier kernel on the same stream) in
  // place of prep.min_a / prep.max_a; null when the caller knows the range on the host
  const float* range_a;
  CanonChain canon;  // filled by the tile dispatch for the kernels that take it
};

// one element of the addend as fp32 (exact for the 8-bit types)
__device__ __forceinline__ float load_addend(const EpilogueArgs& e, int64_t i) {
  if (e.addend_type == ITEXHIP_QINT8) return static_cast<float>(static_cast<const int8_t*>(e.addend)[i]);
  if (e.addend_type == ITEXHIP_QUINT8) return static_cast<float>(static_cast<const uint8_t*>(e.addend)[i]);
  if (e.addend_type == ITEXHIP_BFLOAT16) return bf16_bits_to_f32(static_cast<const uint16_t*>(e.addend)[i]);
  if (e.addend_type == ITEXHIP_HALF) return f16_bits_to_f32(static_cast<const uint16_t*>(e.addend)[i]);
  return static_cast<const float*>(e.addend)[i];
}

// Host: the chain in canonical form.  Returns 0 (no post-op), 1 (ReLU only), 2 (sum, cheap activation and / or linear
// map), 3 (the same with GELU as the activation) or -1 (anything else: two activations, two sums, ...).
inline int canon_chain(const EpilogueArgs& e, CanonChain* c) {
  *c = CanonChain{};
  int k = 0;
  if (k < e.n_eltwise && e.elt[k].alg == ITEXHIP_ELT_SUM) {
    c->flags |= kChainSumFirst; c->sum_scale = e.elt[k].alpha;
    ++k;
  }
  if (k < e.n_eltwise) {
    const itexhip_eltwise& a = e.elt[k];
    if (a.alg == ITEXHIP_ELT_RELU) {
      if (a.alpha == 0.0f) c->flags |= kChainMax0; else { c->flags |= kChainLeaky; c->alpha = a.alpha; }
      ++k;
    } else if (a.alg == ITEXHIP_ELT_CLIP) {
      c->flags |= kChainClip; c->lo = a.alpha; c->hi = a.beta;
      ++k;
    } else if (a.alg == ITEXHIP_ELT_GELU_TANH || a.alg == ITEXHIP_ELT_GELU_ERF) {
      c->flags |= a.alg == ITEXHIP_ELT_GELU_TANH ? kChainGeluTanh : kChainGeluErf;
      ++k;
    } else if (a.alg >= ITEXHIP_ELT_ELU && a.alg <= ITEXHIP_ELT_MISH) {
      c->flags |= kChainOther; c->other = a;
      ++k;
    }
  }
  if (k < e.n_eltwise && e.elt[k].alg == ITEXHIP_ELT_SUM && !(c->flags & kChainSumFirst)) {
    c->flags |= kChainSumLast; c->sum_scale = e.elt[k].alpha;
    ++k;
  }
  if (k < e.n_eltwise && e.elt[k].alg == ITEXHIP_ELT_LINEAR) {
    c->flags |= kChainLinear; c->lin_a = e.elt[k].alpha; c->lin_b = e.elt[k].beta;
    ++k;
  }
  if (k != e.n_eltwise) return -1;
  if (c->flags == 0) return 0;
  if (c->flags == kChainMax0) return 1;
  return (c->flags & (kChainGeluTanh | kChainGeluErf | kChainOther)) ? 3 : 2;
}

// Scale, bias and zero-point compensation of channel n (n < N), however the call supplied them, in two
// stages so that a kernel can issue the loads early and do the arithmetic late.
__device__ __forceinline__ int first_lane_zero() {
  int z = 0;
  asm volatile("" : "+v"(z));
  return z;
}

struct RawChannel {
  float min_bj, max_bj, min_b0, max_b0;  // fused: weight ranges;  else min_bj holds the prepared scale
  uint32_t bias;                         // fused: the raw bias entry as loaded;  else the bits of the prepared fp32 bias
  int colsum;
  float min_a, max_a;                    // load_raw_channel_early only: the activation range the call runs with
};

// Only loads, all of them per-lane vector loads that nothing waits for here: a wavefront can issue them ahead of a
// long stream of other loads and meet the values at the end.  (A load from a wavefront-uniform address would become a
// scalar load, whose result the compiler wants at once: the lane-dependent zero keeps the first weight range on the
// vector path.)
__device__ __forceinline__ RawChannel load_raw_channel(const EpilogueArgs& e, int n, int N) {
  RawChannel r;  // the fields a path does not use stay undefined: assigning them would wait for the loads in flight
  r.colsum = e.colsum ? e.colsum[n] : 0;
  r.bias = e.fused ? bias_bits(e.prep, e.bias, n) : (e.bias ? static_cast<const uint32_t*>(e.bias)[n] : 0u);
  if (e.fused) {
    const int jb = (e.nb == N) ? n : 0;
    const int first = first_lane_zero();
    r.min_bj = e.min_b[jb];
    r.max_bj = e.max_b[jb];
    r.min_b0 = e.min_b[first];
    r.max_b0 = e.max_b[first];
  } else {
    r.min_bj = e.n_scales > 1 ? e.scales[n] : (e.n_scales == 1 ? e.scales[first_lane_zero()] : 1.0f);
  }
  return r;
}

// The same loads as load_raw_channel, written as assembly so that the compiler neither sees them nor waits for them:
// a kernel issues them, then a long run of global -> LDS loads (assembly as well), waits itself until only those are
// outstanding (vector memory loads return in the order issued) and calls settle_raw_channel before it touches a value.
__device__ __forceinline__ uint32_t early_load32(const void* p) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, off" : "=&v"(v) : "v"(p) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t early_load16(const void* p) {
  uint32_t v;
  asm volatile("global_load_ushort %0, %1, off" : "=&v"(v) : "v"(p) : "memory");
  return v;
}
constexpr int kEarlyChannelLoads = 8;  // at most: colsum, bias, four weight-range entries, the activation range
__device__ __forceinline__ RawChannel load_raw_channel_early(const EpilogueArgs& e, int n, int N) {
  RawChannel r;
  r.colsum = 0;
  r.bias = 0u;
  r.min_bj = 1.0f;
  r.max_bj = r.min_b0 = r.max_b0 = r.min_a = r.max_a = 0.0f;
  uint32_t t;
  if (e.colsum) r.colsum = static_cast<int>(early_load32(e.colsum + n));
  if (e.bias) {
    if (e.fused && e.prep.bias_16 != 0) r.bias = early_load16(static_cast<const uint16_t*>(e.bias) + n);
    else r.bias = early_load32(static_cast<const uint32_t*>(e.bias) + n);
  }
  if (e.fused) {
    const int jb = (e.nb == N) ? n : 0;
    t = early_load32(e.min_b + jb); r.min_bj = __uint_as_float(t);
    t = early_load32(e.max_b + jb); r.max_bj = __uint_as_float(t);
    t = early_load32(e.min_b); r.min_b0 = __uint_as_float(t);
    t = early_load32(e.max_b); r.max_b0 = __uint_as_float(t);
    r.min_a = e.prep.min_a;
    r.max_a = e.prep.max_a;
    if (e.range_a) {  // the range left in device memory by a dynamic quantization
      t = early_load32(e.range_a); r.min_a = __uint_as_float(t);
      t = early_load32(e.range_a + 1); r.max_a = __uint_as_float(t);
    }
  } else if (e.n_scales >= 1) {
    t = early_load32(e.scales + (e.n_scales > 1 ? n : 0)); r.min_bj = __uint_as_float(t);
  }
  return r;
}
// after the kernel's own wait: ties every later use of the values to this point of the instruction stream
__device__ __forceinline__ void settle_raw_channel(RawChannel& r) {
  asm volatile("" : "+v"(r.min_bj), "+v"(r.max_bj), "+v"(r.min_b0), "+v"(r.max_b0), "+v"(r.bias), "+v"(r.colsum), "+v"(r.min_a),
               "+v"(r.max_a));
}
// finish_channel for values that load_raw_channel_early brought: no load of its own
__device__ __forceinline__ void finish_channel_early(const EpilogueArgs& e, const RawChannel& r, int* comp, float* scale,
                                                     float* bias) {
  *comp = e.comp_mul * r.colsum;
  if (e.fused) {
    PrepArgs pr = e.prep;
    pr.min_a = r.min_a;
    pr.max_a = r.max_a;
    const ChannelScaleBias c = channel_scale_bias(pr, r.min_bj, r.max_bj, r.min_b0, r.max_b0, bias_from_bits(e.prep, r.bias),
                                                  r.colsum);
    *scale = e.n_scales > 0 ? c.scale : 1.0f;
    *bias = c.bias;
  } else {
    *scale = r.min_bj;
    *bias = __uint_as_float(r.bias);
  }
}

__device__ __forceinline__ void finish_channel(const EpilogueArgs& e, const RawChannel& r, int* comp, float* scale,
                                               float* bias) {
  *comp = e.comp_mul * r.colsum;
  if (e.fused) {
    PrepArgs pr = e.prep;
    if (e.range_a) {
      pr.min_a = e.range_a[0];
      pr.max_a = e.range_a[1];
    }
    const ChannelScaleBias c = channel_scale_bias(pr, r.min_bj, r.max_bj, r.min_b0, r.max_b0, bias_from_bits(e.prep, r.bias),
                                                  r.colsum);
    *scale = e.n_scales > 0 ? c.scale : 1.0f;
    *bias = c.bias;
  } else {
    *scale = r.min_bj;
    *bias = __uint_as_float(r.bias);
  }
}

__device__ __forceinline__ void resolve_channel(const EpilogueArgs& e, int n, int N, int* comp, float* scale, float* bias) {
  const RawChannel r = load_raw_channel(e, n, N);
  finish_channel(e, r, comp, scale, bias);
}

// ------------------------------------------------------------------------------------------------
// Fused epilogue.  A 32x32 accumulator tile is held in MFMA layout: lane l, register r (0..15) ->
//   m = m0 + (l % 32), n = n0 + (r / 4) * 8 + (l / 32) * 4 + (r % 4),
// so a lane owns 4 groups of 4 consecutive output channels of one row; epilogue_store handles one group.  The per-channel parameters of those 4
// channels are resolved once (ChannelParams) and reused for every row of the same channel group.
//   y = fl(fl((float)(acc + comp[n]) * scale[n]) + bias[n]);  eltwise chain;  convert.
// ACT selects the eltwise chain at compile time: 0 = none, 1 = relu (alpha 0), 2 = generic chain.
// ------------------------------------------------------------------------------------------------
struct ChannelParams {
  int comp[4];
  float scale[4];
  float bias[4];
};

// Four final fp32 values (as bit patterns) -> four outputs of type OUT_T in registers, no store.
// 8-bit outputs come back packed in .x, 16-bit ones in .x and .y; 32-bit outputs as 4 lanes of raw bits.
// 8-bit conversion: after the clamp to [lo, hi] (integers, |.| <= 255) adding 1.5 * 2^23 in fp32
// rounds to nearest even and leaves the integer in the low mantissa bits (two's complement for
// negatives), so the low byte of the sum is the result: one add instead of round + convert.
template <int OUT_T>
__device__ __forceinline__ v4i epilogue_pack(const v4i bits) {
  const float y[4] = {__int_as_float(bits[0]), __int_as_float(bits[1]), __int_as_float(bits[2]), __int_as_float(bits[3])};
  if constexpr (OUT_T == ITEXHIP_FLOAT) {
    return v4i{__float_as_int(y[0]), __float_as_int(y[1]), __float_as_int(y[2]), __float_as_int(y[3])};
  } else if constexpr (is_float16_type(OUT_T)) {  // 4 x 16 bits in .x, .y
    return v4i{static_cast<int>(f32x2_to_bits16<OUT_T>(y[0], y[1])), static_cast<int>(f32x2_to_bits16<OUT_T>(y[2], y[3])), 0, 0};
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

// The 4 outputs of one channel group: accumulators (zero-point compensation already included) -> scale, bias,
// activation -> epilogue_pack.
template <int OUT_T, int ACT>
__device__ __forceinline__ v4i epilogue_convert(const v4i acc, const f4 scale, const f4 bias, const EpilogueArgs& e) {
  v4i y;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float v = static_cast<float>(acc[r]);
    v = v * scale[r];
    v = v + bias[r];
    if (ACT == 1) {
      v = fmaxf(v, 0.0f);
    } else if (ACT == 2) {
      for (int k = 0; k < e.n_eltwise; ++k) v = apply_eltwise(e.elt[k], v);
    }
    y[r] = __float_as_int(v);
  }
  return epilogue_pack<OUT_T>(y);
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
      for (int k = 0; k < e.n_eltwise; ++k) {
        if (e.elt[k].alg == ITEXHIP_ELT_SUM) v = v + e.elt[k].alpha * load_addend(e, static_cast<int64_t>(m) * N + min(n + r, N - 1));
        else v = apply_eltwise(e.elt[k], v);
      }
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
  } else if constexpr (is_float16_type(OUT_T)) {
    uint16_t* dst = reinterpret_cast<uint16_t*>(out) + o;
    if (full) {
      typedef unsigned int u2 __attribute__((ext_vector_type(2)));
      *reinterpret_cast<u2*>(dst) = u2{f32x2_to_bits16<OUT_T>(y[0], y[1]), f32x2_to_bits16<OUT_T>(y[2], y[3])};
    } else {
      for (int r = 0; r < 4 && n + r < N; ++r) dst[r] = static_cast<uint16_t>(f32_to_bits16<OUT_T>(y[r]));
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

// Direct global -> LDS loads (global_load_lds_dwordx4): each lane's 16 bytes land at LDS base + 16 * lane, no VGPRs
// and no ds_write on the way.  They count in vmcnt like any other vector memory load and return in order with them.
__device__ __forceinline__ void lds_dma16(const void* gptr, uint32_t lds_addr) {
  // m0 = LDS byte address of lane 0's destination; the instruction adds 16 * lane
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(gptr), "s"(lds_addr) : "memory", "m0");
}
// same with a wavefront-uniform 64-bit base (SGPR pair) and a 32-bit per-lane byte offset: no vector
// address arithmetic per load
__device__ __forceinline__ void lds_dma16(const void* sbase, uint32_t lane_off, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane_off), "s"(sbase), "s"(lds_addr) : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  // s_waitcnt with only vmcnt active (gfx9 encoding: vmcnt[3:0] | expcnt 7 << 4 | lgkmcnt 15 << 8 | vmcnt[5:4] << 14)
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// Division of a dividend below 2^31 by a divisor that is fixed per launch: n / d = (n * mul) >> sh with
// sh = 31 + ceil(log2 d) and mul = ceil(2^sh / d) < 2^32, exact for every 0 <= n < 2^31 because
// 2^sh <= mul * d <= 2^sh + 2^(sh - 31) (Granlund and Montgomery, division by invariant integers).  One 32 x 32 -> 64 bit
// multiply and a shift where the division of two registers is a sequence of some thirty instructions.
struct FastDiv { uint32_t mul, sh; };
inline FastDiv make_fast_div(int64_t d) {  // host; 1 <= d < 2^31
  uint32_t s = 0;
  while ((1ull << s) < static_cast<uint64_t>(d)) ++s;
  const uint32_t sh = 31 + s;
  return FastDiv{static_cast<uint32_t>(((1ull << sh) + static_cast<uint64_t>(d) - 1) / static_cast<uint64_t>(d)), sh};
}
__device__ __forceinline__ int fast_div(int n, FastDiv f) {
  return static_cast<int>((static_cast<uint64_t>(static_cast<uint32_t>(n)) * f.mul) >> f.sh);
}

// Geometry of a Conv2D computed as an implicit GEMM by the tile kernel (32-bit: the host checks the ranges)
struct ConvTileArgs {
  int in_h, in_w, in_c, k_w, out_h, out_w;
  int stride_h, stride_w, dil_h, dil_w, pad_top, pad_left;
  FastDiv by_out_w, by_out_h, by_in_c, by_k_w;  // the kernel's row and window decompositions divide by these
};
constexpr int kMaxConvPieces = 1024;  // 16-byte pieces per patch row: 16 KiB of receptive field per output position

}  // namespace itexhip
#endif  // ITEXHIP_QGEMM_COMMON_HPP_
