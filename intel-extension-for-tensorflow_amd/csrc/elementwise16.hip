// 16-bit floating point ends of the quantization ops: QuantizeV2 from a bfloat16 tensor
// (_ITEXQuantizeV2 with dtype = bfloat16, itex/core/kernels/gpu/quantize_op.cc:38-51) and Dequantize
// to bfloat16 / half (itex/core/kernels/gpu/dequantize_op.cc:24-48).  The arithmetic is the fp32 one
// of the 32-bit kernels: a bfloat16 source widens exactly to fp32 first, a 16-bit destination is the
// fp32 result rounded to nearest even (what oneDNN's reorder does with such memory descriptors).
// 8 elements per lane-iteration: 16 B in / 8 B out for quantize, 8 B in / 16 B out for dequantize.
#include "common.hpp"

namespace itexhip {
namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 4;
typedef unsigned int u2 __attribute__((ext_vector_type(2)));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return bf16_bits_to_f32(h); }
__device__ __forceinline__ uint32_t f32_to_bf16(float f) { return f32_to_bf16_bits(f); }
__device__ __forceinline__ uint32_t f32_to_f16(float f) { return f32_to_f16_bits(f); }
template <int YT>
__device__ __forceinline__ uint32_t narrow(float f) {
  return YT == ITEXHIP_BFLOAT16 ? f32_to_bf16(f) : f32_to_f16(f);
}

template <int T>
__device__ __forceinline__ uint32_t quantize1(float x, float scale, float addend) {
  const float t = x * scale;
  return static_cast<uint32_t>(sat_rne<T>(t + addend)) & 0xffu;
}

template <int T>
__global__ __launch_bounds__(kThreads) void quantize_bf16_vec_kernel(const u4* __restrict__ x, u2* __restrict__ q,
                                                                     int64_t n8, float scale, float addend) {
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
  u4 v[kUnroll];
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const int64_t i = base + j * kThreads;
    if (i < n8) v[j] = __builtin_nontemporal_load(&x[i]);
  }
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const int64_t i = base + j * kThreads;
    if (i < n8) {
      uint32_t o[2] = {0, 0};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t h = (v[j][e >> 1] >> (16 * (e & 1))) & 0xffffu;
        o[e >> 2] |= quantize1<T>(bf16_to_f32(h), scale, addend) << (8 * (e & 3));
      }
      // written through (system scope), like the stores of the other narrowing kernels
      __hip_atomic_store(reinterpret_cast<unsigned long long*>(&q[i]),
                         static_cast<unsigned long long>(o[0]) | (static_cast<unsigned long long>(o[1]) << 32), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}

// any alignment / tails / per-axis parameters: one element per thread
template <int T>
__global__ __launch_bounds__(kThreads) void quantize_bf16_scalar_kernel(const uint16_t* __restrict__ x,
                                                                        uint8_t* __restrict__ q, int64_t begin, int64_t n,
                                                                        int64_t slices, int64_t inner,
                                                                        const float* __restrict__ scales,
                                                                        const float* __restrict__ addends, float scale0,
                                                                        float addend0) {
  const int64_t i = begin + static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) {
    float sc = scale0, ad = addend0;
    if (scales) {
      const int64_t s = (i / inner) % slices;
      sc = scales[s];
      ad = addends ? addends[s] : 0.0f;
    }
    q[i] = static_cast<uint8_t>(quantize1<T>(bf16_to_f32(x[i]), sc, ad));
  }
}

template <int T>
__device__ __forceinline__ float widen8(uint32_t b) {
  if (T == ITEXHIP_QINT8) return static_cast<float>(static_cast<int>(static_cast<int8_t>(b & 0xffu)));
  return static_cast<float>(b & 0xffu);
}

template <int T, int YT>
__global__ __launch_bounds__(kThreads) void dequantize16_vec_kernel(const u2* __restrict__ q, u4* __restrict__ y,
                                                                    int64_t n8, float scale, float zp) {
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
  u2 w[kUnroll];
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const int64_t i = base + j * kThreads;
    if (i < n8) w[j] = q[i];  // ordinary load, as in the fp32 Dequantize
  }
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const int64_t i = base + j * kThreads;
    if (i < n8) {
      uint32_t o[4] = {0, 0, 0, 0};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = (widen8<T>(w[j][e >> 2] >> (8 * (e & 3))) - zp) * scale;
        o[e >> 1] |= narrow<YT>(f) << (16 * (e & 1));
      }
      __builtin_nontemporal_store(u4{o[0], o[1], o[2], o[3]}, &y[i]);
    }
  }
}

template <int T, int YT>
__global__ __launch_bounds__(kThreads) void dequantize16_scalar_kernel(const uint8_t* __restrict__ q,
                                                                       uint16_t* __restrict__ y, int64_t begin, int64_t n,
                                                                       int64_t slices, int64_t inner,
                                                                       const float* __restrict__ scales,
                                                                       const int32_t* __restrict__ zps, float scale0,
                                                                       float zp0) {
  const int64_t i = begin + static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) {
    float sc = scale0, zp = zp0;
    if (scales) {
      const int64_t s = (i / inner) % slices;
      sc = scales[s];
      zp = zps ? static_cast<float>(zps[s]) : 0.0f;
    }
    y[i] = static_cast<uint16_t>(narrow<YT>((widen8<T>(q[i]) - zp) * sc));
  }
}

inline unsigned blocks_for(int64_t n, int64_t per_block) { return static_cast<unsigned>((n + per_block - 1) / per_block); }

template <int T>
void launch_quantize_bf16(const void* x, void* q, int64_t n, int64_t slices, int64_t inner, const float* scales,
                          const float* addends, float scale, float addend, hipStream_t st) {
  int64_t done = 0;
  if (!scales && aligned(x, 16) && aligned(q, 8) && n >= 8) {
    const int64_t n8 = n / 8;
    quantize_bf16_vec_kernel<T><<<blocks_for(n8, kThreads * kUnroll), kThreads, 0, st>>>(
        static_cast<const u4*>(x), static_cast<u2*>(q), n8, scale, addend);
    done = n8 * 8;
  }
  if (done < n)
    quantize_bf16_scalar_kernel<T><<<blocks_for(n - done, kThreads), kThreads, 0, st>>>(
        static_cast<const uint16_t*>(x), static_cast<uint8_t*>(q), done, n, slices, inner, scales, addends, scale, addend);
}

template <int T, int YT>
void launch_dequantize16(const void* q, void* y, int64_t n, int64_t slices, int64_t inner, const float* scales,
                         const int32_t* zps, float scale, float zp, hipStream_t st) {
  int64_t done = 0;
  if (!scales && aligned(q, 8) && aligned(y, 16) && n >= 8) {
    const int64_t n8 = n / 8;
    dequantize16_vec_kernel<T, YT><<<blocks_for(n8, kThreads * kUnroll), kThreads, 0, st>>>(
        static_cast<const u2*>(q), static_cast<u4*>(y), n8, scale, zp);
    done = n8 * 8;
  }
  if (done < n)
    dequantize16_scalar_kernel<T, YT><<<blocks_for(n - done, kThreads), kThreads, 0, st>>>(
        static_cast<const uint8_t*>(q), static_cast<uint16_t*>(y), done, n, slices, inner, scales, zps, scale, zp);
}

int check_types(const char* who, int q_type, int f_type, bool quantize) {
  ITEXHIP_REQUIRE(q_type == ITEXHIP_QINT8 || q_type == ITEXHIP_QUINT8, "%s: the quantized type must be qint8 or quint8, got %d",
                  who, q_type);
  if (quantize) {
    ITEXHIP_REQUIRE(f_type == ITEXHIP_BFLOAT16, "%s: the source type must be bfloat16, got %d", who, f_type);
  } else {
    ITEXHIP_REQUIRE(f_type == ITEXHIP_BFLOAT16 || f_type == ITEXHIP_HALF, "%s: the destination type must be bfloat16 or half, got %d",
                    who, f_type);
  }
  return ITEXHIP_OK;
}

}  // namespace
}  // namespace itexhip

using namespace itexhip;

extern "C" int itexhip_quantize_bf16(const void* x, void* q, int64_t n, int dst_type, float scale, float addend,
                                     void* stream) {
  if (int st = check_types("itexhip_quantize_bf16", dst_type, ITEXHIP_BFLOAT16, true)) return st;
  ITEXHIP_REQUIRE(n >= 0, "itexhip_quantize_bf16: negative size");
  if (n == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(x && q && aligned(x, 2), "itexhip_quantize_bf16: null or misaligned buffer");
  if (dst_type == ITEXHIP_QINT8) launch_quantize_bf16<ITEXHIP_QINT8>(x, q, n, 1, 1, nullptr, nullptr, scale, addend, as_stream(stream));
  else launch_quantize_bf16<ITEXHIP_QUINT8>(x, q, n, 1, 1, nullptr, nullptr, scale, addend, as_stream(stream));
  ITEXHIP_CHECK_LAUNCH("itexhip_quantize_bf16");
  return ITEXHIP_OK;
}

extern "C" int itexhip_quantize_axis_bf16(const void* x, void* q, int64_t outer, int64_t slices, int64_t inner,
                                          int dst_type, const float* scales, const float* addends, void* stream) {
  if (int st = check_types("itexhip_quantize_axis_bf16", dst_type, ITEXHIP_BFLOAT16, true)) return st;
  ITEXHIP_REQUIRE(outer >= 0 && slices >= 0 && inner >= 0, "itexhip_quantize_axis_bf16: negative size");
  const int64_t n = outer * slices * inner;
  if (n == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(x && q && scales && aligned(x, 2), "itexhip_quantize_axis_bf16: null or misaligned buffer");
  if (dst_type == ITEXHIP_QINT8) launch_quantize_bf16<ITEXHIP_QINT8>(x, q, n, slices, inner, scales, addends, 0.0f, 0.0f, as_stream(stream));
  else launch_quantize_bf16<ITEXHIP_QUINT8>(x, q, n, slices, inner, scales, addends, 0.0f, 0.0f, as_stream(stream));
  ITEXHIP_CHECK_LAUNCH("itexhip_quantize_axis_bf16");
  return ITEXHIP_OK;
}

#define ITEXHIP_DEQ16_DISPATCH(...)                                                                         \
  do {                                                                                                      \
    if (src_type == ITEXHIP_QINT8 && y_type == ITEXHIP_BFLOAT16) launch_dequantize16<ITEXHIP_QINT8, ITEXHIP_BFLOAT16>(__VA_ARGS__); \
    else if (src_type == ITEXHIP_QINT8) launch_dequantize16<ITEXHIP_QINT8, ITEXHIP_HALF>(__VA_ARGS__);      \
    else if (y_type == ITEXHIP_BFLOAT16) launch_dequantize16<ITEXHIP_QUINT8, ITEXHIP_BFLOAT16>(__VA_ARGS__); \
    else launch_dequantize16<ITEXHIP_QUINT8, ITEXHIP_HALF>(__VA_ARGS__);                                    \
  } while (0)

extern "C" int itexhip_dequantize16(const void* q, void* y, int64_t n, int src_type, int y_type, float scale,
                                    int32_t zero_point, void* stream) {
  if (int st = check_types("itexhip_dequantize16", src_type, y_type, false)) return st;
  ITEXHIP_REQUIRE(n >= 0, "itexhip_dequantize16: negative size");
  if (n == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(q && y && aligned(y, 2), "itexhip_dequantize16: null or misaligned buffer");
  ITEXHIP_DEQ16_DISPATCH(q, y, n, 1, 1, nullptr, nullptr, scale, static_cast<float>(zero_point), as_stream(stream));
  ITEXHIP_CHECK_LAUNCH("itexhip_dequantize16");
  return ITEXHIP_OK;
}

extern "C" int itexhip_dequantize_axis16(const void* q, void* y, int64_t outer, int64_t slices, int64_t inner,
                                         int src_type, int y_type, const float* scales, const int32_t* zero_points,
                                         void* stream) {
  if (int st = check_types("itexhip_dequantize_axis16", src_type, y_type, false)) return st;
  ITEXHIP_REQUIRE(outer >= 0 && slices >= 0 && inner >= 0, "itexhip_dequantize_axis16: negative size");
  const int64_t n = outer * slices * inner;
  if (n == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(q && y && scales && aligned(y, 2), "itexhip_dequantize_axis16: null or misaligned buffer");
  ITEXHIP_DEQ16_DISPATCH(q, y, n, slices, inner, scales, zero_points, 0.0f, 0.0f, as_stream(stream));
  ITEXHIP_CHECK_LAUNCH("itexhip_dequantize_axis16");
  return ITEXHIP_OK;
}
