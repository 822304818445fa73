// Shared host/device helpers of the itexhip kernels (gfx950 only).
#ifndef ITEXHIP_COMMON_HPP_
#define ITEXHIP_COMMON_HPP_

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "itexhip.h"

// Every fp32 operation in the quantization arithmetic must round on its own: no fused multiply-add.
#pragma clang fp contract(off)

namespace itexhip {

// native vector types (usable with the nontemporal load/store builtins)
typedef float f4 __attribute__((ext_vector_type(4)));
typedef int i4 __attribute__((ext_vector_type(4)));

void set_error(const char* fmt, ...);

// Tile shape forced by itexhip_test_force_tile_shape (-1: chosen from the problem size); [0] MatMul, [1] Conv2D.
extern int g_forced_tile_shape[2];

inline int hip_fail(hipError_t e, const char* what) {
  set_error("%s: %s", what, hipGetErrorString(e));
  return ITEXHIP_INTERNAL;
}

#define ITEXHIP_CHECK_LAUNCH(what)                                   \
  do {                                                               \
    hipError_t e__ = hipGetLastError();                              \
    if (e__ != hipSuccess) return ::itexhip::hip_fail(e__, what);    \
  } while (0)

#define ITEXHIP_REQUIRE(cond, ...)            \
  do {                                        \
    if (!(cond)) {                            \
      ::itexhip::set_error(__VA_ARGS__);      \
      return ITEXHIP_INVALID_ARGUMENT;        \
    }                                         \
  } while (0)

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// One bit per device ordinal (64 of them) for state that is per device, not per process, such as the dynamic
// shared memory limit of a kernel: device_bit(mask, false) tells whether the current device's bit is set,
// device_bit(mask, true) sets it (and returns whether it was set before).  Callers test, do their idempotent set-up,
// then set the bit; two threads that arrive together both do the set-up.
inline bool device_bit(unsigned long long* mask, bool set) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  const unsigned long long bit = 1ull << (dev & 63);
  if (set) return (__atomic_fetch_or(mask, bit, __ATOMIC_ACQ_REL) & bit) != 0;
  return (__atomic_load_n(mask, __ATOMIC_ACQUIRE) & bit) != 0;
}

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Saturation bounds of the destination type, in fp32 (the s32 upper bound is the largest float
// below 2^31).
template <int T> struct Sat;
template <> struct Sat<ITEXHIP_QINT8> { static constexpr float lo = -128.0f, hi = 127.0f; };
template <> struct Sat<ITEXHIP_QUINT8> { static constexpr float lo = 0.0f, hi = 255.0f; };
template <> struct Sat<ITEXHIP_QINT32> { static constexpr float lo = -2147483648.0f, hi = 2147483520.0f; };

// clamp in fp32, then round to nearest even (v_rndne_f32), then convert.
template <int T>
__device__ __forceinline__ int sat_rne(float y) {
  y = fmaxf(y, Sat<T>::lo);
  y = fminf(y, Sat<T>::hi);
  return static_cast<int>(__builtin_rintf(y));
}

// fp32 <-> bfloat16 bit patterns (round to nearest even, NaN kept quiet).  The conversion instruction of this GPU
// (v_cvt_pk_bf16_f32, two values per instruction) returns, for every one of the 2^32 fp32 bit patterns, the bits of the
// integer formula  u = bits(f); NaN ? (u >> 16) | 0x40 : (u + 0x7fff + ((u >> 16) & 1)) >> 16  (compared exhaustively
// on the device), at a twelfth of its instructions.
typedef __bf16 itexhip_bf16x2 __attribute__((ext_vector_type(2)));
typedef float itexhip_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ uint32_t f32x2_to_bf16_bits(float lo, float hi) {  // lo in bits 0..15, hi in bits 16..31
  const itexhip_bf16x2 r = __builtin_convertvector(itexhip_f32x2{lo, hi}, itexhip_bf16x2);
  uint32_t u;
  __builtin_memcpy(&u, &r, 4);
  return u;
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  const __bf16 h = static_cast<__bf16>(f);
  unsigned short bits;
  __builtin_memcpy(&bits, &h, 2);
  return bits;
}

// fp32 <-> half bit patterns (v_cvt_f16_f32 / v_cvt_f32_f16: round to nearest even, denormals kept)
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  // The value must exist as a rounded fp32 number before it is narrowed: without this the compiler may merge
  // the producing multiply / add with the conversion into one mixed-precision instruction that rounds once.
  asm("" : "+v"(f));
  const _Float16 h = static_cast<_Float16>(f);
  unsigned short bits;
  __builtin_memcpy(&bits, &h, 2);
  return bits;
}
__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
  const unsigned short bits = static_cast<unsigned short>(b);
  _Float16 h;
  __builtin_memcpy(&h, &bits, 2);
  return static_cast<float>(h);
}

// the 16-bit float types travel as bit patterns
__host__ __device__ constexpr bool is_float16_type(int t) { return t == ITEXHIP_BFLOAT16 || t == ITEXHIP_HALF; }
// float-like output types: the parameter preparation treats them alike (fp32 epilogue, converted in the store)
__host__ __device__ constexpr bool is_float_out(int t) { return t == ITEXHIP_FLOAT || is_float16_type(t); }
template <int T16>
__device__ __forceinline__ uint32_t f32_to_bits16(float f) {
  if constexpr (T16 == ITEXHIP_BFLOAT16) return f32_to_bf16_bits(f);
  else return f32_to_f16_bits(f);
}
template <int T16>
__device__ __forceinline__ uint32_t f32x2_to_bits16(float lo, float hi) {  // two values packed in a dword, lo first
  if constexpr (T16 == ITEXHIP_BFLOAT16) return f32x2_to_bf16_bits(lo, hi);
  else return f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16);
}

// one output element of a quantized MatMul: fp32 kept, bfloat16 / half rounded, integers saturated + rounded
template <int OUT_T>
__device__ __forceinline__ void store_output(void* __restrict__ out, int64_t idx, float v) {
  if constexpr (OUT_T == ITEXHIP_FLOAT) static_cast<float*>(out)[idx] = v;
  else if constexpr (is_float16_type(OUT_T)) static_cast<uint16_t*>(out)[idx] = static_cast<uint16_t>(f32_to_bits16<OUT_T>(v));
  else if constexpr (OUT_T == ITEXHIP_QINT32) static_cast<int32_t*>(out)[idx] = sat_rne<ITEXHIP_QINT32>(v);
  else static_cast<uint8_t*>(out)[idx] = static_cast<uint8_t>(sat_rne<OUT_T>(v));
}

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
  return (static_cast<uint32_t>(a) & 0xffu) | ((static_cast<uint32_t>(b) & 0xffu) << 8) |
         ((static_cast<uint32_t>(c) & 0xffu) << 16) | ((static_cast<uint32_t>(d) & 0xffu) << 24);
}

__device__ __forceinline__ float apply_eltwise(const itexhip_eltwise& e, float x) {
  switch (e.alg) {
    case ITEXHIP_ELT_RELU:
      if (e.alpha == 0.0f) return fmaxf(x, 0.0f);
      return x > 0.0f ? x : x * e.alpha;
    case ITEXHIP_ELT_CLIP:
      return fminf(fmaxf(x, e.alpha), e.beta);
    case ITEXHIP_ELT_LINEAR:
      return e.alpha * x + e.beta;
    case ITEXHIP_ELT_GELU_TANH: {
      // 0.5 x (1 + tanh(u)), u = sqrt(2/pi) x (1 + 0.044715 x^2), evaluated as x / (1 + exp(-2u)): the same function
      // (1 + tanh(u) = 2 / (1 + exp(-2u))) at a fifth of the instructions of tanhf, within 4e-7 relative of it
      // (hardware exp2 and reciprocal, about 1 ulp each); exp overflows to inf only where the result is -0.
      // exp(-2u) = 2^(x (c1 + c2 x^2)) with c1 = -2 sqrt(2/pi) log2(e), c2 = 0.044715 c1.
      const float e = __builtin_amdgcn_exp2f(x * fmaf(x * x, -0.10294324159622192f, -2.3022081851959229f));
      return x * __builtin_amdgcn_rcpf(1.0f + e);
    }
    case ITEXHIP_ELT_GELU_ERF: {
      // 0.5 x (1 + erf(z)), z = x / sqrt(2).  1 + erf(z) = erfc(-z): q = P(t) exp(-z^2) for z < 0 and 2 - q for z >= 0,
      // with t = 1 / (1 + p |z|) and the five-term polynomial of Abramowitz & Stegun 7.1.26 (|error| <= 1.5e-7 in erf,
      // the form oneDNN's own GELU kernels use): a reciprocal, an exp2 and a dozen other instructions where the library
      // erff took four times as many.  Against erff in double precision over [-12, 12] the result stays within a fifth
      // of 1e-6 + 2e-6 |y|; +-inf and NaN come out as the erff form gives them.
      const float z = x * 0.707106769084930419921875f, az = fabsf(z);
      const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, az, 1.0f));
      float p = fmaf(t, 1.061405429f, -1.453152027f);
      p = fmaf(p, t, 1.421413741f);
      p = fmaf(p, t, -0.284496736f);
      p = fmaf(p, t, 0.254829592f);
      p = p * t;
      const float q = p * __builtin_amdgcn_exp2f((az * az) * -1.44269502162933349609375f);
      const float s = z < 0.0f ? q : 2.0f - q;
      return (0.5f * x) * s;
    }
    // The exponential-based ones go through the hardware exp2 and reciprocal (about 1 ulp each), in forms that neither
    // overflow nor cancel: a few 1e-7 from the libm evaluation, like the GELU above.
    case ITEXHIP_ELT_ELU: {  // x > 0 ? x : alpha (e^x - 1)
      // e^x - 1 without the library's expm1f (which made this the slowest epilogue by far): below -0.35 the hardware
      // exp2 minus one (the subtraction costs less than a bit there), above it x + x^2 (1/2 + x/6 + ... + x^5 / 5040);
      // 1.6e-7 relative against expm1 in double precision at worst.
      const float far = __builtin_amdgcn_exp2f(x * 1.44269502162933349609375f) - 1.0f;
      float h = fmaf(1.0f / 5040.0f, x, 1.0f / 720.0f);
      h = fmaf(h, x, 1.0f / 120.0f);
      h = fmaf(h, x, 1.0f / 24.0f);
      h = fmaf(h, x, 1.0f / 6.0f);
      h = fmaf(h, x, 0.5f);
      const float near = fmaf(x * x, h, x);
      float neg = e.alpha * (x > -0.35f ? near : far);
      asm volatile("" : "+v"(neg));  // computed for every lane, then selected: as a branch per value the 16 values of
      return x > 0.0f ? x : neg;     // a tile ran one after the other, each waiting for its own exp2
    }
    case ITEXHIP_ELT_LOGISTIC:  // 1 / (1 + e^-x)
      return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269502162933349609375f));
    case ITEXHIP_ELT_TANH:  // 1 - 2 / (1 + e^(2x)): e^(2x) = inf gives 1, 0 gives -1
      return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * 2.885390043258667f));
    case ITEXHIP_ELT_SWISH:  // x / (1 + e^(-alpha x))
      return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(e.alpha * x * -1.44269502162933349609375f));
    case ITEXHIP_ELT_MISH: {  // x tanh(ln(1 + e^x)) = x t / (t + 2), t = e^x (e^x + 2); x beyond 20: tanh(.) = 1 in fp32
      const float n = __builtin_amdgcn_exp2f(fminf(x, 20.0f) * 1.44269502162933349609375f);
      const float t = n * (n + 2.0f);
      float y = x * t * __builtin_amdgcn_rcpf(t + 2.0f);
      asm volatile("" : "+v"(y));  // a select, not a branch per value (see ELU)
      return x > 20.0f ? x : y;
    }
    default:
      return x;
  }
}

}  // namespace itexhip
#endif  // ITEXHIP_COMMON_HPP_
