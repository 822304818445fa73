// HBM-bound elementwise kernels: QuantizeV2, Dequantize, RequantizePerChannel and the min/max
// reductions.  One wavefront instruction moves 1 KiB (16 B per lane, lanes contiguous); each thread
// keeps several such loads in flight before it converts and stores.
#include <algorithm>
#include <mutex>

#include "common.hpp"

namespace itexhip {
namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 4;  // 16-byte loads in flight per thread
// Launch shapes of the three streaming conversions, measured at 2^28 elements (5 bytes of traffic per element):
// the narrowing ones (16 bytes in, 4 out per thread and step: QuantizeV2, Requantize) run fastest when a workgroup
// takes two steps a whole grid apart with one load in flight (6.65 TB/s against 6.1 with four loads in one step);
// the widening one (4 bytes in, 16 out: Dequantize) gains about 1 % from two adjacent steps at once instead of four
// (6.2 TB/s either way: its 4-byte loads are a fifth of the traffic, the 16-byte stores set the pace; 16-byte loads
// with four strided stores per lane were measured at a quarter of that).
constexpr int kNarrowSteps = 2;
constexpr int kWidenUnroll = 2;

// ------------------------------------------------------------------------------------------------
// Quantize: q = sat(rne(fl(x * scale) + addend))
// ------------------------------------------------------------------------------------------------
template <int T>
__device__ __forceinline__ uint32_t quantize4(f4 v, float scale, float addend) {
  const float a = v.x * scale, b = v.y * scale, c = v.z * scale, d = v.w * scale;
  return pack4(sat_rne<T>(a + addend), sat_rne<T>(b + addend), sat_rne<T>(c + addend),
               sat_rne<T>(d + addend));
}

// The 4-byte stores of the narrowing kernels (4 or 16 bytes read per byte written) go out as system-scope stores (sc0 sc1:
// written through instead of held in L2): next to streaming loads that measured 6 % faster than streaming (nt) stores
// (QuantizeV2 over 2^28 elements: 199 -> 188 us).  The widening kernels are the other way round (nt stores 182 us, sc1 205 us).
__device__ __forceinline__ void store_through(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// n4 = number of complete groups of 4 elements; the caller handles the tail.
template <int T>
__global__ __launch_bounds__(kThreads) void quantize_vec_kernel(const f4* __restrict__ x,
                                                                uint32_t* __restrict__ q, int64_t n4,
                                                                float scale, float addend,
                                                                const float* __restrict__ dev_params) {
  if (dev_params) {  // {scale, addend} left in device memory by quantize_dynamic_params_kernel
    scale = dev_params[0];
    addend = dev_params[1];
  }
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
#pragma unroll 1
  for (int step = 0; step < kNarrowSteps; ++step, i += stride) {
    if (i < n4) {
      const f4 v = __builtin_nontemporal_load(&x[i]);
      store_through(&q[i], quantize4<T>(v, scale, addend));
    }
  }
}

template <int T>
__global__ __launch_bounds__(kThreads) void quantize_scalar_kernel(const float* __restrict__ x,
                                                                   uint8_t* __restrict__ q,
                                                                   int64_t begin, int64_t n,
                                                                   float scale, float addend,
                                                                   const float* __restrict__ dev_params) {
  if (dev_params) {
    scale = dev_params[0];
    addend = dev_params[1];
  }
  const int64_t i = begin + static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) {
    const float t = x[i] * scale;
    q[i] = static_cast<uint8_t>(sat_rne<T>(t + addend));
  }
}

// [outer, slices, inner] with per-slice scale / addend
template <int T>
__global__ __launch_bounds__(kThreads) void quantize_axis_kernel(const float* __restrict__ x,
                                                                 uint8_t* __restrict__ q, int64_t n,
                                                                 int64_t slices, int64_t inner,
                                                                 const float* __restrict__ scales,
                                                                 const float* __restrict__ addends) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) {
    const int64_t s = (i / inner) % slices;
    const float t = x[i] * scales[s];
    const float a = addends ? addends[s] : 0.0f;
    q[i] = static_cast<uint8_t>(sat_rne<T>(t + a));
  }
}

// The same, 4 elements per lane, 32-bit index arithmetic (the host sends tensors of 2^32 groups or more, odd shapes
// and unaligned buffers to the kernel above).  LAST: the quantized axis is the innermost one (inner == 1, slices a
// multiple of 4): a lane's 4 elements are 4 consecutive slices, their parameters one 16-byte load each.  Otherwise
// inner is a multiple of 4 and the 4 elements share a slice.  Same expression per element as above.
template <int T, bool LAST>
__global__ __launch_bounds__(kThreads) void quantize_axis_vec_kernel(const f4* __restrict__ x, uint32_t* __restrict__ q,
                                                                     uint32_t n4, uint32_t slices, uint32_t inner4,
                                                                     const float* __restrict__ scales,
                                                                     const float* __restrict__ addends) {
  const uint32_t stride = gridDim.x * kThreads;  // two steps a whole grid apart, as in quantize_vec_kernel
  uint32_t i = blockIdx.x * kThreads + threadIdx.x;
#pragma unroll 1
  for (int step = 0; step < kNarrowSteps; ++step, i += stride) {
    if (i >= n4) return;
    const f4 v = __builtin_nontemporal_load(&x[i]);
    f4 sc, ad = {0.0f, 0.0f, 0.0f, 0.0f};
    if constexpr (LAST) {
      const uint32_t s4 = i % (slices >> 2);
      sc = reinterpret_cast<const f4*>(scales)[s4];
      if (addends) ad = reinterpret_cast<const f4*>(addends)[s4];
    } else {
      const uint32_t sl = (i / inner4) % slices;
      const float c = scales[sl], a = addends ? addends[sl] : 0.0f;
      sc = f4{c, c, c, c};
      ad = f4{a, a, a, a};
    }
    const float a = v.x * sc.x, b = v.y * sc.y, c = v.z * sc.z, d = v.w * sc.w;
    store_through(&q[i], pack4(sat_rne<T>(a + ad.x), sat_rne<T>(b + ad.y), sat_rne<T>(c + ad.z), sat_rne<T>(d + ad.w)));
  }
}

// ------------------------------------------------------------------------------------------------
// Dequantize: y = ((float)q - zp) * scale
// ------------------------------------------------------------------------------------------------
template <int T>
__device__ __forceinline__ float widen(uint32_t w, int byte) {
  const uint32_t b = (w >> (8 * byte)) & 0xffu;
  if (T == ITEXHIP_QINT8) return static_cast<float>(static_cast<int>(static_cast<int8_t>(b)));
  return static_cast<float>(b);
}

template <int T>
__global__ __launch_bounds__(kThreads) void dequantize_vec_kernel(const uint32_t* __restrict__ q,
                                                                  f4* __restrict__ y, int64_t n4,
                                                                  float scale, float zp) {
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kThreads * kWidenUnroll) + threadIdx.x;
  uint32_t w[kWidenUnroll];
#pragma unroll
  for (int j = 0; j < kWidenUnroll; ++j) {
    const int64_t i = base + j * kThreads;
    // ordinary loads: a wavefront reads only 256 B per instruction here, and with streaming (nontemporal) loads of that
    // width the kernel measured 10 % slower; the 16-byte loads of the narrowing kernels are the other way round
    if (i < n4) w[j] = q[i];
  }
#pragma unroll
  for (int j = 0; j < kWidenUnroll; ++j) {
    const int64_t i = base + j * kThreads;
    if (i < n4) {
      f4 o;
      o.x = (widen<T>(w[j], 0) - zp) * scale;
      o.y = (widen<T>(w[j], 1) - zp) * scale;
      o.z = (widen<T>(w[j], 2) - zp) * scale;
      o.w = (widen<T>(w[j], 3) - zp) * scale;
      __builtin_nontemporal_store(o, &y[i]);
    }
  }
}

template <int T>
__global__ __launch_bounds__(kThreads) void dequantize_axis_kernel(const uint8_t* __restrict__ q,
                                                                   float* __restrict__ y, int64_t begin,
                                                                   int64_t n, int64_t slices,
                                                                   int64_t inner,
                                                                   const float* __restrict__ scales,
                                                                   const int32_t* __restrict__ zps,
                                                                   float scale0, float zp0) {
  const int64_t i = begin + static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) {
    float sc = scale0, zp = zp0;
    if (scales) {
      const int64_t s = (i / inner) % slices;
      sc = scales[s];
      zp = zps ? static_cast<float>(zps[s]) : 0.0f;
    }
    const float v = (T == ITEXHIP_QINT8) ? static_cast<float>(static_cast<int8_t>(q[i]))
                                         : static_cast<float>(q[i]);
    y[i] = (v - zp) * sc;
  }
}

// Per-slice dequantization, 4 elements per lane; LAST and the index arithmetic as in quantize_axis_vec_kernel.
template <int T, bool LAST>
__global__ __launch_bounds__(kThreads) void dequantize_axis_vec_kernel(const uint32_t* __restrict__ q, f4* __restrict__ y,
                                                                       uint32_t n4, uint32_t slices, uint32_t inner4,
                                                                       const float* __restrict__ scales,
                                                                       const int32_t* __restrict__ zps) {
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= n4) return;
  const uint32_t w = q[i];  // ordinary load, as in dequantize_vec_kernel
  f4 sc, zp = {0.0f, 0.0f, 0.0f, 0.0f};
  if constexpr (LAST) {
    const uint32_t s4 = i % (slices >> 2);
    sc = reinterpret_cast<const f4*>(scales)[s4];
    if (zps) {
      const i4 z = reinterpret_cast<const i4*>(zps)[s4];
      zp = f4{static_cast<float>(z.x), static_cast<float>(z.y), static_cast<float>(z.z), static_cast<float>(z.w)};
    }
  } else {
    const uint32_t sl = (i / inner4) % slices;
    const float c = scales[sl], z = zps ? static_cast<float>(zps[sl]) : 0.0f;
    sc = f4{c, c, c, c};
    zp = f4{z, z, z, z};
  }
  f4 r;
  r.x = (widen<T>(w, 0) - zp.x) * sc.x;
  r.y = (widen<T>(w, 1) - zp.y) * sc.y;
  r.z = (widen<T>(w, 2) - zp.z) * sc.z;
  r.w = (widen<T>(w, 3) - zp.w) * sc.w;
  __builtin_nontemporal_store(r, &y[i]);
}

// ------------------------------------------------------------------------------------------------
// Requantize: q = sat(rne((float)x * scale[c]))
// ------------------------------------------------------------------------------------------------
// kMode 0: one scale passed by value; 1: depth % 4 == 0, scales read as f4; 2: the same with fewer than 2^31 groups,
// where the channel group of a lane is found by one 32-bit remainder and then stepped instead of a 64-bit remainder
// per step (256 channels over 2^28 elements: 199 -> 195 us); n4 = groups of 4
template <int T, int kMode>
__global__ __launch_bounds__(kThreads) void requantize_vec_kernel(const i4* __restrict__ x,
                                                                  uint32_t* __restrict__ q, int64_t n4,
                                                                  float scale,
                                                                  const float* __restrict__ scales,
                                                                  int64_t depth4) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  uint32_t group = 0, group_step = 0;
  if (kMode == 2) {
    group = static_cast<uint32_t>(i) % static_cast<uint32_t>(depth4);
    group_step = static_cast<uint32_t>(stride) % static_cast<uint32_t>(depth4);  // the same for every lane
  }
#pragma unroll 1
  for (int step = 0; step < kNarrowSteps; ++step, i += stride) {
    if (i < n4) {
      const i4 v = __builtin_nontemporal_load(&x[i]);
      f4 s = f4{scale, scale, scale, scale};
      if (kMode == 1) s = reinterpret_cast<const f4*>(scales)[i % depth4];
      if (kMode == 2) {
        s = reinterpret_cast<const f4*>(scales)[group];
        group += group_step;
        if (group >= static_cast<uint32_t>(depth4)) group -= static_cast<uint32_t>(depth4);
      }
      const float a = static_cast<float>(v.x) * s.x, b = static_cast<float>(v.y) * s.y;
      const float c = static_cast<float>(v.z) * s.z, d = static_cast<float>(v.w) * s.w;
      store_through(&q[i], pack4(sat_rne<T>(a), sat_rne<T>(b), sat_rne<T>(c), sat_rne<T>(d)));
    }
  }
}

template <int T>
__global__ __launch_bounds__(kThreads) void requantize_scalar_kernel(const int32_t* __restrict__ x,
                                                                     uint8_t* __restrict__ q,
                                                                     int64_t begin, int64_t n,
                                                                     int64_t depth, float scale,
                                                                     const float* __restrict__ scales) {
  const int64_t i = begin + static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) {
    const float s = scales ? scales[i % depth] : scale;
    q[i] = static_cast<uint8_t>(sat_rne<T>(static_cast<float>(x[i]) * s));
  }
}

// ------------------------------------------------------------------------------------------------
// min / max reductions
// ------------------------------------------------------------------------------------------------
__global__ void fill_minmax_i32_kernel(int32_t* mn, int32_t* mx, int64_t depth) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < depth) {
    mn[i] = INT32_MAX;
    mx[i] = INT32_MIN;
  }
}

__device__ __forceinline__ int wave_min(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ int wave_max(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
  return v;
}

// Whole-tensor reductions.  At most kReduceBlocks workgroups walk the tensor; per round a workgroup
// takes kReduceUnroll consecutive 4 KiB pieces (all loads issued before the first compare).  The
// wavefronts of a workgroup meet in LDS and one thread issues the workgroup's single atomic pair:
// atomics on one address are serialised by the memory system (~10 ns each), so their number, not the
// data, would otherwise set the run time.
constexpr int kReduceUnroll = 8;
constexpr int kReduceBlocks = 512;

template <class V, class Less, class Commit>
__device__ __forceinline__ void block_minmax_commit(V mn, V mx, Less less, Commit commit) {
  __shared__ V smn[kThreads / 64], smx[kThreads / 64];
  if ((threadIdx.x & 63) == 0) {
    smn[threadIdx.x >> 6] = mn;
    smx[threadIdx.x >> 6] = mx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) {
      if (less(smn[w], mn)) mn = smn[w];
      if (less(mx, smx[w])) mx = smx[w];
    }
    commit(mn, mx);
  }
}

__global__ __launch_bounds__(kThreads) void minmax_i32_flat_kernel(const i4* __restrict__ x, int64_t n4,
                                                                   const int32_t* __restrict__ tail,
                                                                   int ntail, int32_t* mn_out,
                                                                   int32_t* mx_out) {
  int mn = INT32_MAX, mx = INT32_MIN;
  const int64_t round = static_cast<int64_t>(gridDim.x) * (kThreads * kReduceUnroll);
  int64_t i = static_cast<int64_t>(blockIdx.x) * (kThreads * kReduceUnroll) + threadIdx.x;
  for (; i + (kReduceUnroll - 1) * kThreads < n4; i += round) {
    i4 v[kReduceUnroll];
#pragma unroll
    for (int j = 0; j < kReduceUnroll; ++j) v[j] = __builtin_nontemporal_load(&x[i + j * kThreads]);
#pragma unroll
    for (int j = 0; j < kReduceUnroll; ++j) {
      mn = min(min(mn, v[j].x), min(v[j].y, min(v[j].z, v[j].w)));
      mx = max(max(mx, v[j].x), max(v[j].y, max(v[j].z, v[j].w)));
    }
  }
  // the tensor's last, partial group of pieces (it belongs to one workgroup only)
  for (int j = 0; j < kReduceUnroll && i + j * kThreads < n4; ++j) {
    const i4 v = x[i + j * kThreads];
    mn = min(min(mn, v.x), min(v.y, min(v.z, v.w)));
    mx = max(max(mx, v.x), max(v.y, max(v.z, v.w)));
  }
  if (blockIdx.x == 0 && static_cast<int>(threadIdx.x) < ntail) {
    mn = min(mn, tail[threadIdx.x]);
    mx = max(mx, tail[threadIdx.x]);
  }
  mn = wave_min(mn);
  mx = wave_max(mx);
  block_minmax_commit(
      mn, mx, [](int p, int q) { return p < q; },
      [&](int lo, int hi) {
        atomicMin(mn_out, lo);
        atomicMax(mx_out, hi);
      });
}

// Per-channel reduction, channel = last dim: thread owns one channel of its block's column group
// and walks a chunk of rows (loads are contiguous across the threads of a wavefront).
__global__ __launch_bounds__(kThreads) void minmax_i32_channel_kernel(const int32_t* __restrict__ x,
                                                                      int64_t rows, int64_t depth,
                                                                      int64_t rows_per_block,
                                                                      int32_t* mn_out, int32_t* mx_out) {
  const int64_t c = static_cast<int64_t>(blockIdx.y) * kThreads + threadIdx.x;
  if (c >= depth) return;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * rows_per_block;
  const int64_t r1 = min(rows, r0 + rows_per_block);
  int mn = INT32_MAX, mx = INT32_MIN;
  for (int64_t r = r0; r < r1; ++r) {
    const int v = x[r * depth + c];
    mn = min(mn, v);
    mx = max(mx, v);
  }
  if (r0 < r1) {
    atomicMin(&mn_out[c], mn);
    atomicMax(&mx_out[c], mx);
  }
}

// order-preserving map fp32 -> int32 (and back)
__device__ __forceinline__ int f2key(float f) {
  const int b = __float_as_int(f);
  return b >= 0 ? b : b ^ 0x7fffffff;
}
__device__ __forceinline__ float key2f(int k) { return __int_as_float(k >= 0 ? k : k ^ 0x7fffffff); }

__global__ void fill_minmax_f32_kernel(int* keys) {
  keys[0] = f2key(__builtin_inff());
  keys[1] = f2key(-__builtin_inff());
}
__global__ void finish_minmax_f32_kernel(int* keys) {
  const float mn = key2f(keys[0]), mx = key2f(keys[1]);
  reinterpret_cast<float*>(keys)[0] = mn;
  reinterpret_cast<float*>(keys)[1] = mx;
}

// PARTIALS: workgroup b leaves its own minimum and maximum as floats in keys[2b], keys[2b + 1] (no initialisation and
// no atomics needed; a consumer reduces the gridDim.x pairs); else the two order-preserving keys are updated atomically.
template <bool PARTIALS>
__global__ __launch_bounds__(kThreads) void minmax_f32_kernel(const f4* __restrict__ x, int64_t n4,
                                                              const float* __restrict__ tail, int ntail,
                                                              int* keys) {
  float mn = __builtin_inff(), mx = -__builtin_inff();
  const int64_t round = static_cast<int64_t>(gridDim.x) * (kThreads * kReduceUnroll);
  int64_t i = static_cast<int64_t>(blockIdx.x) * (kThreads * kReduceUnroll) + threadIdx.x;
  for (; i + (kReduceUnroll - 1) * kThreads < n4; i += round) {
    f4 v[kReduceUnroll];
#pragma unroll
    for (int j = 0; j < kReduceUnroll; ++j) v[j] = __builtin_nontemporal_load(&x[i + j * kThreads]);
#pragma unroll
    for (int j = 0; j < kReduceUnroll; ++j) {
      mn = fminf(fminf(mn, v[j].x), fminf(v[j].y, fminf(v[j].z, v[j].w)));
      mx = fmaxf(fmaxf(mx, v[j].x), fmaxf(v[j].y, fmaxf(v[j].z, v[j].w)));
    }
  }
  // the tensor's last, partial group of pieces (it belongs to one workgroup only)
  for (int j = 0; j < kReduceUnroll && i + j * kThreads < n4; ++j) {
    const f4 v = x[i + j * kThreads];
    mn = fminf(fminf(mn, v.x), fminf(v.y, fminf(v.z, v.w)));
    mx = fmaxf(fmaxf(mx, v.x), fmaxf(v.y, fmaxf(v.z, v.w)));
  }
  if (blockIdx.x == 0 && static_cast<int>(threadIdx.x) < ntail) {
    mn = fminf(mn, tail[threadIdx.x]);
    mx = fmaxf(mx, tail[threadIdx.x]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, o, 64));
    mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  }
  block_minmax_commit(
      mn, mx, [](float p, float q) { return p < q; },
      [&](float lo, float hi) {
        if constexpr (PARTIALS) {
          reinterpret_cast<float*>(keys)[2 * blockIdx.x] = lo;
          reinterpret_cast<float*>(keys)[2 * blockIdx.x + 1] = hi;
        } else {
          atomicMin(&keys[0], f2key(lo));
          atomicMax(&keys[1], f2key(hi));
        }
      });
}

// fill + reduction of n > 0 floats into the two order-preserving integer keys (finish_minmax_f32_kernel, or a
// consumer that decodes the keys itself, turns them into floats)
inline void enqueue_minmax_f32(const float* x, int64_t n, int* keys, hipStream_t st) {
  fill_minmax_f32_kernel<<<1, 1, 0, st>>>(keys);
  // the vector body starts at the first 16-byte boundary; head and tail go through `tail` slots
  const uintptr_t addr = reinterpret_cast<uintptr_t>(x);
  int64_t head = static_cast<int64_t>(((16 - (addr & 15)) & 15) / 4);
  if (head > n) head = n;
  const int64_t n4 = (n - head) / 4;
  const int64_t ntail = n - head - n4 * 4;
  const unsigned grid = static_cast<unsigned>(std::min<int64_t>(
      kReduceBlocks, std::max<int64_t>(1, (n4 + kThreads * kReduceUnroll - 1) / (kThreads * kReduceUnroll))));
  minmax_f32_kernel<false><<<grid, kThreads, 0, st>>>(reinterpret_cast<const f4*>(x + head), n4, x + head + n4 * 4,
                                                      static_cast<int>(ntail), keys);
  if (head > 0) minmax_f32_kernel<false><<<1, kThreads, 0, st>>>(nullptr, 0, x, static_cast<int>(head), keys);
}

inline unsigned blocks_for(int64_t n, int64_t per_block) {
  return static_cast<unsigned>((n + per_block - 1) / per_block);
}

// ------------------------------------------------------------------------------------------------
// Plain device-to-device copy (16 B per lane): the kernel of known traffic against which the memory
// counters are calibrated, and the stream's device copy.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void copy_vec_kernel(const i4* __restrict__ src, i4* __restrict__ dst,
                                                            int64_t n16) {
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
  i4 v[kUnroll];
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const int64_t i = base + j * kThreads;
    if (i < n16) v[j] = __builtin_nontemporal_load(&src[i]);
  }
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const int64_t i = base + j * kThreads;
    if (i < n16) __builtin_nontemporal_store(v[j], &dst[i]);
  }
}

// Read-only sweep: every workgroup walks the buffer a whole grid apart with four 16-byte loads in flight per lane and
// keeps nothing.  Timed by the caller, it gives what one launch that only reads that many bytes costs on a device:
// the floor under any kernel that has to stream the same bytes once.
__global__ __launch_bounds__(kThreads) void read_probe_kernel(const i4* __restrict__ src, int64_t n16, int* __restrict__ sink) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * (kThreads * kUnroll);
  i4 acc = i4{0, 0, 0, 0};
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x; i + (kUnroll - 1) * kThreads < n16; i += stride) {
    i4 v[kUnroll];
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) v[j] = __builtin_nontemporal_load(&src[i + j * kThreads]);
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) acc ^= v[j];
  }
  const int s = acc.x ^ acc.y ^ acc.z ^ acc.w;
  if (s == 0x5a17c0de) sink[threadIdx.x] = s;  // keeps the loads alive; practically never taken
}

__global__ __launch_bounds__(kThreads) void copy_byte_kernel(const uint8_t* __restrict__ src,
                                                             uint8_t* __restrict__ dst, int64_t begin, int64_t n) {
  const int64_t i = begin + static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

}  // namespace
}  // namespace itexhip

using namespace itexhip;

namespace itexhip {
namespace {
// std::min / std::max as the host code evaluates them (the first argument unless the second is smaller / larger)
__device__ __forceinline__ float host_min(float a, float b) { return b < a ? b : a; }
__device__ __forceinline__ float host_max(float a, float b) { return a < b ? b : a; }

// The QuantizeV2 parameter math of a per-tensor range, on the device (quantize_op.h:130-152 range adjustment,
// quantization_util.h:54-84 SCALED scale, quantize_op.h:204-214 legacy MIN_FIRST scale): state[0..1] = the tensor's
// min and max -> state[2..3] = the op's output_min / output_max, state[4..5] = scale and addend of the kernel.
struct DynamicParams {
  float out_min, out_max, scale, addend;
};

__device__ __forceinline__ DynamicParams dynamic_params(float in_min, float in_max, int dst_type, int mode,
                                                        float ensure_minimum_range) {
  const float lo = host_min(0.0f, in_min);
  const float epsilon = host_max(1.0f, host_max(fabsf(in_min), fabsf(in_max))) * ensure_minimum_range;
  const float widened = lo + epsilon;
  float mn = lo, mx = host_max(0.0f, host_max(in_max, widened));
  DynamicParams p;
  if (mode == ITEXHIP_SCALED) {
    const float q_high = dst_type == ITEXHIP_QINT8 ? 127.0f : 255.0f;
    const float r = host_max(fabsf(mn), fabsf(mx));
    mx = r;
    mn = -r;
    p.scale = q_high / r;
    p.addend = 0.0f;
    if (dst_type == ITEXHIP_QUINT8) mn = 0.0f;  // output_min of an unsigned SCALED result (:402-408)
  } else if (mode == ITEXHIP_MIN_FIRST_CLASSIC) {  // scale and zero point, the latter rounded half away from zero
    const float q_high = dst_type == ITEXHIP_QINT8 ? 127.0f : 255.0f;
    const float span = mx - mn;
    p.scale = 255.0f / span;
    const float scaled_max = mx * p.scale;
    p.addend = static_cast<float>(static_cast<int>(roundf(q_high - scaled_max)));
  } else {  // the 255 steps are a double, so the division is done in double and rounded once
    p.scale = static_cast<float>(255.0 / static_cast<double>(mx - mn));
    const float shift = -mn;
    p.addend = shift * p.scale;
  }
  p.out_min = mn;
  p.out_max = mx;
  return p;
}

__global__ void quantize_dynamic_params_kernel(float* state, int dst_type, int mode, float ensure_minimum_range) {
  // state[0..1] arrive as the reduction's integer keys; they leave as floats
  const float in_min = key2f(reinterpret_cast<const int*>(state)[0]), in_max = key2f(reinterpret_cast<const int*>(state)[1]);
  const DynamicParams p = dynamic_params(in_min, in_max, dst_type, mode, ensure_minimum_range);
  state[0] = in_min;
  state[1] = in_max;
  state[2] = p.out_min;
  state[3] = p.out_max;
  state[4] = p.scale;
  state[5] = p.addend;
}

// Small tensors (a decode batch: a few rows of activations) in ONE launch: every workgroup reduces the whole tensor
// (it comes from L2 after the first touch), derives the parameters, and quantizes its own slice; workgroup 0 also
// leaves the state.  Several kernels in a row would cost more in launches than in work at this size.
constexpr int kSmallThreads = 1024;
constexpr int kSmallLoads = 8;                                   // 16-byte loads in flight per thread
constexpr int64_t kSmallMax = 4 * kSmallThreads * kSmallLoads * 4;   // elements: up to 4 rounds of loads per thread

template <int T>
__global__ __launch_bounds__(kSmallThreads) void quantize_dynamic_small_kernel(const f4* __restrict__ x4,
                                                                               uint32_t* __restrict__ q4, int n4,
                                                                               float* __restrict__ state, int mode,
                                                                               float ensure_minimum_range) {
  __shared__ float red[2 * (kSmallThreads / 64)];
  __shared__ float params[2];
  float mn = __builtin_inff(), mx = -__builtin_inff();
  for (int base = threadIdx.x; base < n4; base += kSmallThreads * kSmallLoads) {
    f4 v[kSmallLoads];
#pragma unroll
    for (int j = 0; j < kSmallLoads; ++j) {
      const int i = base + j * kSmallThreads;
      if (i < n4) v[j] = x4[i];
    }
#pragma unroll
    for (int j = 0; j < kSmallLoads; ++j) {
      if (base + j * kSmallThreads < n4) {
        mn = fminf(fminf(mn, v[j].x), fminf(v[j].y, fminf(v[j].z, v[j].w)));
        mx = fmaxf(fmaxf(mx, v[j].x), fmaxf(v[j].y, fmaxf(v[j].z, v[j].w)));
      }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, o, 64));
    mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    red[2 * wave] = mn;
    red[2 * wave + 1] = mx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kSmallThreads / 64; ++w) {
      mn = fminf(mn, red[2 * w]);
      mx = fmaxf(mx, red[2 * w + 1]);
    }
    const DynamicParams p = dynamic_params(mn, mx, T, mode, ensure_minimum_range);
    params[0] = p.scale;
    params[1] = p.addend;
    if (blockIdx.x == 0) {
      state[0] = mn;
      state[1] = mx;
      state[2] = p.out_min;
      state[3] = p.out_max;
      state[4] = p.scale;
      state[5] = p.addend;
    }
  }
  __syncthreads();
  const float scale = params[0], addend = params[1];
  const int per = (n4 + gridDim.x - 1) / gridDim.x;
  const int end = min(n4, static_cast<int>(blockIdx.x + 1) * per);
  for (int i = blockIdx.x * per + threadIdx.x; i < end; i += kSmallThreads) q4[i] = quantize4<T>(x4[i], scale, addend);
}

// Per-row (per-token) form: workgroup m reduces row m, derives its parameters and quantizes it; the rows' output
// ranges go to two device arrays (what itexhip_qmatmul_per_row takes).
constexpr int kRowThreads = 1024;

template <int T>
__global__ __launch_bounds__(kRowThreads) void quantize_dynamic_rows_kernel(const float* __restrict__ x,
                                                                            uint8_t* __restrict__ q, int cols, int vec,
                                                                            float* __restrict__ row_min,
                                                                            float* __restrict__ row_max, int mode,
                                                                            float ensure_minimum_range) {
  __shared__ float red[2 * (kRowThreads / 64)];
  __shared__ float params[2];
  const float* xr = x + static_cast<int64_t>(blockIdx.x) * cols;
  uint8_t* qr = q + static_cast<int64_t>(blockIdx.x) * cols;
  float mn = __builtin_inff(), mx = -__builtin_inff();
  if (vec) {
    const f4* x4 = reinterpret_cast<const f4*>(xr);
    for (int i = threadIdx.x; i < cols / 4; i += kRowThreads) {
      const f4 v = x4[i];
      mn = fminf(fminf(mn, v.x), fminf(v.y, fminf(v.z, v.w)));
      mx = fmaxf(fmaxf(mx, v.x), fmaxf(v.y, fmaxf(v.z, v.w)));
    }
  } else {
    for (int i = threadIdx.x; i < cols; i += kRowThreads) {
      mn = fminf(mn, xr[i]);
      mx = fmaxf(mx, xr[i]);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, o, 64));
    mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  }
  if ((threadIdx.x & 63) == 0) {
    red[2 * (threadIdx.x >> 6)] = mn;
    red[2 * (threadIdx.x >> 6) + 1] = mx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kRowThreads / 64; ++w) {
      mn = fminf(mn, red[2 * w]);
      mx = fmaxf(mx, red[2 * w + 1]);
    }
    const DynamicParams p = dynamic_params(mn, mx, T, mode, ensure_minimum_range);
    params[0] = p.scale;
    params[1] = p.addend;
    row_min[blockIdx.x] = p.out_min;
    row_max[blockIdx.x] = p.out_max;
  }
  __syncthreads();
  const float scale = params[0], addend = params[1];
  if (vec) {
    const f4* x4 = reinterpret_cast<const f4*>(xr);
    uint32_t* q4 = reinterpret_cast<uint32_t*>(qr);
    for (int i = threadIdx.x; i < cols / 4; i += kRowThreads) q4[i] = quantize4<T>(x4[i], scale, addend);
  } else {
    for (int i = threadIdx.x; i < cols; i += kRowThreads) {
      const float t = xr[i] * scale;
      qr[i] = static_cast<uint8_t>(sat_rne<T>(t + addend));
    }
  }
}

// Second half of the two-launch form for larger tensors: every workgroup reduces the partial ranges the reduction
// left behind the state (at most kReduceBlocks pairs), derives the parameters, and quantizes its share; workgroup 0
// also leaves the state and quantizes the last n % 4 elements.
template <int T>
__global__ __launch_bounds__(kThreads) void quantize_dynamic_finish_kernel(const f4* __restrict__ x4, uint32_t* __restrict__ q4,
                                                                           int64_t n4, const float* __restrict__ xtail,
                                                                           uint8_t* __restrict__ qtail, int ntail,
                                                                           float* __restrict__ state,
                                                                           const float* __restrict__ partials, int n_partials,
                                                                           int mode, float ensure_minimum_range) {
  __shared__ float params[2];
  float mn = __builtin_inff(), mx = -__builtin_inff();
  for (int i = threadIdx.x; i < n_partials; i += kThreads) {
    mn = fminf(mn, partials[2 * i]);
    mx = fmaxf(mx, partials[2 * i + 1]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, o, 64));
    mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  }
  block_minmax_commit(
      mn, mx, [](float p, float q) { return p < q; },
      [&](float lo, float hi) {
        const DynamicParams p = dynamic_params(lo, hi, T, mode, ensure_minimum_range);
        params[0] = p.scale;
        params[1] = p.addend;
        if (blockIdx.x == 0) {
          state[0] = lo;
          state[1] = hi;
          state[2] = p.out_min;
          state[3] = p.out_max;
          state[4] = p.scale;
          state[5] = p.addend;
        }
      });
  __syncthreads();
  const float scale = params[0], addend = params[1];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
  f4 v[kUnroll];
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const int64_t i = base + j * kThreads;
    if (i < n4) v[j] = __builtin_nontemporal_load(&x4[i]);
  }
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const int64_t i = base + j * kThreads;
    if (i < n4) store_through(&q4[i], quantize4<T>(v[j], scale, addend));
  }
  if (blockIdx.x == 0 && static_cast<int>(threadIdx.x) < ntail) {
    const float t = xtail[threadIdx.x] * scale;
    qtail[threadIdx.x] = static_cast<uint8_t>(sat_rne<T>(t + addend));
  }
}

int launch_quantize(const char* who, const float* x, void* q, int64_t n, int dst_type, float scale, float addend,
                    const float* dev_params, hipStream_t st) {
  int64_t done = 0;
  if (aligned(x, 16) && aligned(q, 4) && n >= 4) {
    const int64_t n4 = n / 4;
    const unsigned grid = blocks_for(n4, kThreads * kNarrowSteps);
    if (dst_type == ITEXHIP_QINT8)
      quantize_vec_kernel<ITEXHIP_QINT8><<<grid, kThreads, 0, st>>>(
          reinterpret_cast<const f4*>(x), reinterpret_cast<uint32_t*>(q), n4, scale, addend, dev_params);
    else
      quantize_vec_kernel<ITEXHIP_QUINT8><<<grid, kThreads, 0, st>>>(
          reinterpret_cast<const f4*>(x), reinterpret_cast<uint32_t*>(q), n4, scale, addend, dev_params);
    done = n4 * 4;
  }
  if (done < n) {
    const unsigned grid = blocks_for(n - done, kThreads);
    if (dst_type == ITEXHIP_QINT8)
      quantize_scalar_kernel<ITEXHIP_QINT8><<<grid, kThreads, 0, st>>>(
          x, reinterpret_cast<uint8_t*>(q), done, n, scale, addend, dev_params);
    else
      quantize_scalar_kernel<ITEXHIP_QUINT8><<<grid, kThreads, 0, st>>>(
          x, reinterpret_cast<uint8_t*>(q), done, n, scale, addend, dev_params);
  }
  ITEXHIP_CHECK_LAUNCH(who);
  return ITEXHIP_OK;
}
}  // namespace
}  // namespace itexhip

using namespace itexhip;

extern "C" int itexhip_quantize(const float* x, void* q, int64_t n, int dst_type, float scale,
                                float addend, void* stream) {
  ITEXHIP_REQUIRE(dst_type == ITEXHIP_QINT8 || dst_type == ITEXHIP_QUINT8,
                  "itexhip_quantize: dst_type must be qint8 or quint8, got %d", dst_type);
  ITEXHIP_REQUIRE(n >= 0, "itexhip_quantize: negative size");
  if (n == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(x && q, "itexhip_quantize: null buffer");
  return launch_quantize("itexhip_quantize", x, q, n, dst_type, scale, addend, nullptr, as_stream(stream));
}

extern "C" int itexhip_quantize_dynamic(const float* x, void* q, int64_t n, int dst_type, int mode,
                                        float ensure_minimum_range, float* state, void* stream) {
  ITEXHIP_REQUIRE(dst_type == ITEXHIP_QINT8 || dst_type == ITEXHIP_QUINT8,
                  "itexhip_quantize_dynamic: dst_type must be qint8 or quint8, got %d", dst_type);
  ITEXHIP_REQUIRE(mode == ITEXHIP_SCALED || mode == ITEXHIP_MIN_FIRST_CLASSIC || (mode == ITEXHIP_MIN_FIRST && dst_type == ITEXHIP_QUINT8),
                  "itexhip_quantize_dynamic: SCALED, MIN_FIRST_CLASSIC, or MIN_FIRST to quint8");
  ITEXHIP_REQUIRE(n > 0, "itexhip_quantize_dynamic: an empty tensor has no range");
  ITEXHIP_REQUIRE(x && q && state && aligned(state, 8), "itexhip_quantize_dynamic: null or unaligned buffer");
  if (n <= kSmallMax && n % 4 == 0 && aligned(x, 16) && aligned(q, 4)) {
    const int n4 = static_cast<int>(n / 4);
    const unsigned grid = static_cast<unsigned>(std::min<int64_t>(16, (n4 + kSmallThreads - 1) / kSmallThreads));
    if (dst_type == ITEXHIP_QINT8)
      quantize_dynamic_small_kernel<ITEXHIP_QINT8><<<grid, kSmallThreads, 0, as_stream(stream)>>>(
          reinterpret_cast<const f4*>(x), reinterpret_cast<uint32_t*>(q), n4, state, mode, ensure_minimum_range);
    else
      quantize_dynamic_small_kernel<ITEXHIP_QUINT8><<<grid, kSmallThreads, 0, as_stream(stream)>>>(
          reinterpret_cast<const f4*>(x), reinterpret_cast<uint32_t*>(q), n4, state, mode, ensure_minimum_range);
    ITEXHIP_CHECK_LAUNCH("itexhip_quantize_dynamic");
    return ITEXHIP_OK;
  }
  if (aligned(x, 16) && aligned(q, 4) && n >= 4) {  // two launches: partial ranges, then parameters + quantization
    hipStream_t st = as_stream(stream);
    const int64_t n4 = n / 4;
    const int ntail = static_cast<int>(n - n4 * 4);
    const unsigned g1 = static_cast<unsigned>(std::min<int64_t>(
        kReduceBlocks, std::max<int64_t>(1, (n4 + kThreads * kReduceUnroll - 1) / (kThreads * kReduceUnroll))));
    minmax_f32_kernel<true><<<g1, kThreads, 0, st>>>(reinterpret_cast<const f4*>(x), n4, x + n4 * 4, ntail,
                                                     reinterpret_cast<int*>(state + 8));
    const unsigned g2 = blocks_for(n4, kThreads * kUnroll);
    if (dst_type == ITEXHIP_QINT8)
      quantize_dynamic_finish_kernel<ITEXHIP_QINT8><<<g2, kThreads, 0, st>>>(
          reinterpret_cast<const f4*>(x), reinterpret_cast<uint32_t*>(q), n4, x + n4 * 4,
          reinterpret_cast<uint8_t*>(q) + n4 * 4, ntail, state, state + 8, static_cast<int>(g1), mode, ensure_minimum_range);
    else
      quantize_dynamic_finish_kernel<ITEXHIP_QUINT8><<<g2, kThreads, 0, st>>>(
          reinterpret_cast<const f4*>(x), reinterpret_cast<uint32_t*>(q), n4, x + n4 * 4,
          reinterpret_cast<uint8_t*>(q) + n4 * 4, ntail, state, state + 8, static_cast<int>(g1), mode, ensure_minimum_range);
    ITEXHIP_CHECK_LAUNCH("itexhip_quantize_dynamic");
    return ITEXHIP_OK;
  }
  enqueue_minmax_f32(x, n, reinterpret_cast<int*>(state), as_stream(stream));
  quantize_dynamic_params_kernel<<<1, 1, 0, as_stream(stream)>>>(state, dst_type, mode, ensure_minimum_range);
  return launch_quantize("itexhip_quantize_dynamic", x, q, n, dst_type, 0.0f, 0.0f, state + 4, as_stream(stream));
}

extern "C" int itexhip_quantize_dynamic_rows(const float* x, void* q, int64_t rows, int64_t cols, int dst_type, int mode,
                                             float ensure_minimum_range, float* row_min_out, float* row_max_out,
                                             void* stream) {
  ITEXHIP_REQUIRE(dst_type == ITEXHIP_QINT8 || dst_type == ITEXHIP_QUINT8,
                  "itexhip_quantize_dynamic_rows: dst_type must be qint8 or quint8, got %d", dst_type);
  ITEXHIP_REQUIRE(mode == ITEXHIP_SCALED || mode == ITEXHIP_MIN_FIRST_CLASSIC || (mode == ITEXHIP_MIN_FIRST && dst_type == ITEXHIP_QUINT8),
                  "itexhip_quantize_dynamic_rows: SCALED, MIN_FIRST_CLASSIC, or MIN_FIRST to quint8");
  ITEXHIP_REQUIRE(rows >= 0 && rows < (1LL << 31) && cols > 0 && cols < (1LL << 31),
                  "itexhip_quantize_dynamic_rows: bad shape (an empty row has no range)");
  if (rows == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(x && q && row_min_out && row_max_out, "itexhip_quantize_dynamic_rows: null buffer");
  const int vec = cols % 4 == 0 && aligned(x, 16) && aligned(q, 4);
  const unsigned grid = static_cast<unsigned>(rows);
  if (dst_type == ITEXHIP_QINT8)
    quantize_dynamic_rows_kernel<ITEXHIP_QINT8><<<grid, kRowThreads, 0, as_stream(stream)>>>(
        x, reinterpret_cast<uint8_t*>(q), static_cast<int>(cols), vec, row_min_out, row_max_out, mode, ensure_minimum_range);
  else
    quantize_dynamic_rows_kernel<ITEXHIP_QUINT8><<<grid, kRowThreads, 0, as_stream(stream)>>>(
        x, reinterpret_cast<uint8_t*>(q), static_cast<int>(cols), vec, row_min_out, row_max_out, mode, ensure_minimum_range);
  ITEXHIP_CHECK_LAUNCH("itexhip_quantize_dynamic_rows");
  return ITEXHIP_OK;
}

extern "C" int itexhip_quantize_axis(const float* x, void* q, int64_t outer, int64_t slices,
                                     int64_t inner, int dst_type, const float* scales,
                                     const float* addends, void* stream) {
  ITEXHIP_REQUIRE(dst_type == ITEXHIP_QINT8 || dst_type == ITEXHIP_QUINT8,
                  "itexhip_quantize_axis: dst_type must be qint8 or quint8, got %d", dst_type);
  ITEXHIP_REQUIRE(outer >= 0 && slices >= 0 && inner >= 0, "itexhip_quantize_axis: negative size");
  const int64_t n = outer * slices * inner;
  if (n == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(x && q && scales, "itexhip_quantize_axis: null buffer");
  // 4 elements per lane when a group of 4 never straddles two slices in a way one 16-byte parameter load cannot follow
  const bool last = inner == 1 && slices % 4 == 0 && aligned(scales, 16) && (!addends || aligned(addends, 16));
  if ((last || inner % 4 == 0) && aligned(x, 16) && aligned(q, 4) && n / 4 < (1LL << 31) && slices < (1LL << 31)) {
    const uint32_t n4 = static_cast<uint32_t>(n / 4), sl = static_cast<uint32_t>(slices), in4 = static_cast<uint32_t>(inner / 4);
    const unsigned vgrid = blocks_for(n4, kThreads * kNarrowSteps);
    const f4* xv = reinterpret_cast<const f4*>(x);
    uint32_t* qv = reinterpret_cast<uint32_t*>(q);
    hipStream_t st = as_stream(stream);
    if (dst_type == ITEXHIP_QINT8) {
      if (last) quantize_axis_vec_kernel<ITEXHIP_QINT8, true><<<vgrid, kThreads, 0, st>>>(xv, qv, n4, sl, in4, scales, addends);
      else quantize_axis_vec_kernel<ITEXHIP_QINT8, false><<<vgrid, kThreads, 0, st>>>(xv, qv, n4, sl, in4, scales, addends);
    } else {
      if (last) quantize_axis_vec_kernel<ITEXHIP_QUINT8, true><<<vgrid, kThreads, 0, st>>>(xv, qv, n4, sl, in4, scales, addends);
      else quantize_axis_vec_kernel<ITEXHIP_QUINT8, false><<<vgrid, kThreads, 0, st>>>(xv, qv, n4, sl, in4, scales, addends);
    }
    ITEXHIP_CHECK_LAUNCH("itexhip_quantize_axis");
    return ITEXHIP_OK;
  }
  const unsigned grid = blocks_for(n, kThreads);
  if (dst_type == ITEXHIP_QINT8)
    quantize_axis_kernel<ITEXHIP_QINT8><<<grid, kThreads, 0, as_stream(stream)>>>(
        x, reinterpret_cast<uint8_t*>(q), n, slices, inner, scales, addends);
  else
    quantize_axis_kernel<ITEXHIP_QUINT8><<<grid, kThreads, 0, as_stream(stream)>>>(
        x, reinterpret_cast<uint8_t*>(q), n, slices, inner, scales, addends);
  ITEXHIP_CHECK_LAUNCH("itexhip_quantize_axis");
  return ITEXHIP_OK;
}

extern "C" int itexhip_dequantize(const void* q, float* y, int64_t n, int src_type, float scale,
                                  int32_t zero_point, void* stream) {
  ITEXHIP_REQUIRE(src_type == ITEXHIP_QINT8 || src_type == ITEXHIP_QUINT8,
                  "itexhip_dequantize: src_type must be qint8 or quint8, got %d", src_type);
  ITEXHIP_REQUIRE(n >= 0, "itexhip_dequantize: negative size");
  if (n == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(q && y, "itexhip_dequantize: null buffer");
  hipStream_t st = as_stream(stream);
  const float zp = static_cast<float>(zero_point);
  int64_t done = 0;
  if (aligned(q, 4) && aligned(y, 16) && n >= 4) {
    const int64_t n4 = n / 4;
    const unsigned grid = blocks_for(n4, kThreads * kWidenUnroll);
    if (src_type == ITEXHIP_QINT8)
      dequantize_vec_kernel<ITEXHIP_QINT8><<<grid, kThreads, 0, st>>>(
          reinterpret_cast<const uint32_t*>(q), reinterpret_cast<f4*>(y), n4, scale, zp);
    else
      dequantize_vec_kernel<ITEXHIP_QUINT8><<<grid, kThreads, 0, st>>>(
          reinterpret_cast<const uint32_t*>(q), reinterpret_cast<f4*>(y), n4, scale, zp);
    done = n4 * 4;
  }
  if (done < n) {
    const unsigned grid = blocks_for(n - done, kThreads);
    if (src_type == ITEXHIP_QINT8)
      dequantize_axis_kernel<ITEXHIP_QINT8><<<grid, kThreads, 0, st>>>(
          reinterpret_cast<const uint8_t*>(q), y, done, n, 1, 1, nullptr, nullptr, scale, zp);
    else
      dequantize_axis_kernel<ITEXHIP_QUINT8><<<grid, kThreads, 0, st>>>(
          reinterpret_cast<const uint8_t*>(q), y, done, n, 1, 1, nullptr, nullptr, scale, zp);
  }
  ITEXHIP_CHECK_LAUNCH("itexhip_dequantize");
  return ITEXHIP_OK;
}

extern "C" int itexhip_dequantize_axis(const void* q, float* y, int64_t outer, int64_t slices,
                                       int64_t inner, int src_type, const float* scales,
                                       const int32_t* zero_points, void* stream) {
  ITEXHIP_REQUIRE(src_type == ITEXHIP_QINT8 || src_type == ITEXHIP_QUINT8,
                  "itexhip_dequantize_axis: src_type must be qint8 or quint8, got %d", src_type);
  ITEXHIP_REQUIRE(outer >= 0 && slices >= 0 && inner >= 0, "itexhip_dequantize_axis: negative size");
  const int64_t n = outer * slices * inner;
  if (n == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(q && y && scales, "itexhip_dequantize_axis: null buffer");
  const bool last = inner == 1 && slices % 4 == 0 && aligned(scales, 16) && (!zero_points || aligned(zero_points, 16));
  if ((last || inner % 4 == 0) && aligned(q, 4) && aligned(y, 16) && n / 4 < (1LL << 31) && slices < (1LL << 31)) {
    const uint32_t n4 = static_cast<uint32_t>(n / 4), sl = static_cast<uint32_t>(slices), in4 = static_cast<uint32_t>(inner / 4);
    const unsigned vgrid = blocks_for(n4, kThreads);
    const uint32_t* qv = reinterpret_cast<const uint32_t*>(q);
    f4* yv = reinterpret_cast<f4*>(y);
    hipStream_t st = as_stream(stream);
    if (src_type == ITEXHIP_QINT8) {
      if (last) dequantize_axis_vec_kernel<ITEXHIP_QINT8, true><<<vgrid, kThreads, 0, st>>>(qv, yv, n4, sl, in4, scales, zero_points);
      else dequantize_axis_vec_kernel<ITEXHIP_QINT8, false><<<vgrid, kThreads, 0, st>>>(qv, yv, n4, sl, in4, scales, zero_points);
    } else {
      if (last) dequantize_axis_vec_kernel<ITEXHIP_QUINT8, true><<<vgrid, kThreads, 0, st>>>(qv, yv, n4, sl, in4, scales, zero_points);
      else dequantize_axis_vec_kernel<ITEXHIP_QUINT8, false><<<vgrid, kThreads, 0, st>>>(qv, yv, n4, sl, in4, scales, zero_points);
    }
    ITEXHIP_CHECK_LAUNCH("itexhip_dequantize_axis");
    return ITEXHIP_OK;
  }
  const unsigned grid = blocks_for(n, kThreads);
  if (src_type == ITEXHIP_QINT8)
    dequantize_axis_kernel<ITEXHIP_QINT8><<<grid, kThreads, 0, as_stream(stream)>>>(
        reinterpret_cast<const uint8_t*>(q), y, 0, n, slices, inner, scales, zero_points, 0.f, 0.f);
  else
    dequantize_axis_kernel<ITEXHIP_QUINT8><<<grid, kThreads, 0, as_stream(stream)>>>(
        reinterpret_cast<const uint8_t*>(q), y, 0, n, slices, inner, scales, zero_points, 0.f, 0.f);
  ITEXHIP_CHECK_LAUNCH("itexhip_dequantize_axis");
  return ITEXHIP_OK;
}

namespace {
template <int T>
int requantize_impl(const int32_t* x, void* q, int64_t n, int64_t depth, float scale,
                    const float* scales, hipStream_t st) {
  int64_t done = 0;
  const bool vec_ok = aligned(x, 16) && aligned(q, 4) && n >= 4;
  if (vec_ok && scales == nullptr) {
    const int64_t n4 = n / 4;
    requantize_vec_kernel<T, 0><<<blocks_for(n4, kThreads * kNarrowSteps), kThreads, 0, st>>>(
        reinterpret_cast<const i4*>(x), reinterpret_cast<uint32_t*>(q), n4, scale, nullptr, 1);
    done = n4 * 4;
  } else if (vec_ok && depth % 4 == 0 && aligned(scales, 16)) {
    const int64_t n4 = n / 4;  // n is a multiple of depth, hence of 4
    if (n4 < (1LL << 31))
      requantize_vec_kernel<T, 2><<<blocks_for(n4, kThreads * kNarrowSteps), kThreads, 0, st>>>(
          reinterpret_cast<const i4*>(x), reinterpret_cast<uint32_t*>(q), n4, 0.f, scales, depth / 4);
    else
      requantize_vec_kernel<T, 1><<<blocks_for(n4, kThreads * kNarrowSteps), kThreads, 0, st>>>(
          reinterpret_cast<const i4*>(x), reinterpret_cast<uint32_t*>(q), n4, 0.f, scales, depth / 4);
    done = n4 * 4;
  }
  if (done < n) {
    requantize_scalar_kernel<T><<<blocks_for(n - done, kThreads), kThreads, 0, st>>>(
        x, reinterpret_cast<uint8_t*>(q), done, n, depth, scale, scales);
  }
  ITEXHIP_CHECK_LAUNCH("itexhip_requantize");
  return ITEXHIP_OK;
}
}  // namespace

extern "C" int itexhip_requantize_per_channel(const int32_t* x, void* q, int64_t rows, int64_t depth,
                                              int dst_type, const float* scales, void* stream) {
  ITEXHIP_REQUIRE(dst_type == ITEXHIP_QINT8 || dst_type == ITEXHIP_QUINT8,
                  "itexhip_requantize_per_channel: dst_type must be qint8 or quint8, got %d", dst_type);
  ITEXHIP_REQUIRE(rows >= 0 && depth >= 0, "itexhip_requantize_per_channel: negative size");
  const int64_t n = rows * depth;
  if (n == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(x && q && scales, "itexhip_requantize_per_channel: null buffer");
  if (dst_type == ITEXHIP_QINT8)
    return requantize_impl<ITEXHIP_QINT8>(x, q, n, depth, 0.f, scales, as_stream(stream));
  return requantize_impl<ITEXHIP_QUINT8>(x, q, n, depth, 0.f, scales, as_stream(stream));
}

extern "C" int itexhip_requantize(const int32_t* x, void* q, int64_t n, int dst_type, float scale,
                                  void* stream) {
  ITEXHIP_REQUIRE(dst_type == ITEXHIP_QINT8 || dst_type == ITEXHIP_QUINT8,
                  "itexhip_requantize: dst_type must be qint8 or quint8, got %d", dst_type);
  ITEXHIP_REQUIRE(n >= 0, "itexhip_requantize: negative size");
  if (n == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(x && q, "itexhip_requantize: null buffer");
  if (dst_type == ITEXHIP_QINT8)
    return requantize_impl<ITEXHIP_QINT8>(x, q, n, 1, scale, nullptr, as_stream(stream));
  return requantize_impl<ITEXHIP_QUINT8>(x, q, n, 1, scale, nullptr, as_stream(stream));
}

extern "C" int itexhip_minmax_i32_per_channel(const int32_t* x, int64_t rows, int64_t depth,
                                              int32_t* min_out, int32_t* max_out, void* stream) {
  ITEXHIP_REQUIRE(rows >= 0 && depth >= 0, "itexhip_minmax_i32_per_channel: negative size");
  if (depth == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(min_out && max_out, "itexhip_minmax_i32_per_channel: null output");
  hipStream_t st = as_stream(stream);
  fill_minmax_i32_kernel<<<blocks_for(depth, 256), 256, 0, st>>>(min_out, max_out, depth);
  if (rows > 0) {
    ITEXHIP_REQUIRE(x, "itexhip_minmax_i32_per_channel: null input");
    if (depth == 1) {
      const bool vec = aligned(x, 16);
      const int64_t n4 = vec ? rows / 4 : 0;
      const int ntail = static_cast<int>(rows - n4 * 4);
      if (vec) {
        const unsigned grid = static_cast<unsigned>(std::min<int64_t>(
            kReduceBlocks, std::max<int64_t>(1, (n4 + kThreads * kReduceUnroll - 1) / (kThreads * kReduceUnroll))));
        minmax_i32_flat_kernel<<<grid, kThreads, 0, st>>>(reinterpret_cast<const i4*>(x), n4,
                                                          x + n4 * 4, ntail, min_out, max_out);
      } else {
        const int64_t rpb = 4096;
        dim3 grid(blocks_for(rows, rpb), 1);
        minmax_i32_channel_kernel<<<grid, kThreads, 0, st>>>(x, rows, 1, rpb, min_out, max_out);
      }
    } else {
      // enough row chunks to occupy the device, at least 64 rows each
      const int64_t col_blocks = (depth + kThreads - 1) / kThreads;
      int64_t row_blocks = std::max<int64_t>(1, 4096 / col_blocks);
      int64_t rpb = std::max<int64_t>(64, (rows + row_blocks - 1) / row_blocks);
      row_blocks = (rows + rpb - 1) / rpb;
      ITEXHIP_REQUIRE(col_blocks <= 65535, "itexhip_minmax_i32_per_channel: depth too large");
      dim3 grid(static_cast<unsigned>(row_blocks), static_cast<unsigned>(col_blocks));
      minmax_i32_channel_kernel<<<grid, kThreads, 0, st>>>(x, rows, depth, rpb, min_out, max_out);
    }
  }
  ITEXHIP_CHECK_LAUNCH("itexhip_minmax_i32_per_channel");
  return ITEXHIP_OK;
}

extern "C" int itexhip_minmax_f32(const float* x, int64_t n, float* minmax_out, void* stream) {
  ITEXHIP_REQUIRE(n >= 0, "itexhip_minmax_f32: negative size");
  ITEXHIP_REQUIRE(minmax_out, "itexhip_minmax_f32: null output");
  hipStream_t st = as_stream(stream);
  int* keys = reinterpret_cast<int*>(minmax_out);
  if (n > 0) {
    ITEXHIP_REQUIRE(x, "itexhip_minmax_f32: null input");
    enqueue_minmax_f32(x, n, keys, st);
  } else {
    fill_minmax_f32_kernel<<<1, 1, 0, st>>>(keys);
  }
  finish_minmax_f32_kernel<<<1, 1, 0, st>>>(keys);
  ITEXHIP_CHECK_LAUNCH("itexhip_minmax_f32");
  return ITEXHIP_OK;
}

extern "C" int itexhip_memcpy_d2d_async(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(dst && src, "itexhip_memcpy_d2d_async: null buffer");
  hipStream_t st = as_stream(stream);
  int64_t done = 0;
  const int64_t n = static_cast<int64_t>(bytes);
  if (aligned(src, 16) && aligned(dst, 16) && n >= 16) {
    const int64_t n16 = n / 16;
    copy_vec_kernel<<<blocks_for(n16, kThreads * kUnroll), kThreads, 0, st>>>(
        reinterpret_cast<const i4*>(src), reinterpret_cast<i4*>(dst), n16);
    done = n16 * 16;
  }
  if (done < n)
    copy_byte_kernel<<<blocks_for(n - done, kThreads), kThreads, 0, st>>>(
        reinterpret_cast<const uint8_t*>(src), reinterpret_cast<uint8_t*>(dst), done, n);
  ITEXHIP_CHECK_LAUNCH("itexhip_memcpy_d2d_async");
  return ITEXHIP_OK;
}

extern "C" int itexhip_read_probe(const void* src, size_t bytes, int32_t* sink, void* stream) {
  ITEXHIP_REQUIRE(src && sink && aligned(src, 16) && bytes >= 16384, "itexhip_read_probe: 16-byte aligned buffer of at least 16 KiB");
  const int64_t n16 = static_cast<int64_t>(bytes / 16);
  const unsigned grid = static_cast<unsigned>(std::min<int64_t>(1024, n16 / (kThreads * kUnroll)));
  read_probe_kernel<<<grid, kThreads, 0, as_stream(stream)>>>(reinterpret_cast<const i4*>(src), n16, sink);
  ITEXHIP_CHECK_LAUNCH("itexhip_read_probe");
  return ITEXHIP_OK;
}

// ------------------------------------------------------------------------------------------------
// itexhip_quantize_dynamic for callers that cannot allocate (HIP graph capture, serving loops): the partial
// ranges of the reduction's workgroups live in a fixed array of the library's own device memory instead of a
// workspace argument.  Every GPU holds its own copy of the array at its own address, resolved once per device.
// ------------------------------------------------------------------------------------------------
namespace itexhip {
namespace {
// one {min, max} pair per workgroup of the range pass, kReduceBlocks of them at most whatever the tensor's size
static __device__ __align__(256) float scratch[2 * kReduceBlocks];

constexpr int kMaxDevices = 64;
constexpr int64_t kStaticMaxElements = int64_t{1} << 36;  // 256 GiB of fp32: more than a device holds beside its result

// the device address of `scratch` on the current device (the array's name is only a host-side handle)
int scratch_address(float** out) {
  static float* ptrs[kMaxDevices] = {};
  static std::mutex mu;
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return hip_fail(err, "hipGetDevice");
  ITEXHIP_REQUIRE(dev >= 0 && dev < kMaxDevices, "itexhip_quantize_dynamic_static: device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (ptrs[dev] == nullptr) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return hip_fail(err, "hipGetSymbolAddress(scratch)");
    ptrs[dev] = static_cast<float*>(p);
  }
  *out = ptrs[dev];
  return ITEXHIP_OK;
}
}  // namespace
}  // namespace itexhip

extern "C" int itexhip_quantize_dynamic_static(const float* x, void* q, int64_t n, int dst_type, int mode,
                                               float ensure_minimum_range, float* range_out, void* stream) {
  const char* who = "itexhip_quantize_dynamic_static";
  ITEXHIP_REQUIRE(dst_type == ITEXHIP_QINT8 || dst_type == ITEXHIP_QUINT8, "%s: dst_type must be qint8 or quint8, got %d", who, dst_type);
  ITEXHIP_REQUIRE(mode == ITEXHIP_SCALED || mode == ITEXHIP_MIN_FIRST_CLASSIC || (mode == ITEXHIP_MIN_FIRST && dst_type == ITEXHIP_QUINT8),
                  "%s: SCALED, MIN_FIRST_CLASSIC, or MIN_FIRST to quint8", who);
  ITEXHIP_REQUIRE(n >= 4, "%s: at least 4 elements (got %lld)", who, static_cast<long long>(n));
  ITEXHIP_REQUIRE(n <= kStaticMaxElements, "%s: at most 2^36 elements (got %lld)", who, static_cast<long long>(n));
  ITEXHIP_REQUIRE(x && q && range_out, "%s: null buffer", who);
  ITEXHIP_REQUIRE(aligned(x, 16) && aligned(q, 4) && aligned(range_out, 8),
                  "%s: x must be 16-byte, q 4-byte and range_out 8-byte aligned", who);
  float* partials = nullptr;
  if (int st = scratch_address(&partials)) return st;
  hipStream_t st = as_stream(stream);
  const int64_t n4 = n / 4;
  const int ntail = static_cast<int>(n - n4 * 4);
  // every workgroup of the range pass overwrites its own pair, and the second kernel reads exactly those: nothing
  // in the array has to be cleared between calls
  const unsigned g1 = static_cast<unsigned>(std::min<int64_t>(
      kReduceBlocks, std::max<int64_t>(1, (n4 + kThreads * kReduceUnroll - 1) / (kThreads * kReduceUnroll))));
  minmax_f32_kernel<true><<<g1, kThreads, 0, st>>>(reinterpret_cast<const f4*>(x), n4, x + n4 * 4, ntail,
                                                   reinterpret_cast<int*>(partials));
  const unsigned g2 = blocks_for(n4, kThreads * kUnroll);
  if (dst_type == ITEXHIP_QINT8)
    quantize_dynamic_finish_kernel<ITEXHIP_QINT8><<<g2, kThreads, 0, st>>>(
        reinterpret_cast<const f4*>(x), reinterpret_cast<uint32_t*>(q), n4, x + n4 * 4, reinterpret_cast<uint8_t*>(q) + n4 * 4,
        ntail, range_out, partials, static_cast<int>(g1), mode, ensure_minimum_range);
  else
    quantize_dynamic_finish_kernel<ITEXHIP_QUINT8><<<g2, kThreads, 0, st>>>(
        reinterpret_cast<const f4*>(x), reinterpret_cast<uint32_t*>(q), n4, x + n4 * 4, reinterpret_cast<uint8_t*>(q) + n4 * 4,
        ntail, range_out, partials, static_cast<int>(g1), mode, ensure_minimum_range);
  ITEXHIP_CHECK_LAUNCH(who);
  return ITEXHIP_OK;
}
