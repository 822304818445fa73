// Device helpers of the quantized Conv2D ops (itex/core/kernels/common/quantized_conv_ops.h): the patch
// matrix that turns the convolution into the quantized GEMM of qgemm.hip, and the bias scaling.
#include <algorithm>

#include "common.hpp"

namespace itexhip {
namespace {

struct Im2colArgs {
  itexhip_conv_geometry g;
  int64_t row_dwords;   // row_bytes / 4
  int64_t total;        // dwords of the whole matrix
  int K;                // k_h * k_w * in_c
  int vec;              // in_c % 4 == 0 and the input is 4-byte aligned: a dword never straddles a pixel
};

// One dword (4 consecutive k of one row) per thread and iteration.
__global__ __launch_bounds__(256) void im2col8_kernel(const Im2colArgs a, const uint8_t* __restrict__ x,
                                                      uint32_t* __restrict__ cols) {
  const itexhip_conv_geometry& g = a.g;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < a.total; i += stride) {
    const int64_t row = i / a.row_dwords;
    const int k0 = static_cast<int>(i - row * a.row_dwords) * 4;
    const int64_t ow = row % g.out_w, t = row / g.out_w;
    const int64_t oh = t % g.out_h, b = t / g.out_h;
    uint32_t v = 0;
    if (a.vec) {
      if (k0 < a.K) {
        const int c = k0 % static_cast<int>(g.in_c), kk = k0 / static_cast<int>(g.in_c);
        const int kw = kk % static_cast<int>(g.k_w), kh = kk / static_cast<int>(g.k_w);
        const int64_t ih = oh * g.stride_h - g.pad_top + static_cast<int64_t>(kh) * g.dil_h;
        const int64_t iw = ow * g.stride_w - g.pad_left + static_cast<int64_t>(kw) * g.dil_w;
        if (ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w)
          v = *reinterpret_cast<const uint32_t*>(x + ((b * g.in_h + ih) * g.in_w + iw) * g.in_c + c);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int k = k0 + e;
        if (k >= a.K) break;
        const int c = k % static_cast<int>(g.in_c), kk = k / static_cast<int>(g.in_c);
        const int kw = kk % static_cast<int>(g.k_w), kh = kk / static_cast<int>(g.k_w);
        const int64_t ih = oh * g.stride_h - g.pad_top + static_cast<int64_t>(kh) * g.dil_h;
        const int64_t iw = ow * g.stride_w - g.pad_left + static_cast<int64_t>(kw) * g.dil_w;
        if (ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w)
          v |= static_cast<uint32_t>(x[((b * g.in_h + ih) * g.in_w + iw) * g.in_c + c]) << (8 * e);
      }
    }
    cols[i] = v;
  }
}

// Zero-padded copy of a 4-d tensor of bytes: out[n][h][w][c] = x[n][h - lead_h][w - lead_w][c] where that exists, else 0.
// One thread per 4 output bytes (out_c is a multiple of 4, so they belong to one pixel).
struct Pad4dArgs {
  int n, h, w, c, lead_h, lead_w, out_h, out_w, out_c;
  uint32_t total;  // output dwords
};
__global__ __launch_bounds__(256) void pad_nhwc8_kernel(const Pad4dArgs a, const uint8_t* __restrict__ x, uint32_t* __restrict__ out) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= a.total) return;
  const uint32_t per_pixel = static_cast<uint32_t>(a.out_c) >> 2;
  const uint32_t pixel = i / per_pixel, c0 = (i - pixel * per_pixel) * 4;
  const uint32_t row = pixel / static_cast<uint32_t>(a.out_w), ow = pixel - row * static_cast<uint32_t>(a.out_w);
  const uint32_t n = row / static_cast<uint32_t>(a.out_h), oh = row - n * static_cast<uint32_t>(a.out_h);
  const int ih = static_cast<int>(oh) - a.lead_h, iw = static_cast<int>(ow) - a.lead_w;
  uint32_t v = 0;
  if (ih >= 0 && ih < a.h && iw >= 0 && iw < a.w) {
    const uint8_t* src = x + ((static_cast<int64_t>(n) * a.h + ih) * a.w + iw) * a.c;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (static_cast<int>(c0) + e < a.c) v |= static_cast<uint32_t>(src[c0 + e]) << (8 * e);
  }
  out[i] = v;
}

// The same for out_c = 4 or 8 and out_w a multiple of 16 / out_c: one thread per 16 output bytes (4 or 2 pixels of one
// row), so the index decomposition is paid once per 16 bytes (the 4-byte form spent most of its time on it).
template <int OUT_C>
__global__ __launch_bounds__(256) void pad_nhwc8_vec_kernel(const Pad4dArgs a, const uint8_t* __restrict__ x, i4* __restrict__ out) {
  constexpr int PIX = 16 / OUT_C;
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;  // vector index
  if (i >= a.total / 4) return;
  const uint32_t per_row = static_cast<uint32_t>(a.out_w) / PIX;
  const uint32_t row = i / per_row, ow0 = (i - row * per_row) * PIX;
  const uint32_t n = row / static_cast<uint32_t>(a.out_h), oh = row - n * static_cast<uint32_t>(a.out_h);
  const int ih = static_cast<int>(oh) - a.lead_h;
  uint32_t v[4] = {0u, 0u, 0u, 0u};
  if (ih >= 0 && ih < a.h) {
    const uint8_t* src_row = x + (static_cast<int64_t>(n) * a.h + ih) * a.w * a.c;
#pragma unroll
    for (int p = 0; p < PIX; ++p) {
      const int iw = static_cast<int>(ow0) + p - a.lead_w;
      if (iw < 0 || iw >= a.w) continue;
      const uint8_t* src = src_row + static_cast<int64_t>(iw) * a.c;
#pragma unroll
      for (int e = 0; e < OUT_C; ++e)
        if (e < a.c) v[(p * OUT_C + e) >> 2] |= static_cast<uint32_t>(src[e]) << (8 * (e & 3));
    }
  }
  out[i] = i4{static_cast<int>(v[0]), static_cast<int>(v[1]), static_cast<int>(v[2]), static_cast<int>(v[3])};
}

// Few input channels (the first layer of a network: in_c = 3): every byte of a patch row may come from another pixel,
// so the window offsets are tabulated per byte of the row once per workgroup (LDS), a thread decomposes only its row
// index (32-bit), gathers its 4 bytes unconditionally from clamped positions and zeroes those in the padding.
constexpr int kMaxRowBytesTable = 2048;
__global__ __launch_bounds__(256) void im2col8_byte_kernel(const Im2colArgs a, const uint8_t* __restrict__ x,
                                                           uint32_t* __restrict__ cols) {
  __shared__ int t_dhw[kMaxRowBytesTable], t_off[kMaxRowBytesTable];  // (window row << 16 | window column), input byte offset
  const itexhip_conv_geometry& g = a.g;
  const int C = static_cast<int>(g.in_c), KW = static_cast<int>(g.k_w), W = static_cast<int>(g.in_w), H = static_cast<int>(g.in_h);
  const uint32_t row_dwords = static_cast<uint32_t>(a.row_dwords);
  for (uint32_t k = threadIdx.x; k < row_dwords * 4; k += blockDim.x) {
    if (static_cast<int>(k) < a.K) {
      const int c = k % C, kk = k / C, kw = kk % KW, kh = kk / KW;
      t_dhw[k] = ((kh * g.dil_h) << 16) | (kw * g.dil_w);
      t_off[k] = (kh * g.dil_h * W + kw * g.dil_w) * C + c;
    } else {
      t_dhw[k] = -1;  // zero tail of the row
      t_off[k] = 0;
    }
  }
  __syncthreads();
  const uint32_t total = static_cast<uint32_t>(a.total);  // dwords; the host keeps this and the input below 2^31
  const uint32_t OW = static_cast<uint32_t>(g.out_w), OH = static_cast<uint32_t>(g.out_h);
  const uint32_t stride = gridDim.x * blockDim.x;
  const int last = H * W * C * static_cast<int>(g.batch) - 1;
  for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const uint32_t row = i / row_dwords, k0 = (i - row * row_dwords) * 4;
    const uint32_t t = row / OW, ow = row - t * OW;
    const uint32_t b = t / OH, oh = t - b * OH;
    const int ih0 = static_cast<int>(oh) * g.stride_h - static_cast<int>(g.pad_top);
    const int iw0 = static_cast<int>(ow) * g.stride_w - static_cast<int>(g.pad_left);
    const int base = ((static_cast<int>(b) * H + ih0) * W + iw0) * C;
    uint32_t v = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int dhw = t_dhw[k0 + e];
      const int ih = ih0 + (dhw >> 16), iw = iw0 + (dhw & 0xffff);
      const bool ok = dhw >= 0 && ih >= 0 && ih < H && iw >= 0 && iw < W;
      const uint32_t byte = x[min(max(base + t_off[k0 + e], 0), last)];
      v |= (ok ? byte : 0u) << (8 * e);
    }
    cols[i] = v;
  }
}

// in_c a multiple of 16: every 16-byte vector of a patch row lies inside one input pixel.  The workgroup first
// tabulates, per vector of the row, its offset inside the window (rows / columns to add to the window origin,
// byte offset in the input), so that a thread only decomposes its row index.
constexpr int kMaxRowVectors = 1024;  // 16 KiB of receptive field per output position
__global__ __launch_bounds__(256) void im2col8_vec_kernel(const Im2colArgs a, const uint8_t* __restrict__ x,
                                                          i4* __restrict__ cols) {
  __shared__ int t_dh[kMaxRowVectors], t_dw[kMaxRowVectors], t_off[kMaxRowVectors];
  const itexhip_conv_geometry& g = a.g;
  const uint32_t row_vecs = static_cast<uint32_t>(a.row_dwords >> 2);
  const int C = static_cast<int>(g.in_c), KW = static_cast<int>(g.k_w), W = static_cast<int>(g.in_w);
  for (uint32_t u = threadIdx.x; u < row_vecs; u += blockDim.x) {
    const int k0 = static_cast<int>(u) * 16;
    if (k0 < a.K) {
      const int c = k0 % C, kk = k0 / C, kw = kk % KW, kh = kk / KW;
      t_dh[u] = kh * g.dil_h;
      t_dw[u] = kw * g.dil_w;
      t_off[u] = (kh * g.dil_h * W + kw * g.dil_w) * C + c;
    } else {
      t_dh[u] = -1;  // zero tail of the row
      t_dw[u] = 0;
      t_off[u] = 0;
    }
  }
  __syncthreads();
  const uint32_t total = static_cast<uint32_t>(a.total >> 2);  // vectors; the host keeps this below 2^32
  const uint32_t OW = static_cast<uint32_t>(g.out_w), OH = static_cast<uint32_t>(g.out_h);
  const uint32_t stride = gridDim.x * blockDim.x;
  for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const uint32_t row = i / row_vecs, u = i - row * row_vecs;
    const uint32_t t = row / OW, ow = row - t * OW;
    const uint32_t b = t / OH, oh = t - b * OH;
    i4 v = {0, 0, 0, 0};
    const int dh = t_dh[u];
    if (dh >= 0) {
      const int64_t ih0 = static_cast<int64_t>(oh) * g.stride_h - g.pad_top, iw0 = static_cast<int64_t>(ow) * g.stride_w - g.pad_left;
      const int64_t ih = ih0 + dh, iw = iw0 + t_dw[u];
      if (ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w)
        v = *reinterpret_cast<const i4*>(x + ((static_cast<int64_t>(b) * g.in_h + ih0) * g.in_w + iw0) * g.in_c + t_off[u]);
    }
    cols[i] = v;
  }
}

__global__ __launch_bounds__(256) void scale_vector_kernel(const void* __restrict__ bias, int bias_s32,
                                                           const float* __restrict__ factors, int64_t n_factors, int64_t n,
                                                           float* __restrict__ out) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (j >= n) return;
  const float b = bias_s32 ? static_cast<float>(static_cast<const int32_t*>(bias)[j]) : static_cast<const float*>(bias)[j];
  out[j] = b * factors[n_factors == 1 ? 0 : j];
}

// ------------------------------------------------------------------------------------------------
// Depthwise Conv2D: out[b, oh, ow, c * mult + m] = sum over the window of x[b, ih, iw, c] * w[kh, kw, c, m], exact in
// int32, then the MatMul's fp32 epilogue (scale per output channel, bias, post-ops, saturate + round).  No matrix
// product in it (each output channel reads one input channel), so it runs on the vector ALU: one thread per output
// position and group of 4 consecutive output channels; with mult == 1 those are 4 consecutive input channels, i.e.
// one dword of x and one dword of w per window tap.  Memory bound in principle (input + output bytes).
// ------------------------------------------------------------------------------------------------
struct DepthwiseArgs {
  int in_h, in_w, in_c, k_h, k_w, out_h, out_w, stride_h, stride_w, dil_h, dil_w, pad_top, pad_left;
  int mult, out_c, groups4;  // groups of 4 output channels per position
  int x_signed, vec;         // vec: mult == 1, in_c % 4 == 0, x and w 4-byte aligned
  int n_scales, n_eltwise;
  itexhip_eltwise elt[3];
  int64_t total;             // positions * groups4
  // the post-op chain as [ReLU | LeakyReLU | clip] [linear map] when it has that form (3x3 kernel): applied under
  // uniform branches; a loop over the chain with a switch per value costs more instruction fetch than arithmetic
  int chain;                 // bit 0 max(x, 0), 1 leaky, 2 clip, 3 linear
  float alpha, lo, hi, lin_a, lin_b;
};

template <int OUT_T>
__global__ __launch_bounds__(256) void qdwconv_kernel(const DepthwiseArgs a, const uint8_t* __restrict__ x,
                                                      const int8_t* __restrict__ w, const float* __restrict__ scales,
                                                      const float* __restrict__ bias, void* __restrict__ out) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < a.total; i += stride) {
    const int64_t pos = i / a.groups4;
    const int oc0 = static_cast<int>(i - pos * a.groups4) * 4;
    const int ow = static_cast<int>(pos % a.out_w);
    const int64_t t = pos / a.out_w;
    const int oh = static_cast<int>(t % a.out_h);
    const int64_t b = t / a.out_h;
    int acc[4] = {0, 0, 0, 0};
    for (int kh = 0; kh < a.k_h; ++kh) {
      const int ih = oh * a.stride_h - a.pad_top + kh * a.dil_h;
      if (ih < 0 || ih >= a.in_h) continue;
      for (int kw = 0; kw < a.k_w; ++kw) {
        const int iw = ow * a.stride_w - a.pad_left + kw * a.dil_w;
        if (iw < 0 || iw >= a.in_w) continue;
        const uint8_t* xp = x + ((b * a.in_h + ih) * a.in_w + iw) * a.in_c;
        const int8_t* wp = w + static_cast<int64_t>(kh * a.k_w + kw) * a.out_c;
        if (a.vec) {
          const uint32_t xv = *reinterpret_cast<const uint32_t*>(xp + oc0);
          const uint32_t wv = *reinterpret_cast<const uint32_t*>(wp + oc0);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int xs = a.x_signed ? (static_cast<int>(xv << (24 - 8 * r)) >> 24) : static_cast<int>((xv >> (8 * r)) & 0xffu);
            acc[r] += __mul24(xs, static_cast<int>(wv << (24 - 8 * r)) >> 24);
          }
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int oc = oc0 + r;
            if (oc < a.out_c) {
              const int c = oc / a.mult;
              const int xs = a.x_signed ? static_cast<int>(reinterpret_cast<const int8_t*>(xp)[c]) : static_cast<int>(xp[c]);
              acc[r] += __mul24(xs, static_cast<int>(wp[oc]));
            }
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = oc0 + r;
      if (n >= a.out_c) break;
      float v = static_cast<float>(acc[r]);
      if (a.n_scales == 1) v = v * scales[0];
      else if (a.n_scales > 1) v = v * scales[n];
      if (bias) v = v + bias[n];
      for (int k = 0; k < a.n_eltwise; ++k) v = apply_eltwise(a.elt[k], v);
      store_output<OUT_T>(out, pos * a.out_c + n, v);
    }
  }
}

// The common case - 3x3 window, stride 1, dilation 1, multiplier 1, channels a multiple of 4 - with the window
// unrolled and 32-bit index arithmetic: a thread owns 4 consecutive channels of a column of R = 4 output rows, so it
// loads each input dword once for up to 3 of its outputs (18 input + 9 filter dwords for 16 outputs), and a wavefront's
// loads cover 256 contiguous bytes (consecutive lanes = consecutive channel groups, then consecutive columns).
template <int OUT_T, bool X_SIGNED>
__global__ __launch_bounds__(256) void qdwconv3x3_kernel(const DepthwiseArgs a, const uint8_t* __restrict__ x,
                                                         const int8_t* __restrict__ w, const float* __restrict__ scales,
                                                         const float* __restrict__ bias, void* __restrict__ out) {
  constexpr int R = 4;
  const uint32_t row_items = static_cast<uint32_t>(a.out_w) * a.groups4;  // (column, channel group) pairs of one output row
  const uint32_t strips = (a.out_h + R - 1) / R;
  const uint32_t total = static_cast<uint32_t>(a.total);                  // batch * strips * row_items, < 2^31 (host)
  const uint32_t stride = gridDim.x * blockDim.x;
  for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const uint32_t t = i / row_items, item = i - t * row_items;
    const uint32_t b = t / strips, strip = t - b * strips;
    const int ow = static_cast<int>(item / a.groups4);
    const int oc0 = static_cast<int>(item - ow * a.groups4) * 4;
    const int oh0 = static_cast<int>(strip) * R;
    int acc[R][4];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[r][c] = 0;
    const uint8_t* xb = x + static_cast<uint32_t>(b) * static_cast<uint32_t>(a.in_h * a.in_w * a.in_c) + oc0;  // input bytes < 2^31 (host)
    // All 18 input dwords are loaded unconditionally from clamped (valid) positions and zeroed afterwards where the
    // position lies in the padding: a branch around each load would make every load wait for the one before it.
    uint32_t xin[3][R + 2];
#pragma unroll
    for (int kw = 0; kw < 3; ++kw) {
      const int iw = ow - a.pad_left + kw;
      const int iwc = min(max(iw, 0), a.in_w - 1);
#pragma unroll
      for (int rr = 0; rr < R + 2; ++rr) {
        const int ih = oh0 - a.pad_top + rr;
        const int ihc = min(max(ih, 0), a.in_h - 1);
        xin[kw][rr] = *reinterpret_cast<const uint32_t*>(xb + (ihc * a.in_w + iwc) * a.in_c);
      }
    }
#pragma unroll
    for (int kw = 0; kw < 3; ++kw) {
      const int iw = ow - a.pad_left + kw;
      const bool col_ok = iw >= 0 && iw < a.in_w;
      uint32_t wv[3];
#pragma unroll
      for (int kh = 0; kh < 3; ++kh) wv[kh] = *reinterpret_cast<const uint32_t*>(w + (kh * 3 + kw) * a.out_c + oc0);
#pragma unroll
      for (int rr = 0; rr < R + 2; ++rr) {  // input rows oh0 - pad_top + rr feed output rows rr - kh
        const int ih = oh0 - a.pad_top + rr;
        const uint32_t xv = (col_ok && ih >= 0 && ih < a.in_h) ? xin[kw][rr] : 0u;
        int xs[4];
#pragma unroll
        for (int c = 0; c < 4; ++c)
          xs[c] = X_SIGNED ? (static_cast<int>(xv << (24 - 8 * c)) >> 24) : static_cast<int>((xv >> (8 * c)) & 0xffu);
#pragma unroll
        for (int kh = 0; kh < 3; ++kh) {
          const int r = rr - kh;
          if (r < 0 || r >= R) continue;
#pragma unroll
          for (int c = 0; c < 4; ++c)  // 8-bit factors: the 24-bit multiply-add is exact and full rate (a 32-bit multiply is not)
            acc[r][c] = __mul24(xs[c], static_cast<int>(wv[kh] << (24 - 8 * c)) >> 24) + acc[r][c];
        }
      }
    }
    float sc[4], bi[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      sc[c] = a.n_scales == 0 ? 1.0f : scales[a.n_scales == 1 ? 0 : oc0 + c];
      bi[c] = bias ? bias[oc0 + c] : 0.0f;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int oh = oh0 + r;
      if (oh >= a.out_h) break;
      const int64_t o = ((static_cast<int64_t>(b) * a.out_h + oh) * a.out_w + ow) * a.out_c + oc0;
      float y[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        float v = static_cast<float>(acc[r][c]);
        if (a.n_scales != 0) v = v * sc[c];
        if (bias) v = v + bi[c];
        y[c] = v;
      }
      if (a.chain & 1) {
#pragma unroll
        for (int c = 0; c < 4; ++c) y[c] = fmaxf(y[c], 0.0f);
      }
      if (a.chain & 2) {
#pragma unroll
        for (int c = 0; c < 4; ++c) y[c] = y[c] > 0.0f ? y[c] : y[c] * a.alpha;
      }
      if (a.chain & 4) {
#pragma unroll
        for (int c = 0; c < 4; ++c) y[c] = fminf(fmaxf(y[c], a.lo), a.hi);
      }
      if (a.chain & 8) {
#pragma unroll
        for (int c = 0; c < 4; ++c) y[c] = a.lin_a * y[c] + a.lin_b;
      }
      // the 4 channels as one store (the host checked the output's alignment)
      if constexpr (OUT_T == ITEXHIP_FLOAT) {
        *reinterpret_cast<f4*>(static_cast<float*>(out) + o) = f4{y[0], y[1], y[2], y[3]};
      } else if constexpr (is_float16_type(OUT_T)) {
        typedef unsigned int u2 __attribute__((ext_vector_type(2)));
        *reinterpret_cast<u2*>(static_cast<uint16_t*>(out) + o) = u2{f32x2_to_bits16<OUT_T>(y[0], y[1]), f32x2_to_bits16<OUT_T>(y[2], y[3])};
      } else if constexpr (OUT_T == ITEXHIP_QINT32) {
        *reinterpret_cast<i4*>(static_cast<int32_t*>(out) + o) = i4{sat_rne<ITEXHIP_QINT32>(y[0]), sat_rne<ITEXHIP_QINT32>(y[1]),
                                                                    sat_rne<ITEXHIP_QINT32>(y[2]), sat_rne<ITEXHIP_QINT32>(y[3])};
      } else {
        *reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(out) + o) =
            pack4(sat_rne<OUT_T>(y[0]), sat_rne<OUT_T>(y[1]), sat_rne<OUT_T>(y[2]), sat_rne<OUT_T>(y[3]));
      }
    }
  }
}

}  // namespace
}  // namespace itexhip

using namespace itexhip;

extern "C" int itexhip_qdepthwise_conv2d(const void* x, int x_type, const itexhip_conv_geometry* g, int64_t multiplier,
                                         const int8_t* filter, const float* scales, const float* bias,
                                         const itexhip_epilogue* ep, int out_type, void* out, void* stream) {
  const char* who = "itexhip_qdepthwise_conv2d";
  ITEXHIP_REQUIRE(g != nullptr && ep != nullptr, "%s: null geometry or epilogue", who);
  ITEXHIP_REQUIRE(x_type == ITEXHIP_QUINT8 || x_type == ITEXHIP_QINT8, "%s: input type must be quint8 or qint8", who);
  ITEXHIP_REQUIRE(out_type == ITEXHIP_QINT32 || out_type == ITEXHIP_QINT8 || out_type == ITEXHIP_QUINT8 ||
                      out_type == ITEXHIP_FLOAT || out_type == ITEXHIP_BFLOAT16, "%s: unsupported output type %d", who, out_type);
  ITEXHIP_REQUIRE(g->batch >= 0 && g->in_h >= 0 && g->in_w >= 0 && g->in_c >= 0 && g->k_h > 0 && g->k_w > 0 && g->out_h >= 0 &&
                      g->out_w >= 0 && multiplier > 0, "%s: bad extents", who);
  ITEXHIP_REQUIRE(g->stride_h > 0 && g->stride_w > 0 && g->dil_h > 0 && g->dil_w > 0, "%s: strides and dilations must be positive", who);
  ITEXHIP_REQUIRE(g->pad_top >= 0 && g->pad_left >= 0, "%s: negative padding", who);
  const int64_t lim = 1LL << 31;
  const int64_t out_c = g->in_c * multiplier;
  ITEXHIP_REQUIRE(g->in_h < lim && g->in_w < lim && out_c < lim && g->out_h < lim && g->out_w < lim && g->k_h < (1 << 15) &&
                      g->k_w < (1 << 15) && g->pad_top < (1 << 24) && g->pad_left < (1 << 24) &&
                      g->out_h * g->stride_h < (1LL << 30) && g->out_w * g->stride_w < (1LL << 30) &&
                      (g->k_h - 1) * g->dil_h < (1LL << 30) && (g->k_w - 1) * g->dil_w < (1LL << 30),
                  "%s: extent too large", who);
  ITEXHIP_REQUIRE(g->k_h * g->k_w <= 32767 && 255LL * 128 * g->k_h * g->k_w < lim, "%s: window too large for int32 accumulation", who);
  ITEXHIP_REQUIRE(ep->n_eltwise >= 0 && ep->n_eltwise <= 3, "%s: bad eltwise count", who);
  for (int k = 0; k < ep->n_eltwise; ++k)
    ITEXHIP_REQUIRE(ep->elt[k].alg != ITEXHIP_ELT_SUM, "%s: no sum post-op here", who);
  ITEXHIP_REQUIRE(ep->n_scales == 0 || ep->n_scales == 1 || ep->n_scales == out_c, "%s: %d scales for %lld channels", who,
                  ep->n_scales, static_cast<long long>(out_c));
  const int64_t positions = g->batch * g->out_h * g->out_w;
  if (positions == 0 || out_c == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(x && filter && out, "%s: null buffer", who);
  ITEXHIP_REQUIRE(ep->n_scales == 0 || scales, "%s: null scales", who);
  DepthwiseArgs a{};
  a.in_h = static_cast<int>(g->in_h); a.in_w = static_cast<int>(g->in_w); a.in_c = static_cast<int>(g->in_c);
  a.k_h = static_cast<int>(g->k_h); a.k_w = static_cast<int>(g->k_w); a.out_h = static_cast<int>(g->out_h);
  a.out_w = static_cast<int>(g->out_w); a.stride_h = g->stride_h; a.stride_w = g->stride_w; a.dil_h = g->dil_h; a.dil_w = g->dil_w;
  a.pad_top = static_cast<int>(g->pad_top); a.pad_left = static_cast<int>(g->pad_left);
  a.mult = static_cast<int>(multiplier); a.out_c = static_cast<int>(out_c); a.groups4 = static_cast<int>((out_c + 3) / 4);
  a.x_signed = x_type == ITEXHIP_QINT8;
  a.vec = multiplier == 1 && g->in_c % 4 == 0 && aligned(x, 4) && aligned(filter, 4);
  a.n_scales = ep->n_scales; a.n_eltwise = ep->n_eltwise;
  a.elt[0] = ep->elt[0]; a.elt[1] = ep->elt[1]; a.elt[2] = ep->elt[2];
  a.total = positions * a.groups4;
  const uint8_t* xp = static_cast<const uint8_t*>(x);
  hipStream_t st = as_stream(stream);
  const int64_t strip_total = g->batch * ((g->out_h + 3) / 4) * g->out_w * a.groups4;
  bool canonical = true;
  {
    int k = 0;
    if (k < ep->n_eltwise && ep->elt[k].alg == ITEXHIP_ELT_RELU) {
      if (ep->elt[k].alpha == 0.0f) a.chain |= 1; else { a.chain |= 2; a.alpha = ep->elt[k].alpha; }
      ++k;
    } else if (k < ep->n_eltwise && ep->elt[k].alg == ITEXHIP_ELT_CLIP) {
      a.chain |= 4; a.lo = ep->elt[k].alpha; a.hi = ep->elt[k].beta;
      ++k;
    }
    if (k < ep->n_eltwise && ep->elt[k].alg == ITEXHIP_ELT_LINEAR) {
      a.chain |= 8; a.lin_a = ep->elt[k].alpha; a.lin_b = ep->elt[k].beta;
      ++k;
    }
    canonical = k == ep->n_eltwise;
  }
  if (canonical && a.vec && aligned(out, 16) && g->k_h == 3 && g->k_w == 3 && g->stride_h == 1 && g->stride_w == 1 && g->dil_h == 1 && g->dil_w == 1 &&
      strip_total < lim && g->batch * g->in_h * g->in_w * g->in_c < lim) {
    a.total = strip_total;
    const unsigned sblocks = static_cast<unsigned>(std::min<int64_t>((a.total + 255) / 256, 256 * 64));
#define DW3(T)                                                                                           \
  if (a.x_signed) qdwconv3x3_kernel<T, true><<<sblocks, 256, 0, st>>>(a, xp, filter, scales, bias, out); \
  else qdwconv3x3_kernel<T, false><<<sblocks, 256, 0, st>>>(a, xp, filter, scales, bias, out)
    switch (out_type) {
      case ITEXHIP_FLOAT: DW3(ITEXHIP_FLOAT); break;
      case ITEXHIP_BFLOAT16: DW3(ITEXHIP_BFLOAT16); break;
      case ITEXHIP_QINT32: DW3(ITEXHIP_QINT32); break;
      case ITEXHIP_QINT8: DW3(ITEXHIP_QINT8); break;
      default: DW3(ITEXHIP_QUINT8); break;
    }
#undef DW3
    ITEXHIP_CHECK_LAUNCH(who);
    return ITEXHIP_OK;
  }
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((a.total + 255) / 256, 256 * 64));
  switch (out_type) {
    case ITEXHIP_FLOAT: qdwconv_kernel<ITEXHIP_FLOAT><<<blocks, 256, 0, st>>>(a, xp, filter, scales, bias, out); break;
    case ITEXHIP_BFLOAT16: qdwconv_kernel<ITEXHIP_BFLOAT16><<<blocks, 256, 0, st>>>(a, xp, filter, scales, bias, out); break;
    case ITEXHIP_QINT32: qdwconv_kernel<ITEXHIP_QINT32><<<blocks, 256, 0, st>>>(a, xp, filter, scales, bias, out); break;
    case ITEXHIP_QINT8: qdwconv_kernel<ITEXHIP_QINT8><<<blocks, 256, 0, st>>>(a, xp, filter, scales, bias, out); break;
    default: qdwconv_kernel<ITEXHIP_QUINT8><<<blocks, 256, 0, st>>>(a, xp, filter, scales, bias, out); break;
  }
  ITEXHIP_CHECK_LAUNCH(who);
  return ITEXHIP_OK;
}

extern "C" int itexhip_im2col8(const void* x, const itexhip_conv_geometry* g, int64_t row_bytes, void* cols, void* stream) {
  const char* who = "itexhip_im2col8";
  ITEXHIP_REQUIRE(g != nullptr, "%s: null geometry", who);
  ITEXHIP_REQUIRE(g->batch >= 0 && g->in_h >= 0 && g->in_w >= 0 && g->in_c >= 0 && g->k_h > 0 && g->k_w > 0 && g->out_h >= 0 &&
                      g->out_w >= 0, "%s: bad extents", who);
  ITEXHIP_REQUIRE(g->stride_h > 0 && g->stride_w > 0 && g->dil_h > 0 && g->dil_w > 0, "%s: strides and dilations must be positive", who);
  ITEXHIP_REQUIRE(g->pad_top >= 0 && g->pad_left >= 0, "%s: negative padding", who);
  const int64_t K = g->k_h * g->k_w * g->in_c;
  ITEXHIP_REQUIRE(K < (1LL << 31), "%s: receptive field too large", who);
  ITEXHIP_REQUIRE(row_bytes >= K && row_bytes % 16 == 0, "%s: row_bytes must be a multiple of 16 and at least %lld", who,
                  static_cast<long long>(K));
  const int64_t rows = g->batch * g->out_h * g->out_w;
  if (rows == 0 || row_bytes == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(cols != nullptr && aligned(cols, 16), "%s: null or misaligned output", who);
  ITEXHIP_REQUIRE(K == 0 || x != nullptr, "%s: null input", who);
  // every position the kernel may read lies inside the input: it only reads where 0 <= ih < in_h, 0 <= iw < in_w
  Im2colArgs a;
  a.g = *g;
  a.row_dwords = row_bytes / 4;
  a.total = rows * a.row_dwords;
  a.K = static_cast<int>(K);
  a.vec = g->in_c % 4 == 0 && aligned(x, 4);
  // 16-byte vectors when a vector never straddles a pixel and the index arithmetic fits 32 bits
  const int64_t in_bytes = g->batch * g->in_h * g->in_w * g->in_c;
  if (g->in_c % 16 == 0 && aligned(x, 16) && row_bytes / 16 <= kMaxRowVectors && a.total / 4 < (1LL << 32) &&
      in_bytes < (1LL << 31) && rows < (1LL << 31)) {
    const int64_t vecs = a.total / 4;
    const int64_t vblocks = std::min<int64_t>((vecs + 255) / 256, 256 * 32);
    im2col8_vec_kernel<<<static_cast<unsigned>(vblocks), 256, 0, as_stream(stream)>>>(a, static_cast<const uint8_t*>(x),
                                                                                     static_cast<i4*>(cols));
    ITEXHIP_CHECK_LAUNCH(who);
    return ITEXHIP_OK;
  }
  // extremes of the 32-bit byte offsets the table kernel forms before clamping (window origins may lie in the padding)
  const int64_t hi_off = ((g->batch * g->in_h + (g->out_h - 1) * g->stride_h - g->pad_top) * g->in_w + (g->out_w - 1) * g->stride_w -
                          g->pad_left) * g->in_c + ((g->k_h - 1) * g->dil_h * g->in_w + (g->k_w - 1) * g->dil_w + 1) * g->in_c;
  const int64_t lo_off = (g->pad_top * g->in_w + g->pad_left) * g->in_c;
  if (!a.vec && hi_off < (1LL << 31) && lo_off < (1LL << 31) &&
      row_bytes <= kMaxRowBytesTable && a.total < (1LL << 31) && in_bytes > 0 && in_bytes < (1LL << 31) &&
      (g->k_h - 1) * g->dil_h < (1 << 15) && (g->k_w - 1) * g->dil_w < (1 << 15) && g->pad_top < (1 << 24) && g->pad_left < (1 << 24) &&
      g->out_h * g->stride_h < (1LL << 30) && g->out_w * g->stride_w < (1LL << 30)) {
    const int64_t bblocks = std::min<int64_t>((a.total + 255) / 256, 256 * 32);
    im2col8_byte_kernel<<<static_cast<unsigned>(bblocks), 256, 0, as_stream(stream)>>>(a, static_cast<const uint8_t*>(x),
                                                                                      static_cast<uint32_t*>(cols));
    ITEXHIP_CHECK_LAUNCH(who);
    return ITEXHIP_OK;
  }
  const int64_t blocks = std::min<int64_t>((a.total + 255) / 256, 256 * 32);
  im2col8_kernel<<<static_cast<unsigned>(blocks), 256, 0, as_stream(stream)>>>(a, static_cast<const uint8_t*>(x),
                                                                                static_cast<uint32_t*>(cols));
  ITEXHIP_CHECK_LAUNCH(who);
  return ITEXHIP_OK;
}

extern "C" int itexhip_pad_nhwc8(const void* x, int64_t n, int64_t h, int64_t w, int64_t c, int64_t lead_h, int64_t lead_w,
                                 int64_t out_h, int64_t out_w, int64_t out_c, void* out, void* stream) {
  const char* who = "itexhip_pad_nhwc8";
  ITEXHIP_REQUIRE(n >= 0 && h >= 0 && w >= 0 && c >= 0 && lead_h >= 0 && lead_w >= 0, "%s: negative extent", who);
  ITEXHIP_REQUIRE(out_h >= lead_h + h && out_w >= lead_w + w && out_c >= c, "%s: the output must hold the input behind its leading padding", who);
  ITEXHIP_REQUIRE(out_c % 4 == 0, "%s: out_c must be a multiple of 4", who);
  const int64_t lim = 1LL << 31;
  ITEXHIP_REQUIRE(n < lim && h < lim && w < lim && c < lim && out_h < lim && out_w < lim && out_c < lim, "%s: extent too large", who);
  const int64_t total = n * out_h * out_w * out_c / 4;  // factors below 2^31 each; the product is checked next
  ITEXHIP_REQUIRE(n == 0 || out_h == 0 || out_w == 0 || out_c == 0 || (n * out_h < lim && n * out_h * out_w < lim && total < lim),
                  "%s: the padded tensor must stay below 2^31 dwords", who);
  if (total == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(out != nullptr && aligned(out, 4), "%s: null or misaligned output", who);
  ITEXHIP_REQUIRE(x != nullptr || n * h * w * c == 0, "%s: null input", who);
  Pad4dArgs a;
  a.n = static_cast<int>(n); a.h = static_cast<int>(h); a.w = static_cast<int>(w); a.c = static_cast<int>(c);
  a.lead_h = static_cast<int>(lead_h); a.lead_w = static_cast<int>(lead_w);
  a.out_h = static_cast<int>(out_h); a.out_w = static_cast<int>(out_w); a.out_c = static_cast<int>(out_c);
  a.total = static_cast<uint32_t>(total);
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  const unsigned vblocks = static_cast<unsigned>((total / 4 + 255) / 256);
  if (out_c == 4 && out_w % 4 == 0 && aligned(out, 16))
    pad_nhwc8_vec_kernel<4><<<vblocks, 256, 0, as_stream(stream)>>>(a, xb, static_cast<i4*>(out));
  else if (out_c == 8 && out_w % 2 == 0 && aligned(out, 16))
    pad_nhwc8_vec_kernel<8><<<vblocks, 256, 0, as_stream(stream)>>>(a, xb, static_cast<i4*>(out));
  else
    pad_nhwc8_kernel<<<static_cast<unsigned>((total + 255) / 256), 256, 0, as_stream(stream)>>>(a, xb, static_cast<uint32_t*>(out));
  ITEXHIP_CHECK_LAUNCH(who);
  return ITEXHIP_OK;
}

extern "C" int itexhip_scale_vector(const void* bias, int bias_type, const float* factors, int64_t n_factors, int64_t n,
                                    float* out, void* stream) {
  const char* who = "itexhip_scale_vector";
  ITEXHIP_REQUIRE(bias_type == ITEXHIP_FLOAT || bias_type == ITEXHIP_QINT32, "%s: bias type must be float or qint32", who);
  ITEXHIP_REQUIRE(n >= 0 && (n_factors == 1 || n_factors == n), "%s: %lld factors for %lld entries", who,
                  static_cast<long long>(n_factors), static_cast<long long>(n));
  if (n == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(bias && factors && out, "%s: null buffer", who);
  scale_vector_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, as_stream(stream)>>>(
      bias, bias_type == ITEXHIP_QINT32, factors, n_factors, n, out);
  ITEXHIP_CHECK_LAUNCH(who);
  return ITEXHIP_OK;
}
