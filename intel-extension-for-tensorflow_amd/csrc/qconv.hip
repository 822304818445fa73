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

}  // namespace
}  // namespace itexhip

using namespace itexhip;

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
  const int64_t blocks = std::min<int64_t>((a.total + 255) / 256, 256 * 32);
  im2col8_kernel<<<static_cast<unsigned>(blocks), 256, 0, as_stream(stream)>>>(a, static_cast<const uint8_t*>(x),
                                                                                static_cast<uint32_t*>(cols));
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
