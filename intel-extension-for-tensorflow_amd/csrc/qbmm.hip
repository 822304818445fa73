// Quantized BatchMatMul: qint8 x qint8 -> float / bfloat16 / half with fused Mul / Add operands
// (itex/core/kernels/common/batch_matmul_op.h:36-522; device registrations in
// itex/core/kernels/gpu/matmul_op.cc:612-655).
//
// Both operands are activations (the Q.K^T and P.V products of an attention block), so nothing can be
// prepacked: every workgroup stages a 64 x 64 byte tile of each operand in LDS, k-contiguous per output row /
// column, and its four wavefronts each own one 32 x 32 quadrant of the 64 x 64 output tile
// (v_mfma_i32_32x32x32_i8).  An operand stored with k as the slow dimension (x with adj_x, y without
// adj_y) is transposed on the way into LDS, four bytes at a time.  The output orientation keeps
// n on the lanes, so every store instruction writes 128 contiguous bytes per half-wavefront: with fp32
// outputs the op is bound by that write.
#include "common.hpp"

namespace itexhip {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kTile = 64;          // output tile edge and k step
constexpr int kLdsStride = 80;     // bytes per LDS row: 64 + 16, keeps the 16-byte fragment reads aligned
constexpr int kBmmThreads = 256;

struct BmmArgs {
  itexhip_bmm_params p;
  int tiles_m, tiles_n;
  int vec_x, vec_y;  // operand layouts allow aligned vector loads
};

// One 64 (rows or columns of the output) x 64 (k) byte tile into LDS, k-contiguous.
//   KCONT: the operand is stored [R, K] (k fastest);  else [K, R] (r fastest) and is transposed here.
//   VEC:   aligned 16-byte (KCONT) / 4-byte (transposed) global loads are legal and never straddle a bound.
template <bool KCONT, bool VEC>
__device__ __forceinline__ void stage_tile(const int8_t* __restrict__ g, int64_t R, int64_t K, int64_t r0, int64_t k0,
                                           uint8_t* __restrict__ lds, int t) {
  if constexpr (KCONT) {
    const int r = t >> 2, seg = t & 3;
    const int64_t row = r0 + r, k = k0 + seg * 16;
    v4i v = {0, 0, 0, 0};
    if (row < R) {
      const int8_t* src = g + row * K + k;
      if constexpr (VEC) {
        if (k < K) v = *reinterpret_cast<const v4i*>(src);
      } else {
        uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int b = 0; b < 16; ++b)
          if (k + b < K) w[b >> 2] |= static_cast<uint32_t>(static_cast<uint8_t>(src[b])) << (8 * (b & 3));
        v = v4i{static_cast<int>(w[0]), static_cast<int>(w[1]), static_cast<int>(w[2]), static_cast<int>(w[3])};
      }
    }
    *reinterpret_cast<v4i*>(lds + r * kLdsStride + seg * 16) = v;
  } else {
    // 4 (k) x 4 (r) bytes per thread: kb = t / 16 picks the k rows, cb = t % 16 the r columns
    const int kb = t >> 4, cb = t & 15;
    uint32_t rows[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t k = k0 + kb * 4 + i, r = r0 + cb * 4;
      uint32_t w = 0;
      if (k < K) {
        const int8_t* src = g + k * R + r;
        if constexpr (VEC) {
          if (r < R) w = *reinterpret_cast<const uint32_t*>(src);
        } else {
#pragma unroll
          for (int b = 0; b < 4; ++b)
            if (r + b < R) w |= static_cast<uint32_t>(static_cast<uint8_t>(src[b])) << (8 * b);
        }
      }
      rows[i] = w;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {  // byte j of the four k rows -> four consecutive k of column cb * 4 + j
      const uint32_t w = ((rows[0] >> (8 * j)) & 0xffu) | (((rows[1] >> (8 * j)) & 0xffu) << 8) |
                         (((rows[2] >> (8 * j)) & 0xffu) << 16) | (((rows[3] >> (8 * j)) & 0xffu) << 24);
      *reinterpret_cast<uint32_t*>(lds + (cb * 4 + j) * kLdsStride + kb * 4) = w;
    }
  }
}

__device__ __forceinline__ float load_operand(const void* __restrict__ data, int64_t off, int out_type) {
  if (out_type == ITEXHIP_FLOAT) return static_cast<const float*>(data)[off];
  const uint32_t bits = static_cast<const uint16_t*>(data)[off];
  return out_type == ITEXHIP_BFLOAT16 ? bf16_bits_to_f32(bits) : f16_bits_to_f32(bits);
}

template <bool ADJ_X, bool ADJ_Y, bool VEC_X, bool VEC_Y>
__global__ __launch_bounds__(kBmmThreads) void qbmm_kernel(const BmmArgs a, const int8_t* __restrict__ x,
                                                           const int8_t* __restrict__ y, void* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) uint8_t xs[kTile * kLdsStride];
  __shared__ __attribute__((aligned(16))) uint8_t ys[kTile * kLdsStride];
  const itexhip_bmm_params& p = a.p;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // workgroup -> (batch entry, tile); consecutive workgroups walk the tiles of one matrix
  const int64_t tiles = static_cast<int64_t>(a.tiles_m) * a.tiles_n;
  const int64_t bi = blockIdx.x / tiles;
  const int tile = static_cast<int>(blockIdx.x - bi * tiles);
  const int64_t m0 = static_cast<int64_t>(tile / a.tiles_n) * kTile, n0 = static_cast<int64_t>(tile % a.tiles_n) * kTile;

  int64_t xo = 0, yo = 0, bo[ITEXHIP_BMM_MAX_BINARY] = {0, 0};
  {
    int64_t rem = bi;
    for (int d = p.n_batch_dims - 1; d >= 0; --d) {
      const int64_t i = rem % p.batch_dims[d];
      rem /= p.batch_dims[d];
      xo += i * p.x_batch_stride[d];
      yo += i * p.y_batch_stride[d];
      for (int b = 0; b < p.n_binary; ++b) bo[b] += i * p.binary[b].batch_stride[d];
    }
  }
  const int8_t* xb = x + xo;
  const int8_t* yb = y + yo;

  v16i acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0;

  for (int64_t k0 = 0; k0 < p.K; k0 += kTile) {
    stage_tile<!ADJ_X, VEC_X>(xb, p.M, p.K, m0, k0, xs, t);  // x is [M, K] unless adj_x
    stage_tile<ADJ_Y, VEC_Y>(yb, p.N, p.K, n0, k0, ys, t);   // y is [N, K] only with adj_y
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int off = kk * 32 + (lane >> 5) * 16;
      const v4i fx = *reinterpret_cast<const v4i*>(xs + (wm * 32 + (lane & 31)) * kLdsStride + off);
      const v4i fy = *reinterpret_cast<const v4i*>(ys + (wn * 32 + (lane & 31)) * kLdsStride + off);
      acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx, fy, acc, 0, 0, 0);
    }
    __syncthreads();
  }

  // accumulator i of a lane: row (i / 4) * 8 + (lane / 32) * 4 + i % 4, column lane % 32 of the quadrant
  const int64_t n = n0 + wn * 32 + (lane & 31);
  if (n >= p.N) return;
  const int64_t ob = bi * p.M * p.N;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t m = m0 + wm * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
    if (m >= p.M) continue;
    float v = static_cast<float>(acc[i]) * p.scale;
    for (int b = 0; b < p.n_binary; ++b) {
      const float o = load_operand(p.binary[b].data, bo[b] + m * p.binary[b].stride_m + n * p.binary[b].stride_n, p.out_type);
      v = p.binary[b].alg == ITEXHIP_BIN_MUL ? v * o : v + o;
    }
    const int64_t oo = ob + m * p.N + n;
    if (p.out_type == ITEXHIP_FLOAT) static_cast<float*>(out)[oo] = v;
    else if (p.out_type == ITEXHIP_BFLOAT16) static_cast<uint16_t*>(out)[oo] = static_cast<uint16_t>(f32_to_bf16_bits(v));
    else static_cast<uint16_t*>(out)[oo] = static_cast<uint16_t>(f32_to_f16_bits(v));
  }
}

template <bool ADJ_X, bool ADJ_Y>
void launch_layout(const BmmArgs& a, const int8_t* x, const int8_t* y, void* out, unsigned grid, hipStream_t st) {
  if (a.vec_x && a.vec_y) qbmm_kernel<ADJ_X, ADJ_Y, true, true><<<grid, kBmmThreads, 0, st>>>(a, x, y, out);
  else if (a.vec_x) qbmm_kernel<ADJ_X, ADJ_Y, true, false><<<grid, kBmmThreads, 0, st>>>(a, x, y, out);
  else if (a.vec_y) qbmm_kernel<ADJ_X, ADJ_Y, false, true><<<grid, kBmmThreads, 0, st>>>(a, x, y, out);
  else qbmm_kernel<ADJ_X, ADJ_Y, false, false><<<grid, kBmmThreads, 0, st>>>(a, x, y, out);
}

// An operand's matrices may be read with aligned vector loads when every matrix starts on the vector
// width and every row keeps that alignment.
bool vector_layout(const void* base, const int64_t* batch_stride, int n_batch_dims, int64_t row_len, int width) {
  if (!aligned(base, width) || row_len % width != 0) return false;
  for (int d = 0; d < n_batch_dims; ++d)
    if (batch_stride[d] % width != 0) return false;
  return true;
}

}  // namespace
}  // namespace itexhip

using namespace itexhip;

extern "C" int itexhip_qbatch_matmul(const itexhip_bmm_params* p, const int8_t* x, const int8_t* y, void* out, void* stream) {
  const char* who = "itexhip_qbatch_matmul";
  ITEXHIP_REQUIRE(p != nullptr, "%s: null params", who);
  ITEXHIP_REQUIRE(p->n_batch_dims >= 0 && p->n_batch_dims <= ITEXHIP_BMM_MAX_BATCH_DIMS, "%s: %d batch dimensions (at most %d)", who,
                  p->n_batch_dims, ITEXHIP_BMM_MAX_BATCH_DIMS);
  ITEXHIP_REQUIRE(is_float_out(p->out_type), "%s: the output type must be float, bfloat16 or half, got %d", who, p->out_type);
  ITEXHIP_REQUIRE(p->M >= 0 && p->K >= 0 && p->N >= 0 && p->M < (1LL << 31) && p->N < (1LL << 31) && p->K < (1LL << 31),
                  "%s: bad matrix dimensions", who);
  ITEXHIP_REQUIRE(p->n_binary >= 0 && p->n_binary <= ITEXHIP_BMM_MAX_BINARY, "%s: %d binary post-ops (at most %d)", who, p->n_binary,
                  ITEXHIP_BMM_MAX_BINARY);
  int64_t batch = 1;
  for (int d = 0; d < p->n_batch_dims; ++d) {
    ITEXHIP_REQUIRE(p->batch_dims[d] >= 0 && p->x_batch_stride[d] >= 0 && p->y_batch_stride[d] >= 0, "%s: negative batch dimension or stride", who);
    batch *= p->batch_dims[d];
  }
  for (int b = 0; b < p->n_binary; ++b) {
    ITEXHIP_REQUIRE(p->binary[b].alg == ITEXHIP_BIN_MUL || p->binary[b].alg == ITEXHIP_BIN_ADD, "%s: unknown binary post-op %d", who,
                    p->binary[b].alg);
    ITEXHIP_REQUIRE(p->binary[b].data != nullptr && aligned(p->binary[b].data, p->out_type == ITEXHIP_FLOAT ? 4 : 2),
                    "%s: null or misaligned binary operand", who);
    ITEXHIP_REQUIRE(p->binary[b].stride_m >= 0 && p->binary[b].stride_n >= 0, "%s: negative binary operand stride", who);
  }
  if (batch == 0 || p->M == 0 || p->N == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(out != nullptr && aligned(out, p->out_type == ITEXHIP_FLOAT ? 4 : 2), "%s: null or misaligned output", who);
  ITEXHIP_REQUIRE(p->K == 0 || (x != nullptr && y != nullptr), "%s: null operand", who);

  BmmArgs a;
  a.p = *p;
  a.tiles_m = static_cast<int>((p->M + kTile - 1) / kTile);
  a.tiles_n = static_cast<int>((p->N + kTile - 1) / kTile);
  const int64_t grid = batch * a.tiles_m * a.tiles_n;
  ITEXHIP_REQUIRE(grid < (1LL << 31), "%s: %lld output tiles exceed one launch", who, static_cast<long long>(grid));
  // [R, K] layouts load 16 bytes along k, [K, R] layouts 4 bytes along r
  a.vec_x = p->adj_x ? vector_layout(x, p->x_batch_stride, p->n_batch_dims, p->M, 4) : vector_layout(x, p->x_batch_stride, p->n_batch_dims, p->K, 16);
  a.vec_y = p->adj_y ? vector_layout(y, p->y_batch_stride, p->n_batch_dims, p->K, 16) : vector_layout(y, p->y_batch_stride, p->n_batch_dims, p->N, 4);
  hipStream_t st = as_stream(stream);
  const unsigned g = static_cast<unsigned>(grid);
  if (p->adj_x && p->adj_y) launch_layout<true, true>(a, x, y, out, g, st);
  else if (p->adj_x) launch_layout<true, false>(a, x, y, out, g, st);
  else if (p->adj_y) launch_layout<false, true>(a, x, y, out, g, st);
  else launch_layout<false, false>(a, x, y, out, g, st);
  ITEXHIP_CHECK_LAUNCH(who);
  return ITEXHIP_OK;
}
