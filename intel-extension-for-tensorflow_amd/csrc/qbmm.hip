// Quantized BatchMatMul: qint8 x qint8 -> float / bfloat16 / half with fused Mul / Add operands
// (itex/core/kernels/common/batch_matmul_op.h:36-522; device registrations in
// itex/core/kernels/gpu/matmul_op.cc:612-655).
//
// Both operands are activations (the Q.K^T and P.V products of an attention block), so nothing can be
// prepacked: every workgroup stages a 64 x 64 byte tile of each operand in LDS, k-contiguous per output row /
// column, and its four wavefronts each own one 32 x 32 quadrant of the 64 x 64 output tile
// (v_mfma_i32_32x32x32_i8); large calls run tiles of 128 rows (and columns) with two (four) quadrants per
// wavefront.  An operand stored with k as the slow dimension (x with adj_x, y without
// adj_y) is transposed on the way into LDS, four bytes at a time.  The output orientation keeps
// n on the lanes, so every store instruction writes 128 contiguous bytes per half-wavefront: with fp32
// outputs the op is bound by that write.
#include <type_traits>
#include <utility>

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
  int grid3;         // launched as (tiles, innermost batch dimension, the other batch dimensions): no division finds them
  int rm, rn;        // the tile is (64 rm) x (64 rn)
};

// One 64 (rows or columns of the output) x 64 (k) byte tile on its way into LDS, k-contiguous there.  The
// global loads (fetch_tile) and the LDS stores (put_tile) are separate so that the next tile's loads are in
// flight while the current one is multiplied.
//   KCONT: the operand is stored [R, K] (k fastest);  else [K, R] (r fastest) and is transposed in put_tile.
//   VEC:   aligned 16-byte (KCONT) / 4-byte (transposed) global loads are legal and never straddle a bound.
template <bool KCONT, bool VEC>
__device__ __forceinline__ void fetch_tile(const int8_t* __restrict__ g, int64_t R, int64_t K, int64_t r0, int64_t k0,
                                           int t, uint32_t (&w)[4]) {
  w[0] = w[1] = w[2] = w[3] = 0;
  if constexpr (KCONT) {  // thread: row t / 4, 16 consecutive k
    const int64_t row = r0 + (t >> 2), k = k0 + (t & 3) * 16;
    if (row >= R) return;
    const int8_t* src = g + row * K + k;
    if constexpr (VEC) {
      if (k < K) {
        const v4i v = *reinterpret_cast<const v4i*>(src);
        w[0] = v[0]; w[1] = v[1]; w[2] = v[2]; w[3] = v[3];
      }
    } else {
#pragma unroll
      for (int b = 0; b < 16; ++b)
        if (k + b < K) w[b >> 2] |= static_cast<uint32_t>(static_cast<uint8_t>(src[b])) << (8 * (b & 3));
    }
  } else {  // thread: 4 (k) x 4 (r) bytes; kb = t / 16 picks the k rows, cb = t % 16 the r columns; w[i] = k row i
    const int kb = t >> 4, cb = t & 15;
    const int64_t r = r0 + cb * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t k = k0 + kb * 4 + i;
      if (k >= K) continue;
      const int8_t* src = g + k * R + r;
      if constexpr (VEC) {
        if (r < R) w[i] = *reinterpret_cast<const uint32_t*>(src);
      } else {
#pragma unroll
        for (int b = 0; b < 4; ++b)
          if (r + b < R) w[i] |= static_cast<uint32_t>(static_cast<uint8_t>(src[b])) << (8 * b);
      }
    }
  }
}

template <bool KCONT>
__device__ __forceinline__ void put_tile(uint8_t* __restrict__ lds, int t, const uint32_t (&w)[4]) {
  if constexpr (KCONT) {
    *reinterpret_cast<v4i*>(lds + (t >> 2) * kLdsStride + (t & 3) * 16) =
        v4i{static_cast<int>(w[0]), static_cast<int>(w[1]), static_cast<int>(w[2]), static_cast<int>(w[3])};
  } else {
    const int kb = t >> 4, cb = t & 15;
    // 4 x 4 byte transpose in two rounds of byte permutes: byte j of the four k rows -> four consecutive k of column
    // cb * 4 + j  (v_perm_b32 numbers the bytes of its second operand 0..3 and of its first 4..7)
    const uint32_t lo01 = __builtin_amdgcn_perm(w[1], w[0], 0x05010400u);  // w0.b0 w1.b0 w0.b1 w1.b1
    const uint32_t hi01 = __builtin_amdgcn_perm(w[1], w[0], 0x07030602u);  // w0.b2 w1.b2 w0.b3 w1.b3
    const uint32_t lo23 = __builtin_amdgcn_perm(w[3], w[2], 0x05010400u);
    const uint32_t hi23 = __builtin_amdgcn_perm(w[3], w[2], 0x07030602u);
    const uint32_t v[4] = {__builtin_amdgcn_perm(lo23, lo01, 0x05040100u), __builtin_amdgcn_perm(lo23, lo01, 0x07060302u),
                           __builtin_amdgcn_perm(hi23, hi01, 0x05040100u), __builtin_amdgcn_perm(hi23, hi01, 0x07060302u)};
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<uint32_t*>(lds + (cb * 4 + j) * kLdsStride + kb * 4) = v[j];
  }
}

template <int T>
__device__ __forceinline__ float widen(float v) { return v; }
template <int T>
__device__ __forceinline__ float widen(uint16_t bits) {
  return T == ITEXHIP_BFLOAT16 ? bf16_bits_to_f32(bits) : f16_bits_to_f32(bits);
}

// Where one wavefront's 32 x 32 quadrant goes.  Everything that is the same for the whole wavefront is a
// 64-bit base address; what differs between lanes and rows is a 32-bit byte offset (the host bounds N and
// the operand strides so that 64 rows of them fit), which is the addressing form the hardware takes directly.
struct QuadrantSite {
  int rows_left, cols_left;   // of the output below / right of the quadrant's first element
  float scale;
  int n_binary;
  int alg[ITEXHIP_BMM_MAX_BINARY];
  const char* operand[ITEXHIP_BMM_MAX_BINARY];           // address of the quadrant's first operand element
  uint32_t operand_row[ITEXHIP_BMM_MAX_BINARY], operand_col[ITEXHIP_BMM_MAX_BINARY];  // byte strides
  char* out;                                             // address of the quadrant's first output element
  uint32_t out_row;                                      // byte stride between output rows
};

// Operand values of the lane's 16 results.  Straight-line code: every load is issued whatever the operand's
// broadcast pattern (rows and columns outside the output read element (0, 0) of the quadrant instead), so that
// nothing forces a wait before the tiles arrive.
// ROWB: no operand depends on the row (a scalar, or a mask broadcast over the rows): one value per lane and operand
// instead of 16, which is what lets twice as many wavefronts share a SIMD.
template <int OUT_T, int NB, bool ROWB>
__device__ __forceinline__ void fetch_operands(const QuadrantSite& s, int lane, float (&o)[ITEXHIP_BMM_MAX_BINARY][ROWB ? 1 : 16]) {
  using elem_t = typename std::conditional<OUT_T == ITEXHIP_FLOAT, float, uint16_t>::type;
  const uint32_t lrow = (lane >> 5) * 4;
  const uint32_t lcol = static_cast<int>(lane & 31) < s.cols_left ? (lane & 31) : 0;
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    if constexpr (ROWB) {
      o[b][0] = widen<OUT_T>(*reinterpret_cast<const elem_t*>(s.operand[b] + lcol * s.operand_col[b]));
      continue;
    }
#pragma unroll
    for (int i = 0; i < (ROWB ? 1 : 16); ++i) {
      const uint32_t row = lrow + (i >> 2) * 8 + (i & 3);
      const uint32_t off = (static_cast<int>(row) < s.rows_left ? row : 0) * s.operand_row[b] + lcol * s.operand_col[b];
      o[b][i] = widen<OUT_T>(*reinterpret_cast<const elem_t*>(s.operand[b] + off));
    }
  }
}

// One result on its way out: scale, fused operands in order (each separately rounded), narrowing, store.
template <int OUT_T, int NB, bool ROWB, int ALG0, int ALG1>
__device__ __forceinline__ void store_one(int acc, const QuadrantSite& s, int i, uint32_t off,
                                          const float (&o)[ITEXHIP_BMM_MAX_BINARY][ROWB ? 1 : 16]) {
  using elem_t = typename std::conditional<OUT_T == ITEXHIP_FLOAT, float, uint16_t>::type;
  float v = static_cast<float>(acc) * s.scale;
  if constexpr (NB > 0) v = ALG0 == ITEXHIP_BIN_MUL ? v * o[0][ROWB ? 0 : i] : v + o[0][ROWB ? 0 : i];
  if constexpr (NB > 1) v = ALG1 == ITEXHIP_BIN_MUL ? v * o[1][ROWB ? 0 : i] : v + o[1][ROWB ? 0 : i];
  elem_t* dst = reinterpret_cast<elem_t*>(s.out + off);
  // the output is written back as it goes instead of staying dirty in L2 until the kernel ends: as system-scope
  // (write-through) stores without fused operands (P.V over 128 sequences: 21.3 -> 18.8 us), as streaming stores
  // with them (Q.K^T + Mul + Add measured 3 % slower written through)
  if constexpr (OUT_T == ITEXHIP_FLOAT && NB == 0) __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  else if constexpr (OUT_T == ITEXHIP_FLOAT) __builtin_nontemporal_store(v, dst);
  else __builtin_nontemporal_store(static_cast<uint16_t>(f32_to_bits16<OUT_T>(v)), dst);
}

template <int OUT_T, int NB, bool ROWB, int ALG0, int ALG1>
__device__ __forceinline__ void store_rows(const v16i& acc, const QuadrantSite& s, int lane,
                                           const float (&o)[ITEXHIP_BMM_MAX_BINARY][ROWB ? 1 : 16]) {
  using elem_t = typename std::conditional<OUT_T == ITEXHIP_FLOAT, float, uint16_t>::type;
  const uint32_t lrow = (lane >> 5) * 4, lcol = lane & 31;
  const uint32_t obase = lrow * s.out_row + lcol * static_cast<uint32_t>(sizeof(elem_t));
  if (s.rows_left == 32 && s.cols_left == 32) {  // a whole quadrant (the same answer for the wavefront): nothing to test
#pragma unroll
    for (int i = 0; i < 16; ++i)
      store_one<OUT_T, NB, ROWB, ALG0, ALG1>(acc[i], s, i, obase + static_cast<uint32_t>((i >> 2) * 8 + (i & 3)) * s.out_row, o);
    return;
  }
  if (static_cast<int>(lcol) >= s.cols_left) return;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = (i >> 2) * 8 + (i & 3);
    if (static_cast<int>(lrow) + r >= s.rows_left) continue;
    store_one<OUT_T, NB, ROWB, ALG0, ALG1>(acc[i], s, i, obase + r * s.out_row, o);
  }
}

// The operands' algorithms are the same for the whole launch: one copy of the store loop per combination, chosen by
// a branch, instead of computing product and sum of every element and selecting.
template <int OUT_T, int NB, bool ROWB>
__device__ __forceinline__ void store_quadrant(const v16i& acc, const QuadrantSite& s, int lane,
                                               const float (&o)[ITEXHIP_BMM_MAX_BINARY][ROWB ? 1 : 16]) {
  constexpr int MUL = ITEXHIP_BIN_MUL, ADD = ITEXHIP_BIN_ADD;
  if constexpr (NB == 0) {
    store_rows<OUT_T, NB, ROWB, ADD, ADD>(acc, s, lane, o);
  } else if constexpr (NB == 1) {
    if (s.alg[0] == MUL) store_rows<OUT_T, NB, ROWB, MUL, ADD>(acc, s, lane, o);
    else store_rows<OUT_T, NB, ROWB, ADD, ADD>(acc, s, lane, o);
  } else {
    if (s.alg[0] == MUL && s.alg[1] == MUL) store_rows<OUT_T, NB, ROWB, MUL, MUL>(acc, s, lane, o);
    else if (s.alg[0] == MUL) store_rows<OUT_T, NB, ROWB, MUL, ADD>(acc, s, lane, o);
    else if (s.alg[1] == MUL) store_rows<OUT_T, NB, ROWB, ADD, MUL>(acc, s, lane, o);
    else store_rows<OUT_T, NB, ROWB, ADD, ADD>(acc, s, lane, o);
  }
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <class F, int... I>
__device__ __forceinline__ void quadrants_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void quadrants(F&& f) {
  quadrants_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

// Where quadrant (qm, qn) of the output matrix bi goes and what its fused operands are.  A quadrant off the edge of the
// output stores nothing (its wavefront still helps staging the tiles) and addresses the tile's first element, which
// always exists.
template <int NB>
__device__ __forceinline__ QuadrantSite quadrant_site(const itexhip_bmm_params& p, const int64_t (&bo)[ITEXHIP_BMM_MAX_BINARY],
                                                      uint32_t bi, int m0, int n0, int qm_, int qn_, void* __restrict__ out) {
  const bool live = qm_ < p.M && qn_ < p.N;
  const int64_t qm = live ? qm_ : m0, qn = live ? qn_ : n0;
  const uint32_t esz = p.out_type == ITEXHIP_FLOAT ? 4 : 2;
  QuadrantSite s;
  s.rows_left = live ? static_cast<int>(p.M - qm < 32 ? p.M - qm : 32) : 0;
  s.cols_left = live ? static_cast<int>(p.N - qn < 32 ? p.N - qn : 32) : 0;
  s.scale = p.scale;
  s.n_binary = p.n_binary;
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    s.alg[b] = p.binary[b].alg;
    s.operand[b] = static_cast<const char*>(p.binary[b].data) +
                   (bo[b] + qm * p.binary[b].stride_m + qn * p.binary[b].stride_n) * esz;
    s.operand_row[b] = static_cast<uint32_t>(p.binary[b].stride_m) * esz;
    s.operand_col[b] = static_cast<uint32_t>(p.binary[b].stride_n) * esz;
  }
  s.out = static_cast<char*>(out) + ((static_cast<int64_t>(bi) * p.M + qm) * p.N + qn) * esz;
  s.out_row = static_cast<uint32_t>(p.N) * esz;
  return s;
}

// What a workgroup does once it knows where its operands are: a (64 RM) x (64 RN) output tile, each of the four
// wavefronts RM x RN quadrants of 32 x 32.  One straight-line instance per (number of fused operands, output type).
// The larger tiles amortise what a wavefront spends around its MFMAs (a 64 x 64 tile of K = 64 is two MFMAs and some
// 450 other instructions per wavefront) and read each operand half as often; they exist for the calls whose fused
// operands take one register per lane and quadrant column (none, or ROWB).
template <bool ADJ_X, bool ADJ_Y, bool VEC_X, bool VEC_Y, int NB, int OUT_T, bool ROWB, int RM, int RN>
__device__ __forceinline__ void bmm_body(const itexhip_bmm_params& p, const int8_t* __restrict__ xb,
                                         const int8_t* __restrict__ yb, const int64_t (&bo)[ITEXHIP_BMM_MAX_BINARY], uint32_t bi,
                                         int m0, int n0, int wm, int wn, int t, int lane, void* __restrict__ out,
                                         uint8_t* __restrict__ xs, uint8_t* __restrict__ ys) {
  static_assert(RM * RN == 1 || NB == 0 || ROWB, "larger tiles keep the operands of all their quadrants in registers");
  // first tiles and the fused operands: all loads the results depend on are issued before any is needed
  uint32_t wx[RM][4], wy[RN][4];
#pragma unroll
  for (int h = 0; h < RM; ++h) fetch_tile<!ADJ_X, VEC_X>(xb, p.M, p.K, m0 + 64 * h, 0, t, wx[h]);  // x is [M, K] unless adj_x
#pragma unroll
  for (int h = 0; h < RN; ++h) fetch_tile<ADJ_Y, VEC_Y>(yb, p.N, p.K, n0 + 64 * h, 0, t, wy[h]);   // y is [N, K] only with adj_y
  // (the quadrants are walked with compile-time indices: what describes a quadrant is the same for the whole
  // wavefront and must stay in scalar registers, which an indexed array of descriptors does not)
  float o[RM * RN][ITEXHIP_BMM_MAX_BINARY][ROWB ? 1 : 16];
  quadrants<RM * RN>([&](auto q) {
    constexpr int i = decltype(q)::value / RN, j = decltype(q)::value % RN;
    const QuadrantSite s = quadrant_site<NB>(p, bo, bi, m0, n0, m0 + (wm * RM + i) * 32, n0 + (wn * RN + j) * 32, out);
    fetch_operands<OUT_T, NB, ROWB>(s, lane, o[decltype(q)::value]);
  });

  v16i acc[RM * RN];
  quadrants<RM * RN>([&](auto q) {
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[decltype(q)::value][e] = 0;
  });

  for (int64_t k0 = 0; k0 < p.K; k0 += kTile) {
#pragma unroll
    for (int h = 0; h < RM; ++h) put_tile<!ADJ_X>(xs + h * 64 * kLdsStride, t, wx[h]);
#pragma unroll
    for (int h = 0; h < RN; ++h) put_tile<ADJ_Y>(ys + h * 64 * kLdsStride, t, wy[h]);
    __syncthreads();
    if (k0 + kTile < p.K) {  // the next tile travels while this one is multiplied
#pragma unroll
      for (int h = 0; h < RM; ++h) fetch_tile<!ADJ_X, VEC_X>(xb, p.M, p.K, m0 + 64 * h, k0 + kTile, t, wx[h]);
#pragma unroll
      for (int h = 0; h < RN; ++h) fetch_tile<ADJ_Y, VEC_Y>(yb, p.N, p.K, n0 + 64 * h, k0 + kTile, t, wy[h]);
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int off = kk * 32 + (lane >> 5) * 16;
      v4i fx[RM], fy[RN];
#pragma unroll
      for (int i = 0; i < RM; ++i) fx[i] = *reinterpret_cast<const v4i*>(xs + ((wm * RM + i) * 32 + (lane & 31)) * kLdsStride + off);
#pragma unroll
      for (int j = 0; j < RN; ++j) fy[j] = *reinterpret_cast<const v4i*>(ys + ((wn * RN + j) * 32 + (lane & 31)) * kLdsStride + off);
      quadrants<RM * RN>([&](auto q) {
        constexpr int i = decltype(q)::value / RN, j = decltype(q)::value % RN;
        acc[decltype(q)::value] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx[i], fy[j], acc[decltype(q)::value], 0, 0, 0);
      });
    }
    __syncthreads();
  }
  quadrants<RM * RN>([&](auto q) {
    constexpr int i = decltype(q)::value / RN, j = decltype(q)::value % RN;
    const QuadrantSite s = quadrant_site<NB>(p, bo, bi, m0, n0, m0 + (wm * RM + i) * 32, n0 + (wn * RN + j) * 32, out);
    store_quadrant<OUT_T, NB, ROWB>(acc[decltype(q)::value], s, lane, o[decltype(q)::value]);
  });
}

// One kernel per (layouts, number of fused operands, output type, operands independent of the row): compiled as one
// kernel with a switch over these, every variant took the registers of the largest (112 - 140, three or four
// wavefronts per SIMD; P.V over 128 sequences 18.7 -> 16.4 us as a kernel of its own).
template <bool ADJ_X, bool ADJ_Y, bool VEC_X, bool VEC_Y, int NB, int OUT_T, bool ROWB, int RM = 1, int RN = 1>
__global__ __launch_bounds__(kBmmThreads) void qbmm_kernel(const BmmArgs a, const int8_t* __restrict__ x,
                                                           const int8_t* __restrict__ y, void* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) uint8_t xs[RM * kTile * kLdsStride];
  __shared__ __attribute__((aligned(16))) uint8_t ys[RN * kTile * kLdsStride];
  const itexhip_bmm_params& p = a.p;
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // the same for the whole wavefront: keep it scalar
  const int wm = wave >> 1, wn = wave & 1;

  // workgroup -> (batch entry, tile); consecutive workgroups walk the tiles of one matrix.  Launched as a 3-d grid
  // (whenever its extents allow) the innermost batch index and the product of the others come from the workgroup id;
  // otherwise, and for more than two batch dimensions, divisions find them.  The launch has fewer than 2^31
  // workgroups, so 32-bit arithmetic covers the decomposition.
  const uint32_t tile = a.grid3 ? blockIdx.x : blockIdx.x % (static_cast<uint32_t>(a.tiles_m) * static_cast<uint32_t>(a.tiles_n));
  const int tm = a.tiles_n == 1 ? static_cast<int>(tile) : static_cast<int>(tile / a.tiles_n);
  const int m0 = tm * (RM * kTile), n0 = static_cast<int>(tile - tm * a.tiles_n) * (RN * kTile);

  int64_t xo = 0, yo = 0, bo[ITEXHIP_BMM_MAX_BINARY] = {0, 0};
  uint32_t bi;  // index of the output matrix
  {
    int d = p.n_batch_dims - 1;
    uint32_t rem;
    if (a.grid3) {
      if (d >= 0) {  // the innermost batch dimension: blockIdx.y
        const int64_t i = blockIdx.y;
        xo = i * p.x_batch_stride[d];
        yo = i * p.y_batch_stride[d];
#pragma unroll
        for (int b = 0; b < NB; ++b) bo[b] = i * p.binary[b].batch_stride[d];
        --d;
      }
      rem = blockIdx.z;
      bi = blockIdx.z * gridDim.y + blockIdx.y;
    } else {
      bi = blockIdx.x / (static_cast<uint32_t>(a.tiles_m) * static_cast<uint32_t>(a.tiles_n));
      rem = bi;
    }
    for (; d >= 0; --d) {
      const uint32_t dim = static_cast<uint32_t>(p.batch_dims[d]);
      const uint32_t q = d == 0 ? 0 : rem / dim;   // the outermost index needs no division
      const int64_t i = rem - q * dim;
      rem = q;
      xo += i * p.x_batch_stride[d];
      yo += i * p.y_batch_stride[d];
#pragma unroll
      for (int b = 0; b < NB; ++b) bo[b] += i * p.binary[b].batch_stride[d];
    }
  }
  // accumulator e of a lane is row (e / 4) * 8 + (lane / 32) * 4 + e % 4, column lane % 32 of its quadrant
  bmm_body<ADJ_X, ADJ_Y, VEC_X, VEC_Y, NB, OUT_T, ROWB, RM, RN>(p, x + xo, y + yo, bo, bi, m0, n0, wm, wn, t, lane, out, xs, ys);
}

template <bool ADJ_X, bool ADJ_Y, int NB, int OUT_T, bool ROWB>
void launch_vec(const BmmArgs& a, const int8_t* x, const int8_t* y, void* out, dim3 grid, hipStream_t st) {
  if constexpr (NB == 0 || ROWB) {  // the larger tiles (chosen by the host for aligned operands only)
    if (a.rm == 2 && a.rn == 2) {
      qbmm_kernel<ADJ_X, ADJ_Y, true, true, NB, OUT_T, ROWB, 2, 2><<<grid, kBmmThreads, 0, st>>>(a, x, y, out);
      return;
    }
    if (a.rm == 2 && a.rn == 1) {
      qbmm_kernel<ADJ_X, ADJ_Y, true, true, NB, OUT_T, ROWB, 2, 1><<<grid, kBmmThreads, 0, st>>>(a, x, y, out);
      return;
    }
  }
  if (a.vec_x && a.vec_y) qbmm_kernel<ADJ_X, ADJ_Y, true, true, NB, OUT_T, ROWB><<<grid, kBmmThreads, 0, st>>>(a, x, y, out);
  else if (a.vec_x) qbmm_kernel<ADJ_X, ADJ_Y, true, false, NB, OUT_T, ROWB><<<grid, kBmmThreads, 0, st>>>(a, x, y, out);
  else if (a.vec_y) qbmm_kernel<ADJ_X, ADJ_Y, false, true, NB, OUT_T, ROWB><<<grid, kBmmThreads, 0, st>>>(a, x, y, out);
  else qbmm_kernel<ADJ_X, ADJ_Y, false, false, NB, OUT_T, ROWB><<<grid, kBmmThreads, 0, st>>>(a, x, y, out);
}

template <bool ADJ_X, bool ADJ_Y, int OUT_T>
void launch_operands(const BmmArgs& a, const int8_t* x, const int8_t* y, void* out, dim3 grid, hipStream_t st) {
  bool rowb = true;  // no fused operand depends on the row
  for (int b = 0; b < a.p.n_binary; ++b) rowb = rowb && a.p.binary[b].stride_m == 0;
  switch (a.p.n_binary * 2 + (rowb ? 1 : 0)) {
    case 2: launch_vec<ADJ_X, ADJ_Y, 1, OUT_T, false>(a, x, y, out, grid, st); break;
    case 3: launch_vec<ADJ_X, ADJ_Y, 1, OUT_T, true>(a, x, y, out, grid, st); break;
    case 4: launch_vec<ADJ_X, ADJ_Y, 2, OUT_T, false>(a, x, y, out, grid, st); break;
    case 5: launch_vec<ADJ_X, ADJ_Y, 2, OUT_T, true>(a, x, y, out, grid, st); break;
    default: launch_vec<ADJ_X, ADJ_Y, 0, OUT_T, false>(a, x, y, out, grid, st); break;
  }
}

template <bool ADJ_X, bool ADJ_Y>
void launch_layout(const BmmArgs& a, const int8_t* x, const int8_t* y, void* out, dim3 grid, hipStream_t st) {
  if (a.p.out_type == ITEXHIP_FLOAT) launch_operands<ADJ_X, ADJ_Y, ITEXHIP_FLOAT>(a, x, y, out, grid, st);
  else if (a.p.out_type == ITEXHIP_BFLOAT16) launch_operands<ADJ_X, ADJ_Y, ITEXHIP_BFLOAT16>(a, x, y, out, grid, st);
  else launch_operands<ADJ_X, ADJ_Y, ITEXHIP_HALF>(a, x, y, out, grid, st);
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

  // lane offsets inside a quadrant are 32-bit byte offsets: 64 rows of N (or of an operand's row stride) must fit
  ITEXHIP_REQUIRE(p->N < (1LL << 22), "%s: N = %lld is not supported (N < 2^22)", who, static_cast<long long>(p->N));
  for (int b = 0; b < p->n_binary; ++b)
    ITEXHIP_REQUIRE(p->binary[b].stride_m < (1LL << 22) && p->binary[b].stride_n < (1LL << 22),
                    "%s: a binary operand's matrix strides must be below 2^22 elements", who);

  BmmArgs a;
  a.p = *p;
  for (int b = p->n_binary; b < ITEXHIP_BMM_MAX_BINARY; ++b) a.p.binary[b] = itexhip_bmm_binary{};
  // merge adjacent batch dimensions that every tensor walks with one stride (fewer index divisions per workgroup)
  for (int d = a.p.n_batch_dims - 2; d >= 0; --d) {
    const int64_t inner = a.p.batch_dims[d + 1];
    bool same = a.p.x_batch_stride[d] == a.p.x_batch_stride[d + 1] * inner &&
                a.p.y_batch_stride[d] == a.p.y_batch_stride[d + 1] * inner;
    for (int b = 0; b < a.p.n_binary; ++b)
      same = same && a.p.binary[b].batch_stride[d] == a.p.binary[b].batch_stride[d + 1] * inner;
    if (!same) continue;
    a.p.batch_dims[d] *= inner;
    a.p.x_batch_stride[d] = a.p.x_batch_stride[d + 1];
    a.p.y_batch_stride[d] = a.p.y_batch_stride[d + 1];
    for (int b = 0; b < a.p.n_binary; ++b) a.p.binary[b].batch_stride[d] = a.p.binary[b].batch_stride[d + 1];
    for (int e = d + 1; e + 1 < a.p.n_batch_dims; ++e) {
      a.p.batch_dims[e] = a.p.batch_dims[e + 1];
      a.p.x_batch_stride[e] = a.p.x_batch_stride[e + 1];
      a.p.y_batch_stride[e] = a.p.y_batch_stride[e + 1];
      for (int b = 0; b < a.p.n_binary; ++b) a.p.binary[b].batch_stride[e] = a.p.binary[b].batch_stride[e + 1];
    }
    --a.p.n_batch_dims;
  }
  // [R, K] layouts load 16 bytes along k, [K, R] layouts 4 bytes along r
  a.vec_x = p->adj_x ? vector_layout(x, p->x_batch_stride, p->n_batch_dims, p->M, 4) : vector_layout(x, p->x_batch_stride, p->n_batch_dims, p->K, 16);
  a.vec_y = p->adj_y ? vector_layout(y, p->y_batch_stride, p->n_batch_dims, p->K, 16) : vector_layout(y, p->y_batch_stride, p->n_batch_dims, p->N, 4);
  // Tiles of 128 rows (and 128 columns) where more than 64 exist, the operands are aligned, the fused operands do not
  // depend on the row, and at least 1024 tiles remain (four per CU); else 64 x 64.  BERT-base attention over 128
  // sequences, 1536 tiles: Q.K^T + Mul + Add 24.6 -> 20.0 us, P.V 16.9 -> 14.2 us; over 32 sequences the 384 larger
  // tiles measured slower than the 1536 small ones (7.4 against 6.5 us).
  bool rowb = true;
  for (int b = 0; b < p->n_binary; ++b) rowb = rowb && p->binary[b].stride_m == 0;
  a.rm = a.rn = 1;
  if (a.vec_x && a.vec_y && rowb && p->M > kTile) {
    const int rn = p->N > kTile ? 2 : 1;
    if (batch * ((p->M + 2 * kTile - 1) / (2 * kTile)) * ((p->N + rn * kTile - 1) / (rn * kTile)) >= 1024) {
      a.rm = 2;
      a.rn = rn;
    }
  }
  a.tiles_m = static_cast<int>((p->M + a.rm * kTile - 1) / (a.rm * kTile));
  a.tiles_n = static_cast<int>((p->N + a.rn * kTile - 1) / (a.rn * kTile));
  const int64_t grid = batch * a.tiles_m * a.tiles_n;
  ITEXHIP_REQUIRE(grid < (1LL << 31), "%s: %lld output tiles exceed one launch", who, static_cast<long long>(grid));
  hipStream_t st = as_stream(stream);
  // (tiles of a matrix, innermost batch dimension, product of the other batch dimensions) when the extents fit a grid
  const int64_t tiles = static_cast<int64_t>(a.tiles_m) * a.tiles_n;
  const int64_t inner = a.p.n_batch_dims > 0 ? a.p.batch_dims[a.p.n_batch_dims - 1] : 1;
  a.grid3 = inner <= 65535 && batch / inner <= 65535 ? 1 : 0;
  const dim3 g = a.grid3 ? dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(inner), static_cast<unsigned>(batch / inner))
                         : dim3(static_cast<unsigned>(grid));
  if (p->adj_x && p->adj_y) launch_layout<true, true>(a, x, y, out, g, st);
  else if (p->adj_x) launch_layout<true, false>(a, x, y, out, g, st);
  else if (p->adj_y) launch_layout<false, true>(a, x, y, out, g, st);
  else launch_layout<false, false>(a, x, y, out, g, st);
  ITEXHIP_CHECK_LAUNCH(who);
  return ITEXHIP_OK;
}
