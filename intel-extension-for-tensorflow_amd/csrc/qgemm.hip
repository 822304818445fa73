// Quantized MatMul on gfx950: u8/s8 activations x s8 weights -> exact int32 accumulation on the i8
// MFMA (v_mfma_i32_16x16x64_i8), fused fp32 epilogue in registers.
//
// Operand roles.  The weight is the MFMA "A" operand (its 16 rows are 16 output channels n), the
// activation is the "B" operand (its 16 columns are 16 rows m of the activation matrix).  A lane then
// ends up with 4 consecutive output channels of one output row, which is what a row-major [M,N]
// output wants (4 int8 = one dword store, 4 fp32 = one 16-byte store).
//
// Operand tile ("chunk") = 16 rows x 64 k = 1 KiB, stored in lane order: lane l holds 16 consecutive
// k of row (l % 16), k-group (l / 16).  The prepacked weight is the sequence of such chunks
// [n/16][k/64]; activation chunks are formed on the fly.  Both operands use the same (lane, byte) -> k
// mapping, so the order in which the instruction consumes k inside a chunk cannot affect the integer
// sum.
//
// Unsigned activations: the MFMA is signed x signed, so u8 values are fed as (a ^ 0x80) = a - 128 and
// the epilogue adds 128 * colsum[n] back (exact: |acc| <= 255 * 127 * K stays far below 2^31 for the
// K this library accepts).
#include <algorithm>

#include "common.hpp"

namespace itexhip {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kChunkBytes = 1024;  // 16 rows x 64 k
constexpr int64_t kMaxK = 1 << 16; // 255 * 128 * 65536 < 2^31

struct EpilogueArgs {
  const float* scales;
  const float* bias;
  const int32_t* colsum;
  int n_scales;
  int comp_mul;  // 128 for u8 activations, 0 for s8
  int n_eltwise;
  itexhip_eltwise elt[2];
};

// ------------------------------------------------------------------------------------------------
// Epilogue for one 16x16 accumulator tile held in MFMA layout: lane l, register r ->
//   m = m0 + (l % 16), n = n0 + (l / 16) * 4 + r.
// ------------------------------------------------------------------------------------------------
template <int OUT_T>
__device__ __forceinline__ void epilogue_tile(const v4i& acc, int m, int n, int M, int N,
                                              const EpilogueArgs& e, void* __restrict__ out,
                                              bool vec_ok) {
  if (m >= M || n >= N) return;
  float y[4];
  const bool full = (n + 3 < N);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int nn = n + r;
    if (!full && nn >= N) { y[r] = 0.0f; continue; }
    int a = acc[r];
    if (e.comp_mul) a += e.comp_mul * e.colsum[nn];
    float v = static_cast<float>(a);
    if (e.n_scales == 1) v = v * e.scales[0];
    else if (e.n_scales > 1) v = v * e.scales[nn];
    if (e.bias) v = v + e.bias[nn];
    for (int k = 0; k < e.n_eltwise; ++k) v = apply_eltwise(e.elt[k], v);
    y[r] = v;
  }
  const int64_t o = static_cast<int64_t>(m) * N + n;
  if constexpr (OUT_T == ITEXHIP_FLOAT) {
    float* p = reinterpret_cast<float*>(out) + o;
    if (full && vec_ok) {
      *reinterpret_cast<float4*>(p) = make_float4(y[0], y[1], y[2], y[3]);
    } else {
      for (int r = 0; r < 4 && n + r < N; ++r) p[r] = y[r];
    }
  } else if constexpr (OUT_T == ITEXHIP_QINT32) {
    int32_t* p = reinterpret_cast<int32_t*>(out) + o;
    if (full && vec_ok) {
      *reinterpret_cast<int4*>(p) = make_int4(sat_rne<ITEXHIP_QINT32>(y[0]), sat_rne<ITEXHIP_QINT32>(y[1]),
                                              sat_rne<ITEXHIP_QINT32>(y[2]), sat_rne<ITEXHIP_QINT32>(y[3]));
    } else {
      for (int r = 0; r < 4 && n + r < N; ++r) p[r] = sat_rne<ITEXHIP_QINT32>(y[r]);
    }
  } else {
    uint8_t* p = reinterpret_cast<uint8_t*>(out) + o;
    if (full && vec_ok) {
      *reinterpret_cast<uint32_t*>(p) =
          pack4(sat_rne<OUT_T>(y[0]), sat_rne<OUT_T>(y[1]), sat_rne<OUT_T>(y[2]), sat_rne<OUT_T>(y[3]));
    } else {
      for (int r = 0; r < 4 && n + r < N; ++r) p[r] = static_cast<uint8_t>(sat_rne<OUT_T>(y[r]));
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Weight prepack + column sums.  One thread produces one 16-byte piece (row n, 16 consecutive k).
// ------------------------------------------------------------------------------------------------
__global__ void zero_i32_kernel(int32_t* p, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

__global__ __launch_bounds__(256) void prepack_b_kernel(const int8_t* __restrict__ w, int transpose_b,
                                                         int K, int N, int KT, int NT,
                                                         int8_t* __restrict__ packed,
                                                         int32_t* __restrict__ colsum) {
  const int64_t chunk = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (chunk >= static_cast<int64_t>(NT) * KT) return;  // whole wavefront leaves together
  const int lane = threadIdx.x & 63;
  const int nt = static_cast<int>(chunk / KT), kt = static_cast<int>(chunk % KT);
  const int n = nt * 16 + (lane & 15);
  const int k0 = kt * 64 + (lane >> 4) * 16;
  union { int8_t b[16]; v4i v; } piece;
  int sum = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int k = k0 + i;
    int8_t v = 0;
    if (n < N && k < K)
      v = transpose_b ? w[static_cast<int64_t>(n) * K + k] : w[static_cast<int64_t>(k) * N + n];
    piece.b[i] = v;
    sum += v;
  }
  *reinterpret_cast<v4i*>(packed + chunk * kChunkBytes + lane * 16) = piece.v;
  // add up the four k-groups of this row, then one atomic per row and chunk
  sum += __shfl_xor(sum, 16, 64);
  sum += __shfl_xor(sum, 32, 64);
  if (lane < 16 && n < N && sum != 0) atomicAdd(&colsum[n], sum);
}

// ------------------------------------------------------------------------------------------------
// Tile kernel (compute bound, M > 16).
//   block tile BM (activation rows) x BN (output channels), K step 64 (one chunk deep),
//   WAVES_M x WAVES_N wavefronts, each owning a (BM/WAVES_M) x (BN/WAVES_N) sub-tile,
//   double-buffered LDS staging in chunk order, global -> register -> LDS prefetch of the next step
//   while the MFMAs of the current one run.
// ------------------------------------------------------------------------------------------------
template <int BM, int BN, int WAVES_M, int WAVES_N, int OUT_T>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void qgemm_tile_kernel(
    const uint8_t* __restrict__ a, uint32_t a_xor, const uint8_t* __restrict__ bp, int M, int K, int N,
    int KT, int NT, int num_m, int num_n, EpilogueArgs e, void* __restrict__ out) {
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int A_CHUNKS = BM / 16, B_CHUNKS = BN / 16;
  constexpr int A_PER_WAVE = A_CHUNKS / NW, B_PER_WAVE = B_CHUNKS / NW;
  static_assert(A_CHUNKS % NW == 0 && B_CHUNKS % NW == 0, "chunks must divide among wavefronts");
  constexpr int STAGE_BYTES = (A_CHUNKS + B_CHUNKS) * kChunkBytes;

  extern __shared__ __align__(16) uint8_t lds[];

  // ---- block -> tile mapping: consecutive workgroup ids go round-robin to the 8 XCDs; give every
  // XCD a contiguous range of tiles (m fastest) so that the tiles sharing a weight panel share an L2.
  int pid = blockIdx.x;
  const int total = num_m * num_n;
  if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
  const int tile_m = pid % num_m, tile_n = pid / num_m;
  const int m_base = tile_m * BM, n_base = tile_n * BN;

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;
  const int lrow = lane & 15, lgrp = lane >> 4;

  v4i acc[TN][TM];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i) acc[j][i] = v4i{0, 0, 0, 0};

  v4i stage_a[A_PER_WAVE], stage_b[B_PER_WAVE];

  auto load_global = [&](int kt) {
#pragma unroll
    for (int c = 0; c < A_PER_WAVE; ++c) {
      const int chunk = wave * A_PER_WAVE + c;
      const int m = m_base + chunk * 16 + lrow;
      const int k = kt * 64 + lgrp * 16;
      v4i v = v4i{0, 0, 0, 0};
      if (m < M && k < K) v = *reinterpret_cast<const v4i*>(a + static_cast<int64_t>(m) * K + k);
      stage_a[c] = v;
    }
#pragma unroll
    for (int c = 0; c < B_PER_WAVE; ++c) {
      const int nt = (n_base >> 4) + wave * B_PER_WAVE + c;
      v4i v = v4i{0, 0, 0, 0};
      if (nt < NT)
        v = *reinterpret_cast<const v4i*>(bp + (static_cast<int64_t>(nt) * KT + kt) * kChunkBytes + lane * 16);
      stage_b[c] = v;
    }
  };
  auto store_lds = [&](int buf) {
    uint8_t* base = lds + buf * STAGE_BYTES;
#pragma unroll
    for (int c = 0; c < A_PER_WAVE; ++c) {
      v4i v = stage_a[c];
      v.x ^= a_xor; v.y ^= a_xor; v.z ^= a_xor; v.w ^= a_xor;
      *reinterpret_cast<v4i*>(base + (wave * A_PER_WAVE + c) * kChunkBytes + lane * 16) = v;
    }
#pragma unroll
    for (int c = 0; c < B_PER_WAVE; ++c)
      *reinterpret_cast<v4i*>(base + (A_CHUNKS + wave * B_PER_WAVE + c) * kChunkBytes + lane * 16) = stage_b[c];
  };
  auto compute = [&](int buf) {
    const uint8_t* base = lds + buf * STAGE_BYTES;
    v4i fa[TM], fb[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
      fa[i] = *reinterpret_cast<const v4i*>(base + (wm * TM + i) * kChunkBytes + lane * 16);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      fb[j] = *reinterpret_cast<const v4i*>(base + (A_CHUNKS + wn * TN + j) * kChunkBytes + lane * 16);
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int i = 0; i < TM; ++i)
        acc[j][i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[j], fa[i], acc[j][i], 0, 0, 0);
  };

  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) load_global(kt + 1);
    compute(buf);
    if (kt + 1 < KT) store_lds(buf ^ 1);
    __syncthreads();
  }

  const bool vec_ok = (N & 3) == 0;
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = m_base + (wm * TM + i) * 16 + lrow;
      const int n = n_base + (wn * TN + j) * 16 + lgrp * 4;
      epilogue_tile<OUT_T>(acc[j][i], m, n, M, N, e, out, vec_ok);
    }
}

// ------------------------------------------------------------------------------------------------
// Small-M kernel (M <= 16, bandwidth bound on the weight).  One workgroup owns one 16-channel strip
// of the weight, a contiguous stream of KT chunks; its WAVES wavefronts take chunks round-robin
// (all of a wavefront's loads are issued before the first MFMA), multiply them with the matching
// activation chunk, and the partial 16x16 tiles are added up through LDS.
// ------------------------------------------------------------------------------------------------
template <int WAVES, int OUT_T>
__global__ __launch_bounds__(64 * WAVES) void qgemv_kernel(const uint8_t* __restrict__ a, uint32_t a_xor,
                                                           const uint8_t* __restrict__ bp, int M, int K,
                                                           int N, int KT, EpilogueArgs e,
                                                           void* __restrict__ out) {
  constexpr int UNROLL = 4;
  __shared__ int red[WAVES][64 * 4];
  const int nt = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lrow = lane & 15, lgrp = lane >> 4;
  const uint8_t* strip = bp + static_cast<int64_t>(nt) * KT * kChunkBytes + lane * 16;
  const uint8_t* arow = a + static_cast<int64_t>(lrow) * K + lgrp * 16;
  const bool row_ok = lrow < M;

  v4i acc = v4i{0, 0, 0, 0};
  int kt = wave;
  for (; kt + (UNROLL - 1) * WAVES < KT; kt += UNROLL * WAVES) {
    v4i w[UNROLL], x[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
      w[u] = __builtin_nontemporal_load(
          reinterpret_cast<const v4i*>(strip + static_cast<int64_t>(kt + u * WAVES) * kChunkBytes));
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int k = (kt + u * WAVES) * 64 + lgrp * 16;
      v4i v = v4i{0, 0, 0, 0};
      if (row_ok && k < K) {
        v = *reinterpret_cast<const v4i*>(arow + static_cast<int64_t>(kt + u * WAVES) * 64);
        v.x ^= a_xor; v.y ^= a_xor; v.z ^= a_xor; v.w ^= a_xor;
      }
      x[u] = v;
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[u], x[u], acc, 0, 0, 0);
  }
  for (; kt < KT; kt += WAVES) {
    const v4i w = __builtin_nontemporal_load(
        reinterpret_cast<const v4i*>(strip + static_cast<int64_t>(kt) * kChunkBytes));
    const int k = kt * 64 + lgrp * 16;
    v4i v = v4i{0, 0, 0, 0};
    if (row_ok && k < K) {
      v = *reinterpret_cast<const v4i*>(arow + static_cast<int64_t>(kt) * 64);
      v.x ^= a_xor; v.y ^= a_xor; v.z ^= a_xor; v.w ^= a_xor;
    }
    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(w, v, acc, 0, 0, 0);
  }

#pragma unroll
  for (int r = 0; r < 4; ++r) red[wave][r * 64 + lane] = acc[r];
  __syncthreads();
  if (wave == 0) {
    v4i s = v4i{0, 0, 0, 0};
#pragma unroll
    for (int w = 0; w < WAVES; ++w)
#pragma unroll
      for (int r = 0; r < 4; ++r) s[r] += red[w][r * 64 + lane];
    epilogue_tile<OUT_T>(s, lrow, nt * 16 + lgrp * 4, M, N, e, out, (N & 3) == 0);
  }
}

// ------------------------------------------------------------------------------------------------
// Reference-shaped kernel on the unpacked weight: one thread per output element.
// ------------------------------------------------------------------------------------------------
template <int OUT_T>
__global__ __launch_bounds__(256) void qgemm_naive_kernel(const uint8_t* __restrict__ a, int a_is_u8,
                                                           const int8_t* __restrict__ w, int transpose_b,
                                                           int M, int K, int N, EpilogueArgs e,
                                                           void* __restrict__ out) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(M) * N) return;
  const int m = static_cast<int>(idx / N), n = static_cast<int>(idx % N);
  int acc = 0;
  for (int k = 0; k < K; ++k) {
    const int av = a_is_u8 ? static_cast<int>(a[static_cast<int64_t>(m) * K + k])
                           : static_cast<int>(reinterpret_cast<const int8_t*>(a)[static_cast<int64_t>(m) * K + k]);
    const int wv = transpose_b ? w[static_cast<int64_t>(n) * K + k] : w[static_cast<int64_t>(k) * N + n];
    acc += av * wv;
  }
  float v = static_cast<float>(acc);
  if (e.n_scales == 1) v = v * e.scales[0];
  else if (e.n_scales > 1) v = v * e.scales[n];
  if (e.bias) v = v + e.bias[n];
  for (int k = 0; k < e.n_eltwise; ++k) v = apply_eltwise(e.elt[k], v);
  if constexpr (OUT_T == ITEXHIP_FLOAT) reinterpret_cast<float*>(out)[idx] = v;
  else if constexpr (OUT_T == ITEXHIP_QINT32) reinterpret_cast<int32_t*>(out)[idx] = sat_rne<ITEXHIP_QINT32>(v);
  else reinterpret_cast<uint8_t*>(out)[idx] = static_cast<uint8_t>(sat_rne<OUT_T>(v));
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
int check_common(const void* a, int a_type, const void* b, int64_t M, int64_t K, int64_t N,
                 const float* scales, const itexhip_epilogue* ep, int out_type, const void* out,
                 const char* who) {
  ITEXHIP_REQUIRE(a_type == ITEXHIP_QUINT8 || a_type == ITEXHIP_QINT8, "%s: activation type must be quint8 or qint8", who);
  ITEXHIP_REQUIRE(out_type == ITEXHIP_QINT32 || out_type == ITEXHIP_QINT8 || out_type == ITEXHIP_QUINT8 ||
                      out_type == ITEXHIP_FLOAT, "%s: unsupported output type %d", who, out_type);
  ITEXHIP_REQUIRE(M >= 0 && K >= 0 && N >= 0, "%s: negative dimension", who);
  ITEXHIP_REQUIRE(M < (1LL << 31) && N < (1LL << 31) && K <= kMaxK, "%s: dimension too large (K <= %lld)", who,
                  static_cast<long long>(kMaxK));
  ITEXHIP_REQUIRE(ep != nullptr, "%s: null epilogue", who);
  ITEXHIP_REQUIRE(ep->n_eltwise >= 0 && ep->n_eltwise <= 2, "%s: bad eltwise count", who);
  ITEXHIP_REQUIRE(ep->n_scales == 0 || ep->n_scales == 1 || ep->n_scales == N,
                  "%s: %d scales for %lld channels", who, ep->n_scales, static_cast<long long>(N));
  if (M == 0 || N == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(out != nullptr, "%s: null output", who);
  ITEXHIP_REQUIRE(K == 0 || (a && b), "%s: null operand", who);
  ITEXHIP_REQUIRE(ep->n_scales == 0 || scales, "%s: null scales", who);
  return ITEXHIP_OK;
}

EpilogueArgs make_args(int a_type, const int32_t* colsum, const float* scales, const float* bias,
                       const itexhip_epilogue* ep) {
  EpilogueArgs e{};
  e.scales = scales;
  e.bias = bias;
  e.colsum = colsum;
  e.n_scales = ep->n_scales;
  e.comp_mul = (a_type == ITEXHIP_QUINT8) ? 128 : 0;
  e.n_eltwise = ep->n_eltwise;
  e.elt[0] = ep->elt[0];
  e.elt[1] = ep->elt[1];
  return e;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int OUT_T>
int launch_tile(const uint8_t* a, uint32_t a_xor, const uint8_t* bp, int M, int K, int N,
                const EpilogueArgs& e, void* out, hipStream_t st) {
  const int KT = (K + 63) / 64, NT = (N + 15) / 16;
  const int num_m = (M + BM - 1) / BM, num_n = (N + BN - 1) / BN;
  constexpr size_t lds_bytes = 2 * (BM / 16 + BN / 16) * kChunkBytes;
  auto kern = qgemm_tile_kernel<BM, BN, WAVES_M, WAVES_N, OUT_T>;
  static bool attr_set = false;  // benign race: the call is idempotent
  if (!attr_set) {
    hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (err != hipSuccess) return hip_fail(err, "hipFuncSetAttribute(qgemm_tile_kernel)");
    attr_set = true;
  }
  kern<<<dim3(static_cast<unsigned>(num_m * num_n)), dim3(64 * WAVES_M * WAVES_N), lds_bytes, st>>>(
      a, a_xor, bp, M, K, N, KT, NT, num_m, num_n, e, out);
  return ITEXHIP_OK;
}

template <int OUT_T>
int dispatch_tile(const uint8_t* a, uint32_t a_xor, const uint8_t* bp, int M, int K, int N,
                  const EpilogueArgs& e, void* out, hipStream_t st) {
  // pick the largest tile that still gives every CU work
  const int64_t tiles_256 = static_cast<int64_t>((M + 255) / 256) * ((N + 255) / 256);
  const int64_t tiles_128 = static_cast<int64_t>((M + 127) / 128) * ((N + 127) / 128);
  if (tiles_256 >= 256) return launch_tile<256, 256, 2, 2, OUT_T>(a, a_xor, bp, M, K, N, e, out, st);
  if (tiles_128 >= 256) return launch_tile<128, 128, 2, 2, OUT_T>(a, a_xor, bp, M, K, N, e, out, st);
  return launch_tile<64, 64, 2, 2, OUT_T>(a, a_xor, bp, M, K, N, e, out, st);
}

template <int OUT_T>
int dispatch_gemv(const uint8_t* a, uint32_t a_xor, const uint8_t* bp, int M, int K, int N,
                  const EpilogueArgs& e, void* out, hipStream_t st) {
  const int KT = (K + 63) / 64, NT = (N + 15) / 16;
  if (KT >= 128)
    qgemv_kernel<16, OUT_T><<<NT, 64 * 16, 0, st>>>(a, a_xor, bp, M, K, N, KT, e, out);
  else if (KT >= 32)
    qgemv_kernel<8, OUT_T><<<NT, 64 * 8, 0, st>>>(a, a_xor, bp, M, K, N, KT, e, out);
  else
    qgemv_kernel<2, OUT_T><<<NT, 64 * 2, 0, st>>>(a, a_xor, bp, M, K, N, KT, e, out);
  return ITEXHIP_OK;
}

#define ITEXHIP_DISPATCH_OUT(out_type, CALL)                                  \
  switch (out_type) {                                                         \
    case ITEXHIP_FLOAT: st__ = CALL(ITEXHIP_FLOAT); break;                    \
    case ITEXHIP_QINT32: st__ = CALL(ITEXHIP_QINT32); break;                  \
    case ITEXHIP_QINT8: st__ = CALL(ITEXHIP_QINT8); break;                    \
    default: st__ = CALL(ITEXHIP_QUINT8); break;                              \
  }

int packed_path(bool gemv, const void* a, int a_type, const int8_t* packed_b, const int32_t* colsum,
                int64_t M, int64_t K, int64_t N, const float* scales, const float* bias,
                const itexhip_epilogue* ep, int out_type, void* out, void* stream, const char* who) {
  if (int st = check_common(a, a_type, packed_b, M, K, N, scales, ep, out_type, out, who)) return st;
  if (M == 0 || N == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(K % 16 == 0, "%s: K must be a multiple of 16 (got %lld); use itexhip_qgemm_naive", who,
                  static_cast<long long>(K));
  ITEXHIP_REQUIRE(aligned(a, 16) && aligned(packed_b, 16), "%s: operands must be 16-byte aligned", who);
  ITEXHIP_REQUIRE(a_type != ITEXHIP_QUINT8 || colsum, "%s: quint8 activations need colsum", who);
  ITEXHIP_REQUIRE(!gemv || M <= 16, "%s: M must be <= 16", who);
  const uint32_t a_xor = (a_type == ITEXHIP_QUINT8) ? 0x80808080u : 0u;
  const EpilogueArgs e = make_args(a_type, colsum, scales, bias, ep);
  const uint8_t* ap = reinterpret_cast<const uint8_t*>(a);
  const uint8_t* bp = reinterpret_cast<const uint8_t*>(packed_b);
  hipStream_t hs = as_stream(stream);
  const int Mi = static_cast<int>(M), Ki = static_cast<int>(K), Ni = static_cast<int>(N);
  int st__ = ITEXHIP_OK;
  if (gemv) {
#define CALL_GEMV(T) dispatch_gemv<T>(ap, a_xor, bp, Mi, Ki, Ni, e, out, hs)
    ITEXHIP_DISPATCH_OUT(out_type, CALL_GEMV)
#undef CALL_GEMV
  } else {
#define CALL_TILE(T) dispatch_tile<T>(ap, a_xor, bp, Mi, Ki, Ni, e, out, hs)
    ITEXHIP_DISPATCH_OUT(out_type, CALL_TILE)
#undef CALL_TILE
  }
  if (st__ != ITEXHIP_OK) return st__;
  ITEXHIP_CHECK_LAUNCH(who);
  return ITEXHIP_OK;
}

}  // namespace
}  // namespace itexhip

using namespace itexhip;

extern "C" int64_t itexhip_qgemm_packed_bytes(int64_t K, int64_t N) {
  if (K < 0 || N < 0) return -1;
  return ((N + 15) / 16) * ((K + 63) / 64) * kChunkBytes;
}

extern "C" int itexhip_qgemm_prepack_b(const int8_t* w, int transpose_b, int64_t K, int64_t N,
                                       int8_t* packed, int32_t* colsum, void* stream) {
  ITEXHIP_REQUIRE(K >= 0 && N >= 0 && K <= kMaxK && N < (1LL << 31), "itexhip_qgemm_prepack_b: bad dimensions");
  if (N == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(colsum != nullptr, "itexhip_qgemm_prepack_b: null colsum");
  hipStream_t st = as_stream(stream);
  zero_i32_kernel<<<static_cast<unsigned>((N + 255) / 256), 256, 0, st>>>(colsum, N);
  if (K > 0) {
    ITEXHIP_REQUIRE(w && packed, "itexhip_qgemm_prepack_b: null buffer");
    ITEXHIP_REQUIRE(aligned(packed, 16), "itexhip_qgemm_prepack_b: packed buffer must be 16-byte aligned");
    const int KT = static_cast<int>((K + 63) / 64), NT = static_cast<int>((N + 15) / 16);
    const int64_t chunks = static_cast<int64_t>(KT) * NT;
    prepack_b_kernel<<<static_cast<unsigned>((chunks + 3) / 4), 256, 0, st>>>(
        w, transpose_b, static_cast<int>(K), static_cast<int>(N), KT, NT, packed, colsum);
  }
  ITEXHIP_CHECK_LAUNCH("itexhip_qgemm_prepack_b");
  return ITEXHIP_OK;
}

extern "C" int itexhip_qgemm_tile(const void* a, int a_type, const int8_t* packed_b, const int32_t* colsum,
                                  int64_t M, int64_t K, int64_t N, const float* scales, const float* bias,
                                  const itexhip_epilogue* ep, int out_type, void* out, void* stream) {
  return packed_path(false, a, a_type, packed_b, colsum, M, K, N, scales, bias, ep, out_type, out, stream,
                     "itexhip_qgemm_tile");
}

extern "C" int itexhip_qgemv(const void* a, int a_type, const int8_t* packed_b, const int32_t* colsum,
                             int64_t M, int64_t K, int64_t N, const float* scales, const float* bias,
                             const itexhip_epilogue* ep, int out_type, void* out, void* stream) {
  return packed_path(true, a, a_type, packed_b, colsum, M, K, N, scales, bias, ep, out_type, out, stream,
                     "itexhip_qgemv");
}

extern "C" int itexhip_qgemm(const void* a, int a_type, const int8_t* packed_b, const int32_t* colsum,
                             int64_t M, int64_t K, int64_t N, const float* scales, const float* bias,
                             const itexhip_epilogue* ep, int out_type, void* out, void* stream) {
  return packed_path(M <= 16, a, a_type, packed_b, colsum, M, K, N, scales, bias, ep, out_type, out, stream,
                     "itexhip_qgemm");
}

extern "C" int itexhip_qgemm_naive(const void* a, int a_type, const int8_t* w, int transpose_b, int64_t M,
                                   int64_t K, int64_t N, const float* scales, const float* bias,
                                   const itexhip_epilogue* ep, int out_type, void* out, void* stream) {
  if (int st = check_common(a, a_type, w, M, K, N, scales, ep, out_type, out, "itexhip_qgemm_naive")) return st;
  if (M == 0 || N == 0) return ITEXHIP_OK;
  EpilogueArgs e = make_args(a_type, nullptr, scales, bias, ep);
  e.comp_mul = 0;  // the naive kernel multiplies unsigned activations directly
  const unsigned grid = static_cast<unsigned>((M * N + 255) / 256);
  const uint8_t* ap = reinterpret_cast<const uint8_t*>(a);
  const int a_is_u8 = a_type == ITEXHIP_QUINT8;
  hipStream_t hs = as_stream(stream);
  const int Mi = static_cast<int>(M), Ki = static_cast<int>(K), Ni = static_cast<int>(N);
  switch (out_type) {
    case ITEXHIP_FLOAT:
      qgemm_naive_kernel<ITEXHIP_FLOAT><<<grid, 256, 0, hs>>>(ap, a_is_u8, w, transpose_b, Mi, Ki, Ni, e, out);
      break;
    case ITEXHIP_QINT32:
      qgemm_naive_kernel<ITEXHIP_QINT32><<<grid, 256, 0, hs>>>(ap, a_is_u8, w, transpose_b, Mi, Ki, Ni, e, out);
      break;
    case ITEXHIP_QINT8:
      qgemm_naive_kernel<ITEXHIP_QINT8><<<grid, 256, 0, hs>>>(ap, a_is_u8, w, transpose_b, Mi, Ki, Ni, e, out);
      break;
    default:
      qgemm_naive_kernel<ITEXHIP_QUINT8><<<grid, 256, 0, hs>>>(ap, a_is_u8, w, transpose_b, Mi, Ki, Ni, e, out);
      break;
  }
  ITEXHIP_CHECK_LAUNCH("itexhip_qgemm_naive");
  return ITEXHIP_OK;
}
