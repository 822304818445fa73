// Quantized MatMul on gfx950: u8/s8 activations x s8 weights -> exact int32 accumulation on the i8
// MFMA (v_mfma_i32_32x32x32_i8: one wavefront alone keeps the matrix pipe ~94% busy with it, against
// ~60% with the 16x16x64 form), fused fp32 epilogue in registers.
//
// Operand roles.  The weight is the MFMA "A" operand (its 32 rows are 32 output channels n), the
// activation is the "B" operand (its 32 columns are 32 rows m of the activation matrix).  A lane then
// ends up with groups of 4 consecutive output channels of one output row, which is what a row-major
// [M,N] output wants (4 int8 = one dword store, 4 fp32 = one 16-byte store).
//
// Operand tile ("chunk") = 32 rows x 32 k = 1 KiB, stored in lane order: lane l holds 16 consecutive
// k of row (l % 32), k-group (l / 32).  The prepacked weight is the sequence of such chunks
// [n/32][k/32] with k padded to a multiple of 64; activation chunks are formed on the fly.  Both
// operands use the same (lane, byte) -> k mapping, so the order in which the instruction consumes k
// inside a chunk cannot affect the integer sum.
//
// Unsigned activations: the MFMA is signed x signed, so u8 values are fed as (a ^ 0x80) = a - 128 and
// the epilogue adds 128 * colsum[n] back (exact: |acc| <= 255 * 127 * K stays far below 2^31 for the
// K this library accepts).
#include "qgemm_common.hpp"

namespace itexhip {

// MFMA tile kernels, one translation unit per output type (qgemm_tile_*.hip)
template <int OUT_T>
int dispatch_tile(const uint8_t* a, uint32_t a_xor, const uint8_t* bp, int M, int K, int N,
                  const EpilogueArgs& e, void* out, hipStream_t st);

namespace {

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
  const int n = nt * kChunkRows + (lane & 31);
  const int k0 = kt * kChunkK + (lane >> 5) * 16;
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
  // add up the two k-groups of this row, then one atomic per row and chunk
  sum += __shfl_xor(sum, 32, 64);
  if (lane < 32 && n < N && sum != 0) atomicAdd(&colsum[n], sum);
}

// ------------------------------------------------------------------------------------------------
// Small-M kernel (M <= 16, bandwidth bound on the weight).  One workgroup owns a 16-channel strip of
// the weight (half of each 32-channel chunk), so that even N = 4096 gives every CU a workgroup.  Its
// WAVES wavefronts take pairs of consecutive k-chunks round-robin; one wavefront load fetches the
// strip's half of a chunk pair (4 runs of 256 contiguous bytes) in the operand layout of the
// 16x16x64 MFMA: lane l holds channel (l % 16), k-group (l / 16) of the 64 k of the pair.  A batch of
// UNROLL loads is issued before the first MFMA of the batch.  The partial 16x16 tiles of the
// wavefronts are added up in LDS with integer atomics (exact, order free).
// ------------------------------------------------------------------------------------------------
template <int WAVES, int OUT_T>
__global__ __launch_bounds__(64 * WAVES) void qgemv_kernel(const uint8_t* __restrict__ a, uint32_t a_xor,
                                                           const uint8_t* __restrict__ bp, int M, int K,
                                                           int N, int KC, EpilogueArgs e,
                                                           void* __restrict__ out) {
  constexpr int UNROLL = 16;  // weight loads in flight per wavefront
  __shared__ int red[4 * 64];
  const int strip = blockIdx.x;  // 16 channels
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lrow = lane & 15, lgrp = lane >> 4;  // k-group 0..3 of the chunk pair
  const int KP = KC >> 1;                         // chunk pairs (K is padded to a multiple of 64)
  // inside chunk (pair * 2 + lgrp / 2): slot (lgrp % 2) * 32 + (strip % 2) * 16 + lrow
  const uint8_t* wsrc = bp + (static_cast<int64_t>(strip >> 1) * KC + (lgrp >> 1)) * kChunkBytes +
                        (((lgrp & 1) * 32 + (strip & 1) * 16 + lrow) << 4);
  const uint8_t* arow = a + static_cast<int64_t>(lrow) * K + lgrp * 16;
  const bool row_ok = lrow < M;

  v4i acc = v4i{0, 0, 0, 0};
  auto act_piece = [&](int kp) {
    v4i v = v4i{0, 0, 0, 0};
    if (row_ok && kp * 64 + lgrp * 16 < K) {
      v = *reinterpret_cast<const v4i*>(arow + static_cast<int64_t>(kp) * 64);
      v.x ^= a_xor; v.y ^= a_xor; v.z ^= a_xor; v.w ^= a_xor;
    }
    return v;
  };
  // batches of up to UNROLL chunk pairs: every weight load of a batch is issued first (the guard is
  // wavefront uniform), activations are read just before use (they come from L2)
  for (int kp0 = wave; kp0 < KP; kp0 += UNROLL * WAVES) {
    v4i w[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int kp = kp0 + u * WAVES;
      w[u] = v4i{0, 0, 0, 0};
      if (kp < KP)
        w[u] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wsrc + static_cast<int64_t>(kp) * (2 * kChunkBytes)));
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int kp = kp0 + u * WAVES;
      if (kp < KP) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[u], act_piece(kp), acc, 0, 0, 0);
    }
  }

  // cross-wavefront reduction: wavefront 0 stores, the others add
  if (wave == 0) {
#pragma unroll
    for (int r = 0; r < 4; ++r) red[r * 64 + lane] = acc[r];
  }
  __syncthreads();
  if (wave != 0) {
#pragma unroll
    for (int r = 0; r < 4; ++r) atomicAdd(&red[r * 64 + lane], acc[r]);
  }
  __syncthreads();
  if (wave == 0 && row_ok) {
    // accumulator layout of the 16x16 MFMA: lane l, register r -> m = l % 16, n = (l / 16) * 4 + r
    const bool vec_ok = (N & 3) == 0 && aligned16(e.scales) && aligned16(e.bias) && aligned16(e.colsum) && aligned16(out);
    const int n = strip * 16 + lgrp * 4;
    if (n < N) {
      const v4i part = v4i{red[lane], red[64 + lane], red[128 + lane], red[192 + lane]};
      const ChannelParams p = load_channel_params(e, n, N, vec_ok);
      epilogue_store<OUT_T, 2>(part, p, lrow, n, M, N, e, out, vec_ok);
    }
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

template <int OUT_T>
int dispatch_gemv(const uint8_t* a, uint32_t a_xor, const uint8_t* bp, int M, int K, int N,
                  const EpilogueArgs& e, void* out, hipStream_t st) {
  const int KC = 2 * ((K + 63) / 64), strips = (N + 15) / 16;
  const int KP = KC / 2;
  // as many wavefronts per strip as it takes for each to own at most ~16 chunk pairs (one batch of
  // loads), within 16 per workgroup; small problems get fewer
  const int per16 = (KP + 15) / 16;
  if (per16 > 8)
    qgemv_kernel<16, OUT_T><<<strips, 64 * 16, 0, st>>>(a, a_xor, bp, M, K, N, KC, e, out);
  else if (per16 > 2 || KP >= 64)
    qgemv_kernel<8, OUT_T><<<strips, 64 * 8, 0, st>>>(a, a_xor, bp, M, K, N, KC, e, out);
  else if (KP >= 4)
    qgemv_kernel<4, OUT_T><<<strips, 64 * 4, 0, st>>>(a, a_xor, bp, M, K, N, KC, e, out);
  else
    qgemv_kernel<1, OUT_T><<<strips, 64, 0, st>>>(a, a_xor, bp, M, K, N, KC, e, out);
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
  ITEXHIP_REQUIRE(M * K < (1LL << 31), "%s: activation matrix too large (M * K must be < 2^31)", who);
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
  return ((N + kChunkRows - 1) / kChunkRows) * (2 * ((K + 63) / 64)) * kChunkBytes;
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
    const int KT = 2 * static_cast<int>((K + 63) / 64), NT = static_cast<int>((N + kChunkRows - 1) / kChunkRows);
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
