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
#include <algorithm>

#include "qgemm_common.hpp"

namespace itexhip {

// MFMA tile kernels, one translation unit per output type (qgemm_tile_*.hip)
template <int OUT_T>
int dispatch_tile(const uint8_t* a, uint32_t a_xor, const uint8_t* bp, int M, int K, int N,
                  const EpilogueArgs& e, void* out, hipStream_t st);

template <int OUT_T>
int dispatch_tile_conv(const uint8_t* x, uint32_t a_xor, const uint8_t* bp, int M, int K, int N, const EpilogueArgs& e,
                       void* out, hipStream_t st, const ConvTileArgs& cv);

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
// Small-M kernel (bandwidth bound on the weight).  One workgroup owns a strip of 16 * NT output channels and a block
// of 16 R rows (M <= 16: R = 1, the whole problem's rows; up to 128 rows in blocks of 32, R = 2, whose workgroups
// share the strip's weights through one L2) (NT = 2: whole chunks; NT = 1: one half of each chunk, when N alone would not give every CU a
// workgroup); its wavefronts split K into contiguous runs of chunk pairs (64 k each).  Per chunk pair a
// wavefront needs NT weight fragments in the operand layout of the 16x16x64 MFMA (lane l: channel l % 16,
// k-group l / 16; 4 runs of 256 contiguous bytes of the packed weight, loaded to registers) and one
// activation fragment (lane l: row l % 16, the 16 bytes of k-group l / 16).  Loading that fragment straight
// from the row-major activations would put 64 lanes on 64 different 16-byte pieces of 16 rows, which the
// texture addresser serves at a quarter of its rate; instead the 16 rows x 64 bytes travel by a direct
// global -> LDS load whose lanes are contiguous in groups of four (lane 4 q + j: row q, piece
// j ^ ((q >> 2) & 3)) into a 1 KiB slot of a ring private to the wavefront, and the fragment is read back
// from LDS (the rotation of the pieces makes that read conflict free: the 16 lanes served per LDS cycle read 16
// rows, whose slots 4 q + (j ^ (q >> 2)) fall into 16 different bank groups).  The loads of a batch of U pairs
// are issued while the previous batch is multiplied, so 2 U (NT + 1) KiB per wavefront are in flight.
// The partial 16x16 tiles of the wavefronts meet in LDS (the rings, free by then; one barrier) and
// wavefront t finishes tile t.  One more wavefront per workgroup streams nothing: it resolves the strip's
// channel parameters (a chain of dependent kernel-argument and vector loads, then divisions) while the others
// stream, so that no streaming wavefront starts its loads late or stops for arithmetic.  Rows >= M of the
// activation operand repeat row M - 1; their results are never stored.  Pairs past the end of a wavefront's
// run are loaded from clamped addresses and not used.
// ------------------------------------------------------------------------------------------------
constexpr int kGemvBatch = 4;                 // chunk pairs per batch of the 32-row kernel (2 for up to 16 rows, see UB below)
constexpr int kGemvPanelWords = 6 + 32;       // per channel of the strip: 6 parameter words + {scale, bias} of 16 rows

// UB: chunk pairs per batch; two batches of a wavefront are in flight.  2 for up to 16 rows, 4 for the blocks of 32
// rows.  Measured on 4096 -> 14336 / 14336 -> 4096 with the wavefront counts the host picks for each: M = 4 11.6 -> 10.95
// and 11.3 -> 11.0 us, M = 1 11.3 -> 10.95 us and unchanged, M = 16 unchanged and 13.0 -> 12.7 us against batches of 4
// (a form that fetched the 4 rows of a whole batch of 4 pairs in one load of 4 x 256 bytes was no faster and is gone);
// batches of 1 or 3 are slower everywhere, and with 32 rows batches of 2 lose on long K.
template <int NT, int OUT_T, int R, int UB = kGemvBatch>
__global__ __launch_bounds__(576) void qgemv_kernel(const uint8_t* __restrict__ a, uint32_t a_xor,
                                                     const uint8_t* __restrict__ bp, int M, int K, int N,
                                                     int KC, int cnt, EpilogueArgs e,
                                                     void* __restrict__ out) {
  constexpr int SW = 16 * NT;
  constexpr int U = UB, RING = 2 * UB;  // RING: activation slots of 1 KiB per wavefront and row block
  constexpr int L = U * (NT + R);       // loads per batch
  static_assert(RING >= NT, "the partial tiles of a wavefront are handed over in its own ring");
  constexpr int ROWS = 16 * R;     // activation rows per workgroup
  // Per-row activation ranges (M <= 16): the parameter wavefront works out scale and bias of every (row, channel) of
  // the strip while the others stream, and the epilogue reads a table (14336 -> 4096, M = 16: 14.9 -> 13.9 us; 32-channel
  // strips, 4096 -> 14336: 13.0 -> 12.1 us once that wavefront fetched the 16 rows' ranges in one round trip instead of
  // one per table entry - before that it finished last there).
  extern __shared__ __align__(16) uint8_t smem[];  // [waves][RING][R][1 KiB], then the parameter panel [3 or 6][SW]
  // R = 1 (M <= 16): one workgroup per strip.  R = 2 (M > 16): a workgroup takes 32 rows of a strip - every weight
  // fragment meets two activation fragments - and the grid is x = 8 * row blocks, y = groups of 8 strips (x runs
  // fastest in launch order, consecutive workgroup ids go round robin to the 8 XCDs): the row blocks of a strip get
  // ids 8 apart, so they run at the same time on the same XCD and its L2 fetches the strip's weights once.  The grid
  // is padded to whole groups of 8 strips.
  const int strip = R > 1 ? blockIdx.y * 8 + (blockIdx.x & 7) : blockIdx.x;
  const int m_base = R > 1 ? (blockIdx.x >> 3) * ROWS : 0;
  if (R > 1 && strip * SW >= N) return;
  const int waves = (blockDim.x >> 6) - 1;  // streaming wavefronts; one more resolves the channel parameters
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int lrow = lane & 15, lgrp = lane >> 4;  // fragment lane: row / channel, k-group 0..3 of the chunk pair
  const int KP = KC >> 1;                         // chunk pairs (K is padded to a multiple of 64)
  const int p0 = wave * cnt, p1 = min(KP, p0 + cnt);
  // inside chunk (pair * 2 + lgrp / 2): slot (lgrp % 2) * 32 + half * 16 + lrow
  const int chunk_row = (NT == 2) ? strip : (strip >> 1);
  const int half0 = (NT == 2) ? 0 : (strip & 1);
  const uint8_t* wsrc = bp + (static_cast<int64_t>(chunk_row) * KC + (lgrp >> 1)) * kChunkBytes +
                        (((lgrp & 1) * 32 + half0 * 16 + lrow) << 4);
  // activation staging: lane -> (row q, piece j) of the 16 x 64 byte tile
  const int q = lane >> 2;
  const int dpiece = ((lane & 3) ^ ((q >> 2) & 3)) * 16;
  const uint8_t* arow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) arow[r] = a + static_cast<int64_t>(min(m_base + 16 * r + q, M - 1)) * K;
  const int klast = K - 16;  // k beyond K meets zero weights: any in-bounds data will do
  uint8_t* const ring = smem + wave * (RING * R * 1024);
  const uint32_t frag_off = static_cast<uint32_t>((4 * lrow + (lgrp ^ ((lrow >> 2) & 3))) * 16);

  v4i acc[R][NT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[r][t] = v4i{0, 0, 0, 0};

  int* const panel = reinterpret_cast<int*>(smem + waves * (RING * R * 1024));

  // Batches that lie entirely inside the wavefront's run and inside K take their addresses from two running per-lane
  // pointers plus constants; the last, ragged batch clamps every pair (a pair past the end is loaded from a valid
  // address and not used).
  const uint8_t* wptr = wsrc + static_cast<int64_t>(p0) * (2 * kChunkBytes);
  const uint8_t* aptr[R];
#pragma unroll
  for (int r = 0; r < R; ++r) aptr[r] = arow[r] + dpiece + static_cast<int64_t>(p0) * 64;
  const int p_full = min(p1, K >> 6);  // pairs below this index lie entirely inside K
  auto issue = [&](int pb, int slot0, v4i (&w)[U][NT]) {
    if (pb + U <= p_full) {
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int r = 0; r < R; ++r)
          // the builtin, not inline assembly: the compiler's own vmcnt bookkeeping for the weight loads must see these
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(aptr[r] + u * 64),
                                           (__attribute__((address_space(3))) void*)(ring + ((slot0 + u) * R + r) * 1024), 16, 0, 0);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t)
          w[u][t] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wptr + u * (2 * kChunkBytes) + t * 256));
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = min(pb + u, KP - 1);
#pragma unroll
        for (int r = 0; r < R; ++r)
          __builtin_amdgcn_global_load_lds(
              (const __attribute__((address_space(1))) void*)(arow[r] + min(p * 64 + dpiece, klast)),
              (__attribute__((address_space(3))) void*)(ring + ((slot0 + u) * R + r) * 1024), 16, 0, 0);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = min(pb + u, KP - 1);
#pragma unroll
        for (int t = 0; t < NT; ++t)
          w[u][t] = __builtin_nontemporal_load(
              reinterpret_cast<const v4i*>(wsrc + static_cast<int64_t>(p) * (2 * kChunkBytes) + t * 256));
      }
    }
    wptr += U * (2 * kChunkBytes);
#pragma unroll
    for (int r = 0; r < R; ++r) aptr[r] += U * 64;
    __builtin_amdgcn_sched_barrier(0);
  };
  auto compute = [&](int pb, int slot0, const v4i (&w)[U][NT]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (pb + u < p1) {  // wavefront uniform
#pragma unroll
        for (int r = 0; r < R; ++r) {
          v4i x = *reinterpret_cast<const v4i*>(ring + ((slot0 + u) * R + r) * 1024 + frag_off);
          x.x ^= a_xor; x.y ^= a_xor; x.z ^= a_xor; x.w ^= a_xor;
#pragma unroll
          for (int t = 0; t < NT; ++t) acc[r][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[u][t], x, acc[r][t], 0, 0, 0);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // wait until at most the next batch's loads of this wavefront are outstanding (they complete in order), then let
  // the LDS reads of the staged activations go ahead
  auto landed = [&](bool next_in_flight) {
    if (next_in_flight) wait_vmcnt<L>(); else wait_vmcnt<0>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };

  if (wave == waves) {
    // The extra wavefront resolves the strip's channel parameters, one channel per lane, while the others stream:
    // fetching pointers and flags from the kernel arguments (a chain of dependent scalar loads), the parameter loads
    // and the arithmetic (divisions) all stay off the streaming wavefronts' instruction streams.
    if (lane < SW) {
      const RawChannel raw = load_raw_channel(e, min(strip * SW + lane, N - 1), N);
      if (e.row_min_a) {  // per-row ranges: the epilogue lanes finish the arithmetic for their own row
        panel[lane] = raw.colsum;
        panel[SW + lane] = __float_as_int(raw.min_bj);
        panel[2 * SW + lane] = __float_as_int(raw.max_bj);
        panel[3 * SW + lane] = __float_as_int(raw.min_b0);
        panel[4 * SW + lane] = __float_as_int(raw.max_b0);
        panel[5 * SW + lane] = __float_as_int(bias_from_bits(e.prep, raw.bias));
      } else {
        int comp;
        float scale, bias;
        finish_channel(e, raw, &comp, &scale, &bias);
        panel[lane] = comp;
        panel[SW + lane] = __float_as_int(scale);
        panel[2 * SW + lane] = __float_as_int(bias);
      }
    }
    if (e.row_min_a) {
      // Per-row ranges: scale and bias of every (row, channel) of the strip, 16 * SW pairs over the 64 lanes, worked
      // out here while the other wavefronts stream (the raw channel values come back from the panel: LDS operations
      // of one wavefront complete in order).  The epilogue then only reads the table.
      float* const rowtab = reinterpret_cast<float*>(panel + 6 * SW);  // [16][SW]{scale, bias}
      // the 16 rows' ranges: one round trip to memory for all of them (lane r holds row r), handed round by lane index
      float rmin = 0.0f, rmax = 0.0f;
      if (lane < 16 && m_base + lane < M) {
        rmin = e.row_min_a[m_base + lane];
        rmax = e.row_max_a[m_base + lane];
      }
      for (int idx = lane; idx < 16 * SW; idx += 64) {
        const int mm = idx / SW, c = idx - mm * SW;
        const float lo = __shfl(rmin, mm, 64), hi = __shfl(rmax, mm, 64);
        if (m_base + mm < M) {
          PrepArgs pr = e.prep;
          pr.min_a = lo;
          pr.max_a = hi;
          const ChannelScaleBias cs = channel_scale_bias(
              pr, __int_as_float(panel[SW + c]), __int_as_float(panel[2 * SW + c]), __int_as_float(panel[3 * SW + c]),
              __int_as_float(panel[4 * SW + c]), __int_as_float(panel[5 * SW + c]), panel[c]);
          rowtab[2 * idx] = e.n_scales > 0 ? cs.scale : 1.0f;
          rowtab[2 * idx + 1] = cs.bias;
        }
      }
    }
  } else {
    v4i w0[U][NT], w1[U][NT];
    int pb = p0;
    if (pb < p1) issue(pb, 0, w0);
    while (pb < p1) {
      const bool more1 = pb + U < p1;
      if (more1) issue(pb + U, U, w1);
      landed(more1);
      compute(pb, 0, w0);
      pb += U;
      if (!more1) break;
      const bool more2 = pb + U < p1;
      if (more2) issue(pb + U, 0, w0);
      landed(more2);
      compute(pb, U, w1);
      pb += U;
    }
    // partial tiles -> the wavefront's own ring (its loads have landed and its reads are done)
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int t = 0; t < NT; ++t) *reinterpret_cast<v4i*>(ring + (r * NT + t) * 1024 + lane * 16) = acc[r][t];
  }
  // cross-wavefront reduction through the rings
  __syncthreads();
  // the R * NT tiles of 16 x 16 go round the wavefronts (R = 1: wavefront t finishes tile t)
  for (int tile = wave; tile < R * NT; tile += waves + 1) {
    const int tr = tile / NT, tc = tile - tr * NT;
    v4i part = v4i{0, 0, 0, 0};
    for (int w = 0; w < waves; ++w) part += *reinterpret_cast<const v4i*>(smem + w * (RING * R * 1024) + tile * 1024 + lane * 16);
    // accumulator layout of the 16x16 MFMA: lane l, register r -> m = l % 16, n = (l / 16) * 4 + r
    const bool vec_ok = (N & 3) == 0 && aligned16(out);
    const int col = tc * 16 + lgrp * 4, n = strip * SW + col;
    const int m = m_base + 16 * tr + lrow;
    if (m < M && n < N) {
      ChannelParams cp;
      if (e.row_min_a) {
        const float* const rowtab = reinterpret_cast<const float*>(panel + 6 * SW) + 2 * ((m - m_base) * SW + col);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          cp.comp[r] = e.comp_mul * panel[col + r];
          cp.scale[r] = rowtab[2 * r];
          cp.bias[r] = rowtab[2 * r + 1];
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          cp.comp[r] = panel[col + r];
          cp.scale[r] = __int_as_float(panel[SW + col + r]);
          cp.bias[r] = __int_as_float(panel[2 * SW + col + r]);
        }
      }
      epilogue_store<OUT_T, 2>(part, cp, m, n, M, N, e, out, vec_ok);
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Matrix-pipe probe: every wavefront issues `iters` x 8 independent 32x32x32 i8 MFMAs back to back on
// operands taken from `operands` (8 KiB: 4 A and 4 B fragments per lane), no other instruction in the
// loop.  Timing it gives the rate the matrix cores sustain for that operand data: the clock under
// MFMA load depends on how much the operand bits toggle, so the ceiling for quantized data sits well
// below the rate for constant operands.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void mfma_probe_kernel(int iters, const v4i* __restrict__ operands, int* __restrict__ sink) {
  v16i acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[i][j] = 0;
  v4i a[4], b[4];
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = operands[i * 64 + lane];
    b[i] = operands[(4 + i) * 64 + lane];
  }
  // as in the tile kernel: the first operand (weights there) stays for 4 MFMAs, the second (activations) changes with
  // every one; which operand carries which data, and how often it changes, moves the sustained rate by ~10 %
  for (int it = 0; it < iters; it += 2) {  // iters is even (host)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i >> 2], b[i & 3], acc[i], 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[2 + (i >> 2)], b[i & 3], acc[i], 0, 0, 0);
  }
  int s = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += acc[i][j];
  if (s == 0x7fffffff) sink[threadIdx.x] = s;  // keeps the accumulators alive; practically never taken
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
  if (e.bias) v = v + static_cast<const float*>(e.bias)[n];
  for (int k = 0; k < e.n_eltwise; ++k) v = apply_eltwise(e.elt[k], v);  // no sum post-op on this path
  store_output<OUT_T>(out, idx, v);
}

// The whole op on the unpacked weight, any K: the thread also sums its weight column (the zero-point
// compensation needs it) and derives the channel's scale and bias like the packed kernels do.
template <int OUT_T>
__global__ __launch_bounds__(256) void qmatmul_unpacked_kernel(const uint8_t* __restrict__ a, int a_is_u8,
                                                                const int8_t* __restrict__ w, int transpose_b,
                                                                int M, int K, int N, EpilogueArgs e,
                                                                void* __restrict__ out) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(M) * N) return;
  const int m = static_cast<int>(idx / N), n = static_cast<int>(idx % N);
  int acc = 0, wsum = 0;
  for (int k = 0; k < K; ++k) {
    const int av = a_is_u8 ? static_cast<int>(a[static_cast<int64_t>(m) * K + k])
                           : static_cast<int>(reinterpret_cast<const int8_t*>(a)[static_cast<int64_t>(m) * K + k]);
    const int wv = transpose_b ? w[static_cast<int64_t>(n) * K + k] : w[static_cast<int64_t>(k) * N + n];
    acc += av * wv;
    wsum += wv;
  }
  const int jb = (e.nb == N) ? n : 0;
  const ChannelScaleBias c = channel_scale_bias(e.prep, e.min_b[jb], e.max_b[jb], e.min_b[0], e.max_b[0],
                                                bias_entry(e.prep, e.bias, n), wsum);
  float v = static_cast<float>(acc);
  if (e.n_scales > 0) v = v * c.scale;
  v = v + c.bias;
  for (int k = 0; k < e.n_eltwise; ++k) {
    if (e.elt[k].alg == ITEXHIP_ELT_SUM) v = v + e.elt[k].alpha * load_addend(e, idx);
    else v = apply_eltwise(e.elt[k], v);
  }
  store_output<OUT_T>(out, idx, v);
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
int check_common(const void* a, int a_type, const void* b, int64_t M, int64_t K, int64_t N,
                 const float* scales, const itexhip_epilogue* ep, int out_type, const void* out,
                 const char* who, const void* addend = nullptr, int addend_type = 0) {
  ITEXHIP_REQUIRE(a_type == ITEXHIP_QUINT8 || a_type == ITEXHIP_QINT8, "%s: activation type must be quint8 or qint8", who);
  ITEXHIP_REQUIRE(out_type == ITEXHIP_QINT32 || out_type == ITEXHIP_QINT8 || out_type == ITEXHIP_QUINT8 ||
                      is_float_out(out_type), "%s: unsupported output type %d", who, out_type);
  ITEXHIP_REQUIRE(M >= 0 && K >= 0 && N >= 0, "%s: negative dimension", who);
  ITEXHIP_REQUIRE(M < (1LL << 31) && N < (1LL << 31) && K <= kMaxK, "%s: dimension too large (K <= %lld)", who,
                  static_cast<long long>(kMaxK));
  ITEXHIP_REQUIRE(ep != nullptr, "%s: null epilogue", who);
  ITEXHIP_REQUIRE(ep->n_eltwise >= 0 && ep->n_eltwise <= 3, "%s: bad eltwise count", who);
  int n_sum = 0;
  for (int k = 0; k < ep->n_eltwise; ++k) n_sum += ep->elt[k].alg == ITEXHIP_ELT_SUM;
  ITEXHIP_REQUIRE(n_sum == (addend != nullptr ? 1 : 0),
                  "%s: one sum post-op goes with an addend (itexhip_qgemm_sum / itexhip_qconv2d_sum / itexhip_qmatmul), none without", who);
  ITEXHIP_REQUIRE(addend == nullptr || addend_type == ITEXHIP_FLOAT || is_float16_type(addend_type) ||
                      addend_type == ITEXHIP_QINT8 || addend_type == ITEXHIP_QUINT8,
                  "%s: the addend must be float, bfloat16, half, qint8 or quint8", who);
  ITEXHIP_REQUIRE(ep->n_scales == 0 || ep->n_scales == 1 || ep->n_scales == N,
                  "%s: %d scales for %lld channels", who, ep->n_scales, static_cast<long long>(N));
  if (M == 0 || N == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(out != nullptr, "%s: null output", who);
  ITEXHIP_REQUIRE(K == 0 || (a && b), "%s: null operand", who);
  ITEXHIP_REQUIRE(ep->n_scales == 0 || scales, "%s: null scales", who);
  return ITEXHIP_OK;
}

EpilogueArgs make_args(int a_type, const int32_t* colsum, const float* scales, const void* bias,
                       const itexhip_epilogue* ep, const void* addend = nullptr, int addend_type = 0) {
  EpilogueArgs e{};
  e.addend = addend;
  e.addend_type = addend_type;
  e.scales = scales;
  e.bias = bias;
  e.colsum = colsum;
  e.n_scales = ep->n_scales;
  e.comp_mul = (a_type == ITEXHIP_QUINT8) ? 128 : 0;
  e.n_eltwise = ep->n_eltwise;
  e.elt[0] = ep->elt[0];
  e.elt[1] = ep->elt[1];
  e.elt[2] = ep->elt[2];
  return e;
}

inline int gemv_batch(int M) { return M <= 16 ? 2 : kGemvBatch; }  // chunk pairs per batch of the variant that takes M rows

template <int NT, int OUT_T>
int launch_gemv(const uint8_t* a, uint32_t a_xor, const uint8_t* bp, int M, int K, int N, int KC, int waves, int cnt,
                const EpilogueArgs& e, void* out, hipStream_t st) {
  // up to 16 rows: batches of 2 chunk pairs; more: blocks of 32 rows, batches of 4
  const int variant = M > 16 ? 1 : 0;
  auto kern = variant == 1 ? qgemv_kernel<NT, OUT_T, 2, 4> : qgemv_kernel<NT, OUT_T, 1, 2>;
  const int R = M > 16 ? 2 : 1;
  const int ring = 2 * gemv_batch(M);  // KiB per wavefront and row block
  // the kernel's table of per-row parameters holds 16 rows
  ITEXHIP_REQUIRE(e.row_min_a == nullptr || M <= 16, "the small-M kernel takes per-row activation ranges for M <= 16 only");
  const size_t lds_max = static_cast<size_t>(8 * ring * 1024) * R + kGemvPanelWords * 16 * NT * 4;
  static unsigned long long attr_done[2] = {0, 0};  // per variant: devices on which the attribute is set
  if (!device_bit(&attr_done[variant], false)) {
    hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         static_cast<int>(lds_max));
    if (err != hipSuccess) return hip_fail(err, "hipFuncSetAttribute(qgemv_kernel)");
    device_bit(&attr_done[variant], true);
  }
  const size_t lds = static_cast<size_t>(waves) * ring * 1024 * R + kGemvPanelWords * 16 * NT * 4;
  const int strips = (N + 16 * NT - 1) / (16 * NT);
  const int rbs = (M + 31) / 32;  // row blocks of the R = 2 kernel
  const dim3 grid = M > 16 ? dim3(8 * rbs, (strips + 7) / 8) : dim3(strips);
  kern<<<grid, 64 * (waves + 1), lds, st>>>(a, a_xor, bp, M, K, N, KC, cnt, e, out);
  return ITEXHIP_OK;
}

template <int OUT_T>
int dispatch_gemv(const uint8_t* a, uint32_t a_xor, const uint8_t* bp, int M, int K, int N,
                  const EpilogueArgs& e, void* out, hipStream_t st) {
  const int KC = 2 * ((K + 63) / 64), KP = KC / 2;
  // 32-channel strips when they give every CU a workgroup, else 16-channel strips; a strip is finished by one
  // wavefront per 16-channel tile, so never fewer wavefronts than that.  Wavefronts per strip, at most 8, measured on
  // 4096 x 14336 and 14336 x 4096 with every count from 2 to 8, both strip widths and both batch sizes: up to 4 rows
  // about 8 chunk pairs (four batches of 2) each (4096 -> 14336 at M = 1 / 4: 11.3 -> 10.95 us with 8 instead of 4);
  // 5 to 16 rows about 16 pairs each (4096 -> 14336 at M = 16: 4 wavefronts 11.7 us, 8 over 11.8 us; 14336 -> 4096: 8
  // wavefronts 12.7 us, 4 wavefronts 15.2 us); prefer a count that divides K into whole batches.
  // (blocks of 32 rows count as workgroups of their own: 14336 -> 4096 at M = 64 28.1 -> 20.0 us with 32-channel strips,
  // 256 workgroups instead of 512 that read the activations twice as often)
  const int row_blocks = M > 16 ? (M + 31) / 32 : 1;
  const int nt = ((N + 31) / 32) * row_blocks >= 256 ? 2 : 1;
  const int per_wave = M <= 4 ? 8 : 16;
  int waves = std::max(nt, std::min(8, (KP + per_wave - 1) / per_wave));
  for (int w = waves; w >= std::max(nt, waves / 2 + 1); --w)
    if (KP % (gemv_batch(M) * w) == 0) { waves = w; break; }
  // Blocks of 32 rows (batches of 4): half as many wavefronts with runs twice as long, fewer partial tiles to reduce
  // and fewer rings.
  if (M > 16) waves = std::max(nt, waves / 2);
  const int cnt = (KP + waves - 1) / waves;
  if (nt == 2) return launch_gemv<2, OUT_T>(a, a_xor, bp, M, K, N, KC, waves, cnt, e, out, st);
  return launch_gemv<1, OUT_T>(a, a_xor, bp, M, K, N, KC, waves, cnt, e, out, st);
}

#define ITEXHIP_DISPATCH_OUT(out_type, CALL)                                  \
  switch (out_type) {                                                         \
    case ITEXHIP_FLOAT: st__ = CALL(ITEXHIP_FLOAT); break;                    \
    case ITEXHIP_BFLOAT16: st__ = CALL(ITEXHIP_BFLOAT16); break;              \
    case ITEXHIP_HALF: st__ = CALL(ITEXHIP_HALF); break;                      \
    case ITEXHIP_QINT32: st__ = CALL(ITEXHIP_QINT32); break;                  \
    case ITEXHIP_QINT8: st__ = CALL(ITEXHIP_QINT8); break;                    \
    default: st__ = CALL(ITEXHIP_QUINT8); break;                              \
  }

// Which packed kernel takes a call.  The small-M kernel (a strip of channels x 16 rows x all of K per workgroup)
// streams the weight once per block of 16 rows; the tile kernel needs enough 64 x 64 tiles to fill the device.
// Measured on 4096 x 14336 / 14336 x 4096 weights (us, small-M against tile kernel): M = 32: 15 / 17 against 23 / 67;
// M = 64: 23 / 21 against 23 / 68; M = 128: 28 / 34 against 28 / 67; on a 1024 x 1024 weight the small-M kernel takes
// 3.6 against 4.8 up to M = 128.  Both kernels accumulate exactly and share the epilogue: the same bytes either way.
constexpr int kSmallMaxRows = 128;
static bool small_m(int64_t M, int64_t K, int64_t N) {
  if (M <= 32) return true;
  if (M > kSmallMaxRows) return false;
  if (K * N <= (8LL << 20)) return true;                       // the weight stays in L2: launch-bound either way
  return ((M + 63) / 64) * ((N + 63) / 64) <= 128;             // the tile kernel would leave half of the CUs idle
}

int launch_packed(bool gemv, const void* a, int a_type, const int8_t* packed_b, int64_t M, int64_t K, int64_t N,
                  const EpilogueArgs& e, int out_type, void* out, void* stream, const char* who) {
  ITEXHIP_REQUIRE(K % 16 == 0, "%s: K must be a multiple of 16 (got %lld); use itexhip_qgemm_naive", who,
                  static_cast<long long>(K));
  ITEXHIP_REQUIRE(aligned(a, 16) && aligned(packed_b, 16), "%s: operands must be 16-byte aligned", who);
  ITEXHIP_REQUIRE(a_type != ITEXHIP_QUINT8 || e.colsum, "%s: quint8 activations need colsum", who);
  ITEXHIP_REQUIRE(!gemv || M <= kSmallMaxRows, "%s: M must be <= %d", who, kSmallMaxRows);
  ITEXHIP_REQUIRE(M * K < (1LL << 31), "%s: activation matrix too large (M * K must be < 2^31)", who);
  const uint32_t a_xor = (a_type == ITEXHIP_QUINT8) ? 0x80808080u : 0u;
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

int packed_path(bool gemv, const void* a, int a_type, const int8_t* packed_b, const int32_t* colsum,
                int64_t M, int64_t K, int64_t N, const float* scales, const float* bias,
                const itexhip_epilogue* ep, int out_type, void* out, void* stream, const char* who,
                const void* addend = nullptr, int addend_type = 0) {
  if (int st = check_common(a, a_type, packed_b, M, K, N, scales, ep, out_type, out, who, addend, addend_type)) return st;
  if (M == 0 || N == 0) return ITEXHIP_OK;
  return launch_packed(gemv, a, a_type, packed_b, M, K, N, make_args(a_type, colsum, scales, bias, ep, addend, addend_type),
                       out_type, out, stream, who);
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
  return packed_path(small_m(M, K, N), a, a_type, packed_b, colsum, M, K, N, scales, bias, ep, out_type, out, stream,
                     "itexhip_qgemm");
}

extern "C" int itexhip_qgemm_sum(const void* a, int a_type, const int8_t* packed_b, const int32_t* colsum,
                                 int64_t M, int64_t K, int64_t N, const float* scales, const float* bias,
                                 const itexhip_epilogue* ep, const void* addend, int addend_type, int out_type, void* out,
                                 void* stream) {
  ITEXHIP_REQUIRE(addend != nullptr || M == 0 || N == 0, "itexhip_qgemm_sum: null addend");
  return packed_path(small_m(M, K, N), a, a_type, packed_b, colsum, M, K, N, scales, bias, ep, out_type, out, stream,
                     "itexhip_qgemm_sum", addend, addend_type);
}

// ------------------------------------------------------------------------------------------------
// Conv2D as an implicit GEMM
// ------------------------------------------------------------------------------------------------
namespace {
bool conv_implicit_ok(const itexhip_conv_geometry* g, const void* x, int64_t out_channels, int out_type, const void* out) {
  const int esz = (out_type == ITEXHIP_QINT8 || out_type == ITEXHIP_QUINT8) ? 1 : out_type == ITEXHIP_BFLOAT16 ? 2 : 4;
  if (out_type == ITEXHIP_HALF || out_channels <= 0 || out_channels >= (1LL << 31) || (out_channels * esz) % 16 != 0 || !aligned(out, 16))
    return false;
  if (!g || g->batch <= 0 || g->in_h <= 0 || g->in_w <= 0 || g->in_c <= 0 || g->k_h <= 0 || g->k_w <= 0 ||
      g->out_h <= 0 || g->out_w <= 0 || g->stride_h <= 0 || g->stride_w <= 0 || g->dil_h <= 0 || g->dil_w <= 0)
    return false;
  const int64_t K = g->k_h * g->k_w * g->in_c;
  const int64_t lim = 1LL << 31;
  // A 16-byte piece of a patch row must be 16 contiguous input bytes that exist (or lie in the padding) as a whole.
  // With in_c a multiple of 16 a piece is part of one pixel.  With 4 or 8 channels it is a run of 4 or 2 pixels of one
  // window row: contiguous without dilation along the row, whole runs when the window row is a multiple of 16 bytes, and
  // never cut by the edge of the input when no window needs padding (the caller pads the input itself: itexhip_pad_nhwc8).
  const bool pixel_pieces = g->in_c % 16 == 0;
  const bool run_pieces = (g->in_c == 4 || g->in_c == 8) && (g->k_w * g->in_c) % 16 == 0 && g->dil_w == 1 &&
                          g->pad_top == 0 && g->pad_left == 0 &&
                          (g->out_h - 1) * g->stride_h + (g->k_h - 1) * g->dil_h + 1 <= g->in_h &&
                          (g->out_w - 1) * g->stride_w + g->k_w <= g->in_w;
  return (pixel_pieces || run_pieces) && K / 16 <= kMaxConvPieces && aligned(x, 16) && g->batch * g->in_h * g->in_w * g->in_c < lim &&
         g->batch * g->out_h * g->out_w < lim && (g->k_h - 1) * g->dil_h < (1 << 15) && (g->k_w - 1) * g->dil_w < (1 << 15) &&
         g->pad_top >= 0 && g->pad_left >= 0 && g->pad_top < (1 << 24) && g->pad_left < (1 << 24) &&
         g->out_h * g->stride_h < (1LL << 30) && g->out_w * g->stride_w < (1LL << 30);
}
}  // namespace

extern "C" int itexhip_qconv2d_implicit_ok(const itexhip_conv_geometry* g, const void* x, int64_t out_channels, int out_type,
                                           const void* out) {
  return conv_implicit_ok(g, x, out_channels, out_type, out) ? 1 : 0;
}

namespace {
int qconv2d_impl(const char* who, const void* x, int x_type, const itexhip_conv_geometry* g, const int8_t* packed_filter,
                 const int32_t* colsum, int64_t out_channels, const float* scales, const float* bias,
                 const itexhip_epilogue* ep, const void* addend, int addend_type, int out_type, void* out, void* stream) {
  ITEXHIP_REQUIRE(g != nullptr, "%s: null geometry", who);
  ITEXHIP_REQUIRE(conv_implicit_ok(g, x, out_channels, out_type, out),
                  "%s: not a shape for the implicit GEMM (in_c %% 16 == 0, or 4 / 8 channels with unpadded windows whose rows are "
                  "a multiple of 16 bytes; window <= 16 KiB, 16-byte aligned input below 2 GiB, 16-byte aligned output rows); "
                  "use itexhip_im2col8 + itexhip_qgemm", who);
  ITEXHIP_REQUIRE(bias != nullptr, "%s: needs a bias vector (zeros when the op has none)", who);
  const int64_t M = g->batch * g->out_h * g->out_w, K = g->k_h * g->k_w * g->in_c, N = out_channels;
  if (int st = check_common(x, x_type, packed_filter, M, K, N, scales, ep, out_type, out, who, addend, addend_type)) return st;
  if (N == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(aligned(packed_filter, 16), "%s: the packed filter must be 16-byte aligned", who);
  ITEXHIP_REQUIRE(x_type != ITEXHIP_QUINT8 || colsum, "%s: quint8 input needs colsum", who);
  const EpilogueArgs e = make_args(x_type, colsum, scales, bias, ep, addend, addend_type);
  ConvTileArgs cv;
  cv.in_h = static_cast<int>(g->in_h); cv.in_w = static_cast<int>(g->in_w); cv.in_c = static_cast<int>(g->in_c);
  cv.k_w = static_cast<int>(g->k_w); cv.out_h = static_cast<int>(g->out_h); cv.out_w = static_cast<int>(g->out_w);
  cv.stride_h = g->stride_h; cv.stride_w = g->stride_w; cv.dil_h = g->dil_h; cv.dil_w = g->dil_w;
  cv.pad_top = static_cast<int>(g->pad_top); cv.pad_left = static_cast<int>(g->pad_left);
  cv.by_out_w = make_fast_div(g->out_w); cv.by_out_h = make_fast_div(g->out_h);
  cv.by_in_c = make_fast_div(g->in_c); cv.by_k_w = make_fast_div(g->k_w);
  const uint32_t a_xor = (x_type == ITEXHIP_QUINT8) ? 0x80808080u : 0u;
  const uint8_t* xp = reinterpret_cast<const uint8_t*>(x);
  const uint8_t* bp = reinterpret_cast<const uint8_t*>(packed_filter);
  hipStream_t hs = as_stream(stream);
  const int Mi = static_cast<int>(M), Ki = static_cast<int>(K), Ni = static_cast<int>(N);
  int st__ = ITEXHIP_OK;
  switch (out_type) {
    case ITEXHIP_FLOAT: st__ = dispatch_tile_conv<ITEXHIP_FLOAT>(xp, a_xor, bp, Mi, Ki, Ni, e, out, hs, cv); break;
    case ITEXHIP_BFLOAT16: st__ = dispatch_tile_conv<ITEXHIP_BFLOAT16>(xp, a_xor, bp, Mi, Ki, Ni, e, out, hs, cv); break;
    case ITEXHIP_QINT32: st__ = dispatch_tile_conv<ITEXHIP_QINT32>(xp, a_xor, bp, Mi, Ki, Ni, e, out, hs, cv); break;
    case ITEXHIP_QINT8: st__ = dispatch_tile_conv<ITEXHIP_QINT8>(xp, a_xor, bp, Mi, Ki, Ni, e, out, hs, cv); break;
    default: st__ = dispatch_tile_conv<ITEXHIP_QUINT8>(xp, a_xor, bp, Mi, Ki, Ni, e, out, hs, cv); break;
  }
  if (st__ != ITEXHIP_OK) return st__;
  ITEXHIP_CHECK_LAUNCH(who);
  return ITEXHIP_OK;
}
}  // namespace

extern "C" int itexhip_qconv2d(const void* x, int x_type, const itexhip_conv_geometry* g, const int8_t* packed_filter,
                               const int32_t* colsum, int64_t out_channels, const float* scales, const float* bias,
                               const itexhip_epilogue* ep, int out_type, void* out, void* stream) {
  return qconv2d_impl("itexhip_qconv2d", x, x_type, g, packed_filter, colsum, out_channels, scales, bias, ep, nullptr, 0,
                      out_type, out, stream);
}

extern "C" int itexhip_qconv2d_sum(const void* x, int x_type, const itexhip_conv_geometry* g, const int8_t* packed_filter,
                                   const int32_t* colsum, int64_t out_channels, const float* scales, const float* bias,
                                   const itexhip_epilogue* ep, const void* addend, int addend_type, int out_type, void* out,
                                   void* stream) {
  ITEXHIP_REQUIRE(addend != nullptr, "itexhip_qconv2d_sum: null addend");
  return qconv2d_impl("itexhip_qconv2d_sum", x, x_type, g, packed_filter, colsum, out_channels, scales, bias, ep, addend,
                      addend_type, out_type, out, stream);
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
    case ITEXHIP_BFLOAT16:
      qgemm_naive_kernel<ITEXHIP_BFLOAT16><<<grid, 256, 0, hs>>>(ap, a_is_u8, w, transpose_b, Mi, Ki, Ni, e, out);
      break;
    case ITEXHIP_HALF:
      qgemm_naive_kernel<ITEXHIP_HALF><<<grid, 256, 0, hs>>>(ap, a_is_u8, w, transpose_b, Mi, Ki, Ni, e, out);
      break;
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

namespace {
int qmatmul_impl(const char* who, const itexhip_matmul_params* p, const void* a, const int8_t* packed_b,
                 const int32_t* colsum, int64_t M, int64_t K, int64_t N, const float* row_min_a,
                 const float* row_max_a, const float* min_b, const float* max_b, int64_t nb, const void* bias,
                 const void* addend, void* out, void* stream, const float* range_a = nullptr) {
  itexhip_epilogue ep;
  if (int st = itexhip_qmatmul_epilogue_desc(p, nb, &ep)) return st;
  ITEXHIP_REQUIRE(nb == 1 || nb == N, "%s: %lld weight ranges for %lld channels", who, static_cast<long long>(nb),
                  static_cast<long long>(N));
  ITEXHIP_REQUIRE(M >= 0 && K >= 0 && N >= 0, "%s: negative dimension", who);
  ITEXHIP_REQUIRE(M < (1LL << 31) && N < (1LL << 31) && K <= kMaxK, "%s: dimension too large (K <= %lld)", who,
                  static_cast<long long>(kMaxK));
  if (M == 0 || N == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(out != nullptr && min_b != nullptr && max_b != nullptr, "%s: null buffer", who);
  ITEXHIP_REQUIRE(K == 0 || (a && packed_b), "%s: null operand", who);
  ITEXHIP_REQUIRE(colsum != nullptr, "%s: null colsum", who);
  ITEXHIP_REQUIRE((p->add_position != 0) == (addend != nullptr), "%s: the addend goes with \"Add\" in fused_ops", who);
  EpilogueArgs e = make_args(p->t_in, colsum, nullptr, bias, &ep);
  e.fused = 1;
  e.nb = static_cast<int>(nb);
  e.min_b = min_b;
  e.max_b = max_b;
  e.prep = make_prep_args(p, ep);
  e.row_min_a = row_min_a;
  e.row_max_a = row_max_a;
  e.range_a = range_a;
  e.addend = addend;
  e.addend_type = is_float16_type(p->t_out) ? p->t_out : ITEXHIP_FLOAT;  // the addend has the output's type
  return launch_packed(small_m(M, K, N), a, p->t_in, packed_b, M, K, N, e, p->t_out, out, stream, who);
}
}  // namespace

extern "C" int itexhip_qmatmul(const itexhip_matmul_params* p, const void* a, const int8_t* packed_b,
                               const int32_t* colsum, int64_t M, int64_t K, int64_t N, const float* min_b,
                               const float* max_b, int64_t nb, const void* bias, const void* addend, void* out,
                               void* stream) {
  return qmatmul_impl("itexhip_qmatmul", p, a, packed_b, colsum, M, K, N, nullptr, nullptr, min_b, max_b, nb, bias,
                      addend, out, stream);
}

extern "C" int itexhip_qmatmul_device_range(const itexhip_matmul_params* p, const void* a, const int8_t* packed_b,
                                           const int32_t* colsum, int64_t M, int64_t K, int64_t N, const float* range_a,
                                           const float* min_b, const float* max_b, int64_t nb, const void* bias,
                                           const void* addend, void* out, void* stream) {
  ITEXHIP_REQUIRE(range_a != nullptr, "itexhip_qmatmul_device_range: null activation range");
  ITEXHIP_REQUIRE(p->t_out != ITEXHIP_QINT32, "itexhip_qmatmul_device_range: a qint32 result's range is computed on the "
                                              "host from the activation range; use itexhip_qmatmul");
  return qmatmul_impl("itexhip_qmatmul_device_range", p, a, packed_b, colsum, M, K, N, nullptr, nullptr, min_b, max_b, nb,
                      bias, addend, out, stream, range_a);
}

extern "C" int itexhip_qmatmul_per_row(const itexhip_matmul_params* p, const void* a, const int8_t* packed_b,
                                       const int32_t* colsum, int64_t M, int64_t K, int64_t N,
                                       const float* row_min_a, const float* row_max_a, const float* min_b,
                                       const float* max_b, int64_t nb, const void* bias, const void* addend,
                                       void* out, void* stream) {
  ITEXHIP_REQUIRE(M <= 16, "itexhip_qmatmul_per_row: per-row activation ranges are implemented for M <= 16 (got %lld)",
                  static_cast<long long>(M));
  ITEXHIP_REQUIRE(M == 0 || (row_min_a && row_max_a), "itexhip_qmatmul_per_row: null row ranges");
  return qmatmul_impl("itexhip_qmatmul_per_row", p, a, packed_b, colsum, M, K, N, row_min_a, row_max_a, min_b, max_b, nb,
                      bias, addend, out, stream);
}

extern "C" int itexhip_mfma_probe(int workgroups, int iters, const void* operands, int32_t* sink, void* stream) {
  ITEXHIP_REQUIRE(workgroups > 0 && workgroups <= 65536 && iters > 0 && iters <= (1 << 22) && iters % 2 == 0,
                  "itexhip_mfma_probe: bad launch size (iters must be even)");
  ITEXHIP_REQUIRE(operands && sink && aligned(operands, 16), "itexhip_mfma_probe: null or unaligned buffer");
  mfma_probe_kernel<<<workgroups, 256, 0, as_stream(stream)>>>(iters, reinterpret_cast<const v4i*>(operands), sink);
  ITEXHIP_CHECK_LAUNCH("itexhip_mfma_probe");
  return ITEXHIP_OK;
}

extern "C" int itexhip_qmatmul_unpacked(const itexhip_matmul_params* p, const void* a, const int8_t* w, int transpose_b,
                                        int64_t M, int64_t K, int64_t N, const float* min_b, const float* max_b,
                                        int64_t nb, const void* bias, const void* addend, void* out, void* stream) {
  const char* who = "itexhip_qmatmul_unpacked";
  itexhip_epilogue ep;
  if (int st = itexhip_qmatmul_epilogue_desc(p, nb, &ep)) return st;
  ITEXHIP_REQUIRE(nb == 1 || nb == N, "%s: %lld weight ranges for %lld channels", who, static_cast<long long>(nb),
                  static_cast<long long>(N));
  ITEXHIP_REQUIRE(M >= 0 && K >= 0 && N >= 0 && M < (1LL << 31) && N < (1LL << 31) && K <= kMaxK, "%s: bad dimensions", who);
  // the reference's compensation indexes the weight as [K, N] whatever transpose_b says; that combination is refused
  ITEXHIP_REQUIRE(!(transpose_b && p->input_mode == ITEXHIP_MIN_FIRST), "%s: transpose_b with MIN_FIRST input is not supported", who);
  if (M == 0 || N == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(out != nullptr && min_b != nullptr && max_b != nullptr, "%s: null buffer", who);
  ITEXHIP_REQUIRE(K == 0 || (a && w), "%s: null operand", who);
  ITEXHIP_REQUIRE((p->add_position != 0) == (addend != nullptr), "%s: the addend goes with \"Add\" in fused_ops", who);
  EpilogueArgs e = make_args(p->t_in, nullptr, nullptr, bias, &ep);
  e.comp_mul = 0;  // unsigned activations are multiplied directly
  e.fused = 1;
  e.nb = static_cast<int>(nb);
  e.min_b = min_b;
  e.max_b = max_b;
  e.prep = make_prep_args(p, ep);
  e.addend = addend;
  e.addend_type = is_float16_type(p->t_out) ? p->t_out : ITEXHIP_FLOAT;  // the addend has the output's type
  const int a_is_u8 = p->t_in == ITEXHIP_QUINT8;
  const uint8_t* ap = reinterpret_cast<const uint8_t*>(a);
  const unsigned grid = static_cast<unsigned>((M * N + 255) / 256);
  hipStream_t hs = as_stream(stream);
  const int Mi = static_cast<int>(M), Ki = static_cast<int>(K), Ni = static_cast<int>(N);
  switch (p->t_out) {
    case ITEXHIP_FLOAT: qmatmul_unpacked_kernel<ITEXHIP_FLOAT><<<grid, 256, 0, hs>>>(ap, a_is_u8, w, transpose_b, Mi, Ki, Ni, e, out); break;
    case ITEXHIP_BFLOAT16: qmatmul_unpacked_kernel<ITEXHIP_BFLOAT16><<<grid, 256, 0, hs>>>(ap, a_is_u8, w, transpose_b, Mi, Ki, Ni, e, out); break;
    case ITEXHIP_HALF: qmatmul_unpacked_kernel<ITEXHIP_HALF><<<grid, 256, 0, hs>>>(ap, a_is_u8, w, transpose_b, Mi, Ki, Ni, e, out); break;
    case ITEXHIP_QINT32: qmatmul_unpacked_kernel<ITEXHIP_QINT32><<<grid, 256, 0, hs>>>(ap, a_is_u8, w, transpose_b, Mi, Ki, Ni, e, out); break;
    case ITEXHIP_QINT8: qmatmul_unpacked_kernel<ITEXHIP_QINT8><<<grid, 256, 0, hs>>>(ap, a_is_u8, w, transpose_b, Mi, Ki, Ni, e, out); break;
    default: qmatmul_unpacked_kernel<ITEXHIP_QUINT8><<<grid, 256, 0, hs>>>(ap, a_is_u8, w, transpose_b, Mi, Ki, Ni, e, out); break;
  }
  ITEXHIP_CHECK_LAUNCH(who);
  return ITEXHIP_OK;
}
