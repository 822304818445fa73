// MFMA tile kernel of the quantized MatMul (see qgemm.hip for the operand format).  Included by the
// per-output-type translation units qgemm_tile_*.hip, each of which instantiates dispatch_tile<T>.
#ifndef ITEXHIP_QGEMM_TILE_HPP_
#define ITEXHIP_QGEMM_TILE_HPP_

#include "qgemm_common.hpp"

namespace itexhip {

// ------------------------------------------------------------------------------------------------
// Tile kernel (compute bound, M > 16).
//   Block tile BM (activation rows) x BN (output channels), K step 64 (two chunks deep),
//   WAVES_M x WAVES_N wavefronts, each owning a (BM/WAVES_M) x (BN/WAVES_N) sub-tile of accumulators
//   (TM x TN tiles of 32x32, 16 registers each, kept in AGPRs).
//
//   Software pipeline over K steps, one barrier per step, ring of 3 LDS stages:
//     step k computes from stage k%3; it reads the fragments of step k+1 from stage (k+1)%3 (published
//     by the previous barrier), writes the chunks of step k+2 (loaded from global memory during step
//     k-1) into stage (k+2)%3 and issues the global loads of step k+3.
//   Inside a step the work is cut into 2*TN slices (k-chunk kc, channel tile j) of TM MFMAs: the weight
//   fragment of the next slice is read while the MFMAs of the current one run, so only two weight
//   fragments are live; the activation fragments of the next step are read one slice at a time into a
//   second register set; staging stores and global loads are spread over the slices the same way.
//
//   Activation staging.  One wavefront load covers 16 rows x 64 B (4 lanes per row: the texture
//   addresser serves a quad of lanes per cycle only when the quad is contiguous).  In LDS the piece
//   (row r, k-chunk kc, k-group g) lives in chunk kc of its 32-row tile at 16-byte slot
//   (g*32 + r) ^ (4*kc + 2*g); the XOR spreads the 8 lanes an LDS cycle serves over the 8 bank groups
//   for the staging stores and keeps the fragment reads (lane l reads slot l ^ (4*kc + 2*(l/32)))
//   conflict free.  Weight chunks are already in lane order in memory and are copied linearly.
//
//   Rows >= M and channel tiles >= NT are loaded from clamped (valid) addresses: whatever they
//   contribute lands in outputs that are never stored.  Columns k >= K multiply zero-padded weights.
// ------------------------------------------------------------------------------------------------
template <int BM, int BN, int WAVES_M, int WAVES_N, int OUT_T, int ACT>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void qgemm_tile_kernel(
    const uint8_t* __restrict__ a, uint32_t a_xor, const uint8_t* __restrict__ bp, int M, int K, int N,
    int KT, int NT, int num_m, int num_n, EpilogueArgs e, void* __restrict__ out) {
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int A_TILES = BM / 32, B_TILES = BN / 32;      // 32-row tiles per block
  constexpr int A_LOADS = A_TILES * 2, B_LOADS = B_TILES * 2;  // wavefront loads (1 KiB each) per step
  constexpr int A_PER_WAVE = A_LOADS / NW, B_PER_WAVE = B_LOADS / NW;
  constexpr int NSTG = A_PER_WAVE + B_PER_WAVE;
  constexpr int NSLICE = 2 * TN;
  static_assert(A_LOADS % NW == 0 && B_LOADS % NW == 0, "loads must divide among wavefronts");
  constexpr int STAGE_BYTES = (A_LOADS + B_LOADS) * kChunkBytes;
  constexpr int B_REGION = A_LOADS * kChunkBytes;

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
  const int lrow = lane & 31, lgrp = lane >> 5;

  v16i acc[TN * TM];
  static_for<TN * TM>([&](auto t) {
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0;
  });

  // ---- staging sources / destinations of this wavefront
  // activation load c covers rows [16*h, 16*h+16) of 32-row tile rt, both k-chunks: lane -> (row, piece)
  const int q_row = lane >> 2, q_piece = lane & 3;  // piece = kc*2 + g
  uint32_t off_a[A_PER_WAVE];   // byte offset of (row, piece 0.., k = 0) in the activation matrix
  uint32_t dst_a[A_PER_WAVE];   // byte offset inside a stage
  const uint8_t* src_b[B_PER_WAVE];
  uint32_t dst_b[B_PER_WAVE];
  static_for<A_PER_WAVE>([&](auto c) {
    const int ld = wave * A_PER_WAVE + c;  // 0 .. A_LOADS-1
    const int rt = ld >> 1, h = ld & 1;
    const int r = h * 16 + q_row;
    const int m = min(m_base + rt * 32 + r, M - 1);
    off_a[c] = static_cast<uint32_t>(m) * static_cast<uint32_t>(K);  // M * K < 2^31 checked by the host
    const int kc = q_piece >> 1, g = q_piece & 1;
    dst_a[c] = static_cast<uint32_t>((rt * 2 + kc) * kChunkBytes + (((g * 32 + r) ^ (4 * kc + 2 * g)) << 4));
  });
  static_for<B_PER_WAVE>([&](auto c) {
    const int ld = wave * B_PER_WAVE + c;  // 0 .. B_LOADS-1: (channel tile, k-chunk)
    const int nt = min((n_base >> 5) + (ld >> 1), NT - 1);
    src_b[c] = bp + (static_cast<int64_t>(nt) * (2 * KT) + (ld & 1)) * kChunkBytes + lane * 16;
    dst_b[c] = static_cast<uint32_t>(B_REGION + ld * kChunkBytes + lane * 16);
  });

  v4i stg[NSTG];
  auto load_chunk = [&](auto c, int kt) {
    constexpr int ci = decltype(c)::value;
    if constexpr (ci < A_PER_WAVE) {
      const uint32_t kofs = static_cast<uint32_t>(min(kt * 64 + q_piece * 16, K - 16));
      stg[ci] = *reinterpret_cast<const v4i*>(a + off_a[ci] + kofs);
    } else {
      stg[ci] = *reinterpret_cast<const v4i*>(src_b[ci - A_PER_WAVE] + static_cast<int64_t>(kt) * (2 * kChunkBytes));
    }
  };
  auto store_chunk = [&](auto c, int stage) {
    constexpr int ci = decltype(c)::value;
    uint8_t* base = lds + stage * STAGE_BYTES;
    if constexpr (ci < A_PER_WAVE) {
      v4i v = stg[ci];
      v.x ^= a_xor; v.y ^= a_xor; v.z ^= a_xor; v.w ^= a_xor;
      *reinterpret_cast<v4i*>(base + dst_a[ci]) = v;
    } else {
      *reinterpret_cast<v4i*>(base + dst_b[ci - A_PER_WAVE]) = stg[ci];
    }
  };
  // fragment reads: activation fragment (k-chunk kc, row tile i of this wavefront), weight fragment (kc, j)
  const uint32_t frag_a_lane[2] = {static_cast<uint32_t>((lane ^ (2 * lgrp)) << 4),
                                   static_cast<uint32_t>((lane ^ (4 + 2 * lgrp)) << 4)};
  auto lds_a = [&](int stage, int kc, int i) {
    return *reinterpret_cast<const v4i*>(lds + stage * STAGE_BYTES + ((wm * TM + i) * 2 + kc) * kChunkBytes + frag_a_lane[kc]);
  };
  auto lds_b = [&](int stage, int kc, int j) {
    return *reinterpret_cast<const v4i*>(lds + stage * STAGE_BYTES + B_REGION + ((wn * TN + j) * 2 + kc) * kChunkBytes + lane * 16);
  };

  // ---- prologue: stages 0 and 1 filled, chunks of step 2 in flight
  static_for<NSTG>([&](auto c) { load_chunk(c, 0); });
  static_for<NSTG>([&](auto c) { store_chunk(c, 0); });
  static_for<NSTG>([&](auto c) { load_chunk(c, min(1, KT - 1)); });
  static_for<NSTG>([&](auto c) { store_chunk(c, 1); });
  static_for<NSTG>([&](auto c) { load_chunk(c, min(2, KT - 1)); });
  __syncthreads();

  v4i fa_cur[2 * TM], fa_nxt[2 * TM], fb[2], fb_first;
  static_for<2 * TM>([&](auto x) { fa_cur[x] = lds_a(0, decltype(x)::value / TM, decltype(x)::value % TM); });
  fb[0] = lds_b(0, 0, 0);

  // K loop, branch free: past the end of K the prefetches read stale stages / clamped addresses and
  // the staging stores go to a stage nobody reads any more.  All LDS reads of a step are issued in
  // slices 0 .. NSLICE-2, so the MFMAs of the last slice cover their latency before the barrier.
  int st_cur = 0, st_nxt = 1, st_fill = 2;
  for (int kt = 0; kt < KT; ++kt) {
    const int kt_load = min(kt + 3, KT - 1);
    static_for<NSLICE>([&](auto sl) {
      constexpr int s = decltype(sl)::value;
      constexpr int kc = s / TN, j = s % TN;
      // staging traffic of this slice
      static_for<NSTG>([&](auto c) {
        if constexpr (decltype(c)::value * NSLICE / NSTG == s) {
          store_chunk(c, st_fill);
          load_chunk(c, kt_load);
        }
      });
      // fragment prefetch of this slice
      if constexpr (s + 1 < NSLICE) fb[(s + 1) & 1] = lds_b(st_cur, (s + 1) / TN, (s + 1) % TN);
      if constexpr (s == NSLICE - 2) fb_first = lds_b(st_nxt, 0, 0);
      static_for<2 * TM>([&](auto x) {
        if constexpr (decltype(x)::value * (NSLICE - 1) / (2 * TM) == s)
          fa_nxt[x] = lds_a(st_nxt, decltype(x)::value / TM, decltype(x)::value % TM);
      });
      static_for<TM>([&](auto i) {
        constexpr int t = j * TM + decltype(i)::value;
        acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[s & 1], fa_cur[kc * TM + decltype(i)::value], acc[t], 0, 0, 0);
      });
      __builtin_amdgcn_sched_barrier(0);
    });
    static_for<2 * TM>([&](auto x) { fa_cur[x] = fa_nxt[x]; });
    fb[0] = fb_first;
    __syncthreads();
    const int t = st_cur;
    st_cur = st_nxt;
    st_nxt = st_fill;
    st_fill = t;
  }

  // ---- epilogue straight from the accumulator registers
  const bool vec_ok = (N & 3) == 0 && aligned16(e.scales) && aligned16(e.bias) && aligned16(e.colsum) && aligned16(out);
  static_for<TN>([&](auto j) {
    static_for<4>([&](auto g) {
      const int n = n_base + (wn * TN + j) * 32 + decltype(g)::value * 8 + lgrp * 4;
      if (n < N) {
        const ChannelParams p = load_channel_params(e, n, N, vec_ok);
        static_for<TM>([&](auto i) {
          constexpr int t = decltype(j)::value * TM + decltype(i)::value;
          constexpr int r0 = decltype(g)::value * 4;
          const int m = m_base + (wm * TM + i) * 32 + lrow;
          const v4i part = v4i{acc[t][r0], acc[t][r0 + 1], acc[t][r0 + 2], acc[t][r0 + 3]};
          epilogue_store<OUT_T, ACT>(part, p, m, n, M, N, e, out, vec_ok);
        });
      }
    });
  });
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int OUT_T, int ACT>
int launch_tile(const uint8_t* a, uint32_t a_xor, const uint8_t* bp, int M, int K, int N,
                const EpilogueArgs& e, void* out, hipStream_t st) {
  const int KT = (K + 63) / 64, NT = (N + kChunkRows - 1) / kChunkRows;
  const int num_m = (M + BM - 1) / BM, num_n = (N + BN - 1) / BN;
  constexpr size_t lds_bytes = 3 * (BM / 16 + BN / 16) * kChunkBytes;
  auto kern = qgemm_tile_kernel<BM, BN, WAVES_M, WAVES_N, OUT_T, ACT>;
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

template <int OUT_T, int ACT>
int dispatch_tile_shape(const uint8_t* a, uint32_t a_xor, const uint8_t* bp, int M, int K, int N,
                        const EpilogueArgs& e, void* out, hipStream_t st) {
  // pick the largest tile that still gives every CU work
  const int64_t tiles_256 = static_cast<int64_t>((M + 255) / 256) * ((N + 255) / 256);
  const int64_t tiles_128 = static_cast<int64_t>((M + 127) / 128) * ((N + 127) / 128);
  if (tiles_256 >= 256) return launch_tile<256, 256, 2, 2, OUT_T, ACT>(a, a_xor, bp, M, K, N, e, out, st);
  if (tiles_128 >= 256) return launch_tile<128, 128, 2, 2, OUT_T, ACT>(a, a_xor, bp, M, K, N, e, out, st);
  return launch_tile<64, 64, 2, 2, OUT_T, ACT>(a, a_xor, bp, M, K, N, e, out, st);
}

template <int OUT_T>
int dispatch_tile(const uint8_t* a, uint32_t a_xor, const uint8_t* bp, int M, int K, int N,
                  const EpilogueArgs& e, void* out, hipStream_t st) {
  if (e.n_eltwise == 0) return dispatch_tile_shape<OUT_T, 0>(a, a_xor, bp, M, K, N, e, out, st);
  if (e.n_eltwise == 1 && e.elt[0].alg == ITEXHIP_ELT_RELU && e.elt[0].alpha == 0.0f)
    return dispatch_tile_shape<OUT_T, 1>(a, a_xor, bp, M, K, N, e, out, st);
  return dispatch_tile_shape<OUT_T, 2>(a, a_xor, bp, M, K, N, e, out, st);
}

}  // namespace itexhip
#endif  // ITEXHIP_QGEMM_TILE_HPP_
