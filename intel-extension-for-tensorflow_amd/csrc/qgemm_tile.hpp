// MFMA tile kernel of the quantized MatMul (see qgemm.hip for the operand format).  Included by the
// per-output-type translation units qgemm_tile_*.hip, each of which instantiates dispatch_tile<T>.
#ifndef ITEXHIP_QGEMM_TILE_HPP_
#define ITEXHIP_QGEMM_TILE_HPP_

#include <algorithm>
#include <cmath>
#include <cstdlib>

#include "qgemm_common.hpp"

// Measurement builds only (ablate.py): a bit mask of parts of the kernel that are compiled out, so that time, power
// and energy of a launch can be attributed to them.  Such a build computes wrong results; the library is built with 0.
//   1: no activation-fragment reads from LDS      2: no weight-fragment reads from LDS
//   4: no operand loads inside the K loop (global -> LDS)      8: no MFMAs
//  16: no epilogue (conversion, transposition, stores)        32: no sign flips of the activation fragments
#ifndef ITEXHIP_ABLATE
#define ITEXHIP_ABLATE 0
#endif

namespace itexhip {

// ------------------------------------------------------------------------------------------------
// Tile kernel (compute bound, M > 16).
//   Block tile BM (activation rows) x BN (output channels), K step 64 (two 32-deep MFMA chunks),
//   WAVES_M x WAVES_N wavefronts, each owning a (BM/WAVES_M) x (BN/WAVES_N) sub-tile of accumulators
//   (TM x TN tiles of 32x32, 16 registers each, kept in AGPRs).
//
//   Operands reach LDS by direct global->LDS loads (global_load_lds_dwordx4: each lane's 16 bytes land
//   at LDS base + 16 * lane, no VGPRs and no ds_write on the way).  LDS is the busiest unit of this
//   kernel (128 B/clk shared by fragment reads and staging), so staging must not cost store slots.
//
//   Software pipeline over K steps, one barrier per step, ring of 4 LDS stages:
//     step k computes from stage k%4 and reads the fragments of step k+1 from stage (k+1)%4; the loads
//     of step k+3 are issued into stage (k+3)%4; before the barrier that ends step k each wavefront
//     waits for its loads of step k+2 (issued during step k-1, a full step earlier).
//   Inside a step the work is cut into 2*TN slices (k-chunk kc, channel tile j) of TM MFMAs: the weight
//   fragment of the next slice is read while the MFMAs of the current one run, so only two weight
//   fragments are live; the activation fragments of the next step are read one slice at a time into a
//   second register set; the loads are spread over the slices the same way.
//
//   Activation staging.  One wavefront load covers 16 rows x 64 B, 4 consecutive lanes per row (the
//   texture addresser serves a quad of lanes per cycle only when the quad is contiguous).  Quad q of a
//   load holds row q; inside the quad, piece p (= 2*kc + g, 16 bytes of k) sits at lane
//   p ^ ((q >> 2) & 3).  That rotation makes the fragment reads conflict free: the 16 lanes an LDS cycle
//   serves (256 B per cycle on this device) read 16 consecutive rows, whose 16-byte slots then fall into 16
//   different bank groups (slot 4 q + (p ^ (q >> 2)): q & 3 picks a group of four, the rotation one of them).
//   Rotating by (q >> 1), which spreads 8 lanes over 8 bank groups, left a two-way conflict on every
//   activation fragment read (SQ_LDS_BANK_CONFLICT: a third of the K loop's LDS cycles).
//   Weight chunks are already in fragment lane order in memory and are copied linearly.
//   Unsigned activations are turned into signed ones (x ^ 0x80) after the fragment read.
//
//   Rows >= M and channel tiles >= NT are loaded from clamped (valid) addresses: whatever they
//   contribute lands in outputs that are never stored.  Columns k >= K multiply zero-padded weights.
// ------------------------------------------------------------------------------------------------
// How the tile grid is dealt to the 8 XCDs (each with an L2 of its own).  0: every XCD takes a contiguous range of
// tiles, m fastest.  When the grid fits the device in one round and such a range would pull more operand bytes
// through one L2 than it keeps (3 of its 4 MB), the grid is cut into gm x (8 / gm) rectangles of tiles instead, one
// per XCD, as square in bytes as the divisors of the grid allow; the result describes the rectangles (see below).  Below that size the contiguous
// range measured faster (BERT-base 768 -> 768 at 4096 tokens: 7.2 against 7.9 us), above it the rectangles
// (3072 -> 768: 15.4 against 18.7 us).
inline int xcd_rectangles(int num_m, int num_n, int BM, int BN, int K) {
  const int total = num_m * num_n, per_xcd = total >> 3;
  if (total > 256 || (total & 7) != 0) return 0;
  const int range_cost = std::min(num_m, per_xcd) * BM + (per_xcd + num_m - 1) / num_m * BN;
  if (static_cast<int64_t>(range_cost) * K <= 3 * 1024 * 1024) return 0;
  int gm = 0, best = range_cost;
  for (int g = 1; g <= 8; g *= 2) {
    const int gn = 8 / g;
    if (num_m % g != 0 || num_n % gn != 0) continue;
    const int cost = (num_m / g) * BM + (num_n / gn) * BN;
    if (cost < best) { best = cost; gm = g; }
  }
  if (gm == 0) return 0;
  // what the kernel needs, packed: log2(gm) + 1, the rectangle's extent in tiles (sm x sn, each <= 32 because the grid
  // has at most 256 tiles) and ceil(2^12 / sm) for its division by sm
  const int sm = num_m / gm, sn = num_n / (8 / gm);
  int lg = 0;
  while ((1 << lg) < gm) ++lg;
  return (lg + 1) | (sm << 3) | (sn << 9) | (((4096 + sm - 1) / sm) << 15);
}

// Implicit GEMM of a Conv2D (NHWC input): the activation "matrix" is the patch matrix
// [batch * out_h * out_w, k_h * k_w * in_c], never materialised.  With in_c a multiple of 16 a 16-byte piece of a patch
// row lies inside one input pixel (or in the padding, then it is read from 16 zero bytes); with 4 or 8 channels it is a
// run of 4 or 2 pixels of one window row, which the host admits only where no window touches the padding.  Either way
// only the source address of an activation load changes: row -> window origin once per kernel, piece -> offset inside
// the window from a table in LDS.
struct NoConvArgs {};
template <bool CONV> struct conv_args_of { using type = NoConvArgs; };
template <> struct conv_args_of<true> { using type = ConvTileArgs; };
static __device__ __align__(16) const uint32_t kZeroPiece[4] = {0u, 0u, 0u, 0u};

// amask: 0x80808080 when the activations are unsigned (they are fed as x ^ 0x80), else 0; a scalar
// register operand, so the sign flip costs a 4-byte instruction per dword.  KALIGNED: K is a multiple
// of 64, so activation loads never need a per-lane clamp and use a uniform base that advances by 64
// bytes per step.
template <int BM, int BN, int WAVES_M, int WAVES_N, int OUT_T, int ACT, bool KALIGNED, bool CONV = false, bool ELEMENTWISE = false>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void qgemm_tile_kernel(
    const uint8_t* __restrict__ a, uint32_t amask, const uint8_t* __restrict__ bp, int M, int K, int N,
    int KT, int NT, int num_m, int num_n, int xcd_gm, EpilogueArgs e, void* __restrict__ out,
    typename conv_args_of<CONV>::type cv) {
  static_assert(!CONV || !KALIGNED, "the implicit GEMM addresses every activation piece per lane");
  static_assert(!ELEMENTWISE || (ACT == 2 && !KALIGNED && !CONV), "the element-wise epilogue exists in the conservative form only");
  static_assert(ACT >= 0 && ACT <= 3, "0 none, 1 ReLU, 2 canonical chain (cheap activation), 3 canonical chain (GELU)");
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int A_TILES = BM / 32, B_TILES = BN / 32;          // 32-row tiles per block
  constexpr int A_LOADS = A_TILES * 2, B_LOADS = B_TILES * 2;  // wavefront loads (1 KiB each) per step
  constexpr int A_PER_WAVE = A_LOADS / NW, B_PER_WAVE = B_LOADS / NW;
  constexpr int NLD = A_PER_WAVE + B_PER_WAVE;                 // loads per wavefront per step
  constexpr int NSLICE = 2 * TN;
  constexpr int NSTAGE = 4;
  static_assert(A_LOADS % NW == 0 && B_LOADS % NW == 0, "loads must divide among wavefronts");
  static_assert(NLD < 32, "vmcnt budget");
  static_assert(NSLICE % 2 == 0, "slices come in two halves");
  constexpr int STAGE_BYTES = (A_LOADS + B_LOADS) * kChunkBytes;
  constexpr int B_REGION = A_LOADS * kChunkBytes;
  // behind the ring: the per-channel epilogue parameters of this block's BN channels
  constexpr int PANEL_OFF = NSTAGE * STAGE_BYTES;
  // the element-wise (any alignment, any N, optional bias, addend) epilogue is a kernel of its own; the host
  // sends the calls that need it there.  Compiled next to the vector epilogue it slowed that one down by a third.
  constexpr bool GENERAL = ELEMENTWISE;
  static_assert(BN <= 64 * NW, "one thread per channel fills the parameter panel");
  // behind the panel (implicit GEMM only): per 16-byte piece of a patch row, {window row << 16 | window column,
  // byte offset from the window origin}
  constexpr int CONV_TAB_OFF = PANEL_OFF + 12 * BN;

  extern __shared__ __align__(16) uint8_t lds[];
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) void*)lds));

  // ---- block -> tile mapping: consecutive workgroup ids go round-robin to the 8 XCDs.  By default every XCD
  // gets a contiguous range of tiles (m fastest), so that the tiles sharing a weight panel share an L2; with
  // xcd_gm != 0 (see xcd_rectangles) the tile grid is cut into xcd_gm x (8 / xcd_gm) rectangles, one per XCD.
  int pid = blockIdx.x;
  int tile_m, tile_n;
  if (xcd_gm != 0) {  // packed by xcd_rectangles: no division here, the first operand loads wait for this arithmetic
    const int lg = (xcd_gm & 7) - 1, sm = (xcd_gm >> 3) & 63, sn = (xcd_gm >> 9) & 63, inv = xcd_gm >> 15;
    const int xcd = pid & 7, local = pid >> 3;
    const int ln = (local * inv) >> 12;  // local / sm, exact for local, sm <= 32
    tile_m = (xcd & ((1 << lg) - 1)) * sm + (local - ln * sm);
    tile_n = (xcd >> lg) * sn + ln;
  } else {
    const int total = num_m * num_n;
    if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
    tile_m = pid % num_m;
    tile_n = pid / num_m;
  }
  const int m_base = tile_m * BM, n_base = tile_n * BN;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;
  const int lrow = lane & 31, lgrp = lane >> 5;

  v16i acc[TN * TM];
  int* const panel_comp = reinterpret_cast<int*>(lds + PANEL_OFF);
  float* const panel_scale = reinterpret_cast<float*>(lds + PANEL_OFF + BN * 4);
  float* const panel_bias = reinterpret_cast<float*>(lds + PANEL_OFF + BN * 8);

  // ---- staging sources of this wavefront
  // activation load `ld` covers rows [16*h, 16*h+16) of 32-row tile rt: lane -> (row q, piece p)
  const int q_row = lane >> 2;
  const int q_piece = (lane & 3) ^ ((q_row >> 2) & 3);  // piece = 2*kc + g
  uint32_t off_a[A_PER_WAVE];       // byte offset of the lane's row (+ piece when KALIGNED) in the activation matrix
  const uint8_t* src_b[B_PER_WAVE];  // wavefront-uniform chunk pointers of step 0
  int win_h[A_PER_WAVE], win_w[A_PER_WAVE];  // implicit GEMM: window origin of the lane's row (may lie in the padding)
  const int2* const conv_tab = reinterpret_cast<const int2*>(lds + CONV_TAB_OFF);
  static_for<A_PER_WAVE>([&](auto c) {
    const int ld = wave * A_PER_WAVE + c;  // 0 .. A_LOADS-1 = (rt, h)
    const int m = min(m_base + ld * 16 + q_row, M - 1);
    if constexpr (CONV) {
      const int t = fast_div(m, cv.by_out_w), ow = m - t * cv.out_w;
      const int b = fast_div(t, cv.by_out_h), oh = t - b * cv.out_h;
      win_h[c] = oh * cv.stride_h - cv.pad_top;
      win_w[c] = ow * cv.stride_w - cv.pad_left;
      // input bytes < 2^31 checked by the host; the origin may be negative, origin + an in-bounds piece is not
      off_a[c] = static_cast<uint32_t>(((b * cv.in_h + win_h[c]) * cv.in_w + win_w[c]) * cv.in_c);
    } else {
      off_a[c] = static_cast<uint32_t>(m) * static_cast<uint32_t>(K) +  // M * K < 2^31 checked by the host
                 (KALIGNED ? q_piece * 16 : 0);
    }
  });
  if constexpr (CONV) {
    for (int p = threadIdx.x; p < (K >> 4); p += 64 * NW) {
      const int k0 = p * 16;
      const int kk = fast_div(k0, cv.by_in_c), cc = k0 - kk * cv.in_c;
      const int kh = fast_div(kk, cv.by_k_w), kw = kk - kh * cv.k_w;
      const int dh = kh * cv.dil_h, dw = kw * cv.dil_w;  // < 2^15 each, checked by the host
      reinterpret_cast<int2*>(lds + CONV_TAB_OFF)[p] = make_int2((dh << 16) | dw, (dh * cv.in_w + dw) * cv.in_c + cc);
    }
    __syncthreads();
  }
  // the table entry of the lane's piece in K step kt (the same for all of the lane's loads of that step)
  auto conv_piece = [&](int kt) {
    if constexpr (CONV) return conv_tab[min(kt * 4 + q_piece, (K >> 4) - 1)];
    else return make_int2(0, 0);
  };
  static_for<B_PER_WAVE>([&](auto c) {
    const int ld = wave * B_PER_WAVE + c;  // 0 .. B_LOADS-1 = (channel tile, k-chunk)
    const int nt = min((n_base >> 5) + (ld >> 1), NT - 1);
    src_b[c] = bp + (static_cast<int64_t>(nt) * (2 * KT) + (ld & 1)) * kChunkBytes;
  });
  const uint32_t lane16 = lane * 16;
  auto issue_load = [&](auto c, int kt, int stage, int2 piece) {
    constexpr int ci = decltype(c)::value;
    const uint32_t stage_addr = lds_base + stage * STAGE_BYTES;
    if constexpr (ci < A_PER_WAVE) {
      if constexpr (CONV) {
        const int ih = win_h[ci] + (piece.x >> 16), iw = win_w[ci] + (piece.x & 0xffff);
        const bool inside = static_cast<unsigned>(ih) < static_cast<unsigned>(cv.in_h) &&
                            static_cast<unsigned>(iw) < static_cast<unsigned>(cv.in_w);
        const uint8_t* src = inside ? a + static_cast<int>(off_a[ci] + static_cast<uint32_t>(piece.y))
                                    : reinterpret_cast<const uint8_t*>(kZeroPiece);
        lds_dma16(src, stage_addr + (wave * A_PER_WAVE + ci) * kChunkBytes);
      } else if constexpr (KALIGNED) {
        lds_dma16(a + static_cast<int64_t>(kt) * 64, off_a[ci], stage_addr + (wave * A_PER_WAVE + ci) * kChunkBytes);
      } else {
        const uint32_t kofs = static_cast<uint32_t>(min(kt * 64 + q_piece * 16, K - 16));
        lds_dma16(a + off_a[ci] + kofs, stage_addr + (wave * A_PER_WAVE + ci) * kChunkBytes);
      }
    } else {
      lds_dma16(src_b[ci - A_PER_WAVE] + static_cast<int64_t>(kt) * (2 * kChunkBytes), lane16,
                stage_addr + B_REGION + (wave * B_PER_WAVE + (ci - A_PER_WAVE)) * kChunkBytes);
    }
  };
  // fragment reads: activation fragment (k-chunk kc, row tile i of this wavefront), weight fragment (kc, j)
  const int fq = lrow & 15, fh = lrow >> 4;
  const uint32_t frag_a_lane[2] = {
      static_cast<uint32_t>(fh * kChunkBytes + ((4 * fq + ((0 + lgrp) ^ ((fq >> 2) & 3))) << 4)),
      static_cast<uint32_t>(fh * kChunkBytes + ((4 * fq + ((2 + lgrp) ^ ((fq >> 2) & 3))) << 4))};
  auto lds_a_raw = [&](int stage, int kc, int i) {
    return *reinterpret_cast<const v4i*>(lds + stage * STAGE_BYTES + (wm * TM + i) * (2 * kChunkBytes) + frag_a_lane[kc]);
  };
  auto flip = [&](v4i v) {  // u8 -> s8 (x - 128) for unsigned activations, identity for signed ones
    v.x ^= amask; v.y ^= amask; v.z ^= amask; v.w ^= amask;
    return v;
  };
  auto lds_b = [&](int stage, int kc, int j) {
    return *reinterpret_cast<const v4i*>(lds + stage * STAGE_BYTES + B_REGION + ((wn * TN + j) * 2 + kc) * kChunkBytes + lane * 16);
  };

  // ---- prologue.  First the few loads of the channel parameters (thread t resolves channel n_base + t once, so the
  // epilogue is free of global loads and of branches on them), then the operand loads of steps 0, 1, 2.  Loads return
  // in the order issued: the parameters are there when only the operand loads are outstanding, and their arithmetic
  // runs while those travel.
  static_assert(kEarlyChannelLoads + 3 * NLD < 64, "vmcnt budget of the prologue");
  const bool panel_thread = threadIdx.x < BN;
  RawChannel raw;
  if (panel_thread) raw = load_raw_channel_early(e, min(n_base + static_cast<int>(threadIdx.x), N - 1), N);
  {
    const int2 p0 = conv_piece(0), p1 = conv_piece(min(1, KT - 1)), p2 = conv_piece(min(2, KT - 1));
    static_for<NLD>([&](auto c) { issue_load(c, 0, 0, p0); });
    static_for<NLD>([&](auto c) { issue_load(c, min(1, KT - 1), 1, p1); });
    static_for<NLD>([&](auto c) { issue_load(c, min(2, KT - 1), 2, p2); });
  }
  wait_vmcnt<3 * NLD>();
  if (panel_thread) {
    settle_raw_channel(raw);
    int comp;
    float scale, bias;
    finish_channel_early(e, raw, &comp, &scale, &bias);
    panel_comp[threadIdx.x] = comp;
    panel_scale[threadIdx.x] = scale;
    panel_bias[threadIdx.x] = bias;
  }
  wait_vmcnt<NLD>();
  __syncthreads();
  // the accumulators start from the zero-point compensation of their channel (exact in int32)
  static_for<TN>([&](auto j) {
    static_for<4>([&](auto g) {
      const v4i c = *reinterpret_cast<const v4i*>(panel_comp + (wn * TN + decltype(j)::value) * 32 + decltype(g)::value * 8 + lgrp * 4);
      static_for<TM>([&](auto i) {
        constexpr int t = decltype(j)::value * TM + decltype(i)::value;
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[t][decltype(g)::value * 4 + r] = c[r];
      });
    });
  });

  // weight fragments rotate through FBN registers sets and are read FBD slices ahead of their use
  constexpr int FBD = (NSLICE % 4 == 0) ? 2 : 1;
  constexpr int FBN = (NSLICE % 4 == 0) ? 4 : 2;
  static_assert(NSLICE % FBN == 0, "the weight fragment rotation must close over a step");
  v4i fa0[2 * TM], fa1[2 * TM], fb[FBN];
  static_for<2 * TM>([&](auto x) { fa0[x] = lds_a_raw(0, decltype(x)::value / TM, decltype(x)::value % TM); });
  static_for<2 * TM>([&](auto x) { fa0[x] = flip(fa0[x]); });
  static_for<FBD>([&](auto d) { fb[d] = lds_b(0, decltype(d)::value / TN, decltype(d)::value % TN); });

  // One K step, branch free: past the end of K the loads re-fetch the last step into stages nobody
  // reads and the prefetches read stale stages.
  //
  // A wavefront that runs alone on its SIMD only hides other instructions in the shadow of an MFMA
  // (32 cycles for 32x32x32) if they are issued between two MFMAs, so the step is laid out as
  // NSLICE * TM slots of "one MFMA + a little other work" and the compiler is kept from regrouping
  // them.  Per slice (k-chunk kc, channel tile j): slot 0 reads the weight fragment of the next
  // slice, the following slots read (first half of the step) or sign-flip (second half) the
  // activation fragments of the next step, the last slot issues one global->LDS load.
  // The two activation fragment sets swap roles from step to step (loop unrolled by two).
  constexpr int FA = 2 * TM;                       // activation fragments per step
  auto step = [&](int kt, const v4i (&fa_cur)[FA], v4i (&fa_nxt)[FA]) {
    const int st_cur = kt & 3, st_nxt = (kt + 1) & 3, st_fill = (kt + 3) & 3;
    const int kt_load = min(kt + 3, KT - 1);
    const int2 piece = conv_piece(kt_load);  // read at the top of the step, used by the load slots
    static_for<NSLICE>([&](auto sl) {
      constexpr int s = decltype(sl)::value;
      constexpr int kc = s / TN, j = s % TN;
      static_for<TM>([&](auto i) {
        constexpr int ii = decltype(i)::value;
        constexpr int t = j * TM + ii;
        if constexpr ((ITEXHIP_ABLATE & 8) == 0) acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[s % FBN], fa_cur[kc * TM + ii], acc[t], 0, 0, 0);
        else asm volatile("" : : "v"(fb[s % FBN]), "v"(fa_cur[kc * TM + ii]));  // the fragments stay live
        // ---- the slot behind this MFMA
        if constexpr (ii == 0) {
          constexpr int sn = s + FBD;  // the slice whose weight fragment is read now
          if constexpr ((ITEXHIP_ABLATE & 2) != 0) asm volatile("" : "+v"(fb[sn % FBN]));
          else if constexpr (sn < NSLICE) fb[sn % FBN] = lds_b(st_cur, sn / TN, sn % TN);
          else fb[sn % FBN] = lds_b(st_nxt, (sn - NSLICE) / TN, (sn - NSLICE) % TN);
        }
        if constexpr (ii == TM - 1) {
          static_for<NLD>([&](auto c) {
            if constexpr ((ITEXHIP_ABLATE & 4) == 0 && decltype(c)::value * NSLICE / NLD == s) issue_load(c, kt_load, st_fill, piece);
          });
        }
        // activation fragments of the next step: read during the first half of the slices, sign
        // flipped (dword by dword) during the second half, spread evenly over the MFMA slots
        {
          constexpr int HALF = NSLICE / 2, Q = HALF * TM;  // slots per half
          constexpr int q = (s % HALF) * TM + ii;          // this slot's index inside its half
          constexpr int shift = (Q >= 2 * FA) ? 1 : 0;     // keep clear of the weight-fragment slot when there is room
          if constexpr (s < HALF) {
            static_for<FA>([&](auto x) {
              if constexpr ((ITEXHIP_ABLATE & 1) == 0 && decltype(x)::value * Q / FA + shift == q)
                fa_nxt[decltype(x)::value] = lds_a_raw(st_nxt, decltype(x)::value / TM, decltype(x)::value % TM);
            });
          } else {
            static_for<4 * FA>([&](auto d) {
              if constexpr ((ITEXHIP_ABLATE & 32) == 0 && decltype(d)::value * Q / (4 * FA) == q)
                fa_nxt[decltype(d)::value / 4][decltype(d)::value % 4] ^= amask;
            });
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    wait_vmcnt<NLD>();  // the loads of step kt+2 (issued during step kt-1) have landed
    __syncthreads();
  };
  int kt = 0;
  if (KT & 1) {  // odd step count: one step first, then hand its prefetched fragments to set 0
    step(0, fa0, fa1);
    static_for<2 * TM>([&](auto x) { fa0[x] = fa1[x]; });
    kt = 1;
  }
  for (; kt < KT; kt += 2) {
    step(kt, fa0, fa1);
    step(kt + 1, fa1, fa0);
  }
  wait_vmcnt<0>();  // no load may still be writing LDS when the epilogue reuses it
  __syncthreads();
  if constexpr ((ITEXHIP_ABLATE & 16) != 0) {  // every accumulator stays live, nothing is stored
    int all = 0;
#pragma unroll
    for (int t = 0; t < TN * TM; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) all ^= acc[t][r];
    if (all == 0x12345678) reinterpret_cast<int*>(out)[threadIdx.x] = all;
    return;
  }

  // ---- epilogue.  Fast path: convert in registers, transpose through a private LDS buffer (the ring
  // is free after the last barrier) and store rows of 128 contiguous bytes, 16 B per lane.  A lane of
  // the MFMA layout owns one row and scattered 4-channel groups, which would make every store a
  // 64-address scatter.  The buffer holds [WM rows][ROWB bytes] with a 16-byte pad per row: for 8-bit
  // outputs all TN channel tiles at once, for 32-bit outputs one channel tile per pass.
  constexpr int ESZ = (OUT_T == ITEXHIP_QINT8 || OUT_T == ITEXHIP_QUINT8) ? 1 : is_float16_type(OUT_T) ? 2 : 4;
  constexpr int JB = (ESZ == 1) ? TN : (ESZ == 2) ? ((TN % 2 == 0) ? 2 : TN) : 1;  // channel tiles per pass
  constexpr int ROWB = JB * 32 * ESZ;        // row bytes in the buffer
  constexpr int PITCH = ROWB + 16;
  constexpr int LPR = ROWB / 16;             // lanes per row when flushing
  constexpr int RPP = 64 / LPR;              // rows per flush instruction (lanes >= RPP * LPR idle)
  constexpr int PASSES = (WM + RPP - 1) / RPP;
  static_assert(NW * WM * PITCH <= NSTAGE * STAGE_BYTES, "epilogue buffer must fit in the ring");
  if constexpr (!GENERAL) {
    uint8_t* ebuf = lds + wave * (WM * PITCH);
    const int f_row = lane / LPR, f_piece = lane % LPR;
    // Post-op chain in canonical form (ACT == 2: cheap activation, ACT == 3: GELU or another transcendental one; then
    // an optional linear map),
    // applied to the 16 values of one 32x32 tile at a time under wavefront-uniform branches.  A loop over the chain
    // with a switch per value made the epilogue several times longer than the whole K loop (instruction fetch, not
    // arithmetic).  Same expressions as apply_eltwise.
    // the addend of the 16 values of a tile: row m, channels n0 + 8 g + r (g, r < 4); 4 consecutive channels are
    // one 16-byte (fp32), 8-byte (16-bit types) or 4-byte (8-bit types) load, aligned because N is a multiple of 4 and
    // the host checked the base
    auto add_sum = [&](float (&v)[16], int m, int n0) {
      const CanonChain& c = e.canon;
      if (m >= M) return;
      // An 8-bit addend (the residual of a ResNet block): the lane's 16 values are dwords lgrp, 2 + lgrp, 4 + lgrp and
      // 6 + lgrp of the 32 bytes its row has in this tile.  Read as four single dwords a wavefront load fetched 8 bytes
      // of each of 32 rows (56x56x64 -> 256 with a quint8 addend: 18.9 us without the Sum, 49.3 us with it); the whole
      // row segment in two 16-byte loads (4-byte aligned: N % 4 == 0) brings that to 39.3 us.  Fetching the segments a
      // column of tiles ahead measured slower (43.1 us), and staging the addend through LDS in rows of contiguous bytes
      // gained only 1 us more: the rest of the Sum's cost is the arithmetic of the general chain epilogue, not memory.
      const bool addend8 = e.addend_type == ITEXHIP_QUINT8 || e.addend_type == ITEXHIP_QINT8;
      const int seg = n0 - lgrp * 4;  // first channel of the tile
      if (addend8 && seg + 32 <= N) {
        typedef int v4i_a4 __attribute__((ext_vector_type(4), aligned(4)));
        const uint8_t* src = static_cast<const uint8_t*>(e.addend) + static_cast<int64_t>(m) * N + seg;
        const v4i_a4 lo = *reinterpret_cast<const v4i_a4*>(src), hi = *reinterpret_cast<const v4i_a4*>(src + 16);
        const uint32_t w4[4] = {static_cast<uint32_t>(lgrp ? lo.y : lo.x), static_cast<uint32_t>(lgrp ? lo.w : lo.z),
                                static_cast<uint32_t>(lgrp ? hi.y : hi.x), static_cast<uint32_t>(lgrp ? hi.w : hi.z)};
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const uint32_t w = w4[g];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float a = e.addend_type == ITEXHIP_QUINT8 ? static_cast<float>((w >> (8 * r)) & 0xffu)
                                                            : static_cast<float>(static_cast<int>(w << (24 - 8 * r)) >> 24);
            v[g * 4 + r] = v[g * 4 + r] + c.sum_scale * a;
          }
        }
        return;
      }
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + g * 8;
        if (n < N) {
          const int64_t o = static_cast<int64_t>(m) * N + n;
          float a[4];
          if (e.addend_type == ITEXHIP_FLOAT) {
            const f4 t = *reinterpret_cast<const f4*>(static_cast<const float*>(e.addend) + o);
            a[0] = t[0]; a[1] = t[1]; a[2] = t[2]; a[3] = t[3];
          } else if (is_float16_type(e.addend_type)) {
            const uint2 t = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(e.addend) + o);
            const uint32_t h[4] = {t.x & 0xffffu, t.x >> 16, t.y & 0xffffu, t.y >> 16};
#pragma unroll
            for (int r = 0; r < 4; ++r) a[r] = e.addend_type == ITEXHIP_BFLOAT16 ? bf16_bits_to_f32(h[r]) : f16_bits_to_f32(h[r]);
          } else {
            const uint32_t w = *reinterpret_cast<const uint32_t*>(static_cast<const uint8_t*>(e.addend) + o);
            if (e.addend_type == ITEXHIP_QUINT8) {
#pragma unroll
              for (int r = 0; r < 4; ++r) a[r] = static_cast<float>((w >> (8 * r)) & 0xffu);
            } else {
#pragma unroll
              for (int r = 0; r < 4; ++r) a[r] = static_cast<float>(static_cast<int>(w << (24 - 8 * r)) >> 24);
            }
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) v[g * 4 + r] = v[g * 4 + r] + c.sum_scale * a[r];
        }
      }
    };
    // the same sum with the lane's 16 addend values already at hand (staged through the transposition buffer)
    auto add_staged = [&](float (&v)[16], const f4 (&ad)[4]) {
      const CanonChain& c = e.canon;
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int r = 0; r < 4; ++r) v[g * 4 + r] = v[g * 4 + r] + c.sum_scale * ad[g][r];
    };
    auto apply_chain = [&](float (&v)[16], int m, int n0, const f4 (&ad)[4], bool staged) {
      const CanonChain& c = e.canon;
      if (c.flags & kChainSumFirst) {
        if (staged) add_staged(v, ad); else add_sum(v, m, n0);
      }
      if constexpr (ACT == 3) {
        if (c.flags & kChainGeluTanh) {
          const itexhip_eltwise el{ITEXHIP_ELT_GELU_TANH, 0.0f, 0.0f};
#pragma unroll
          for (int r = 0; r < 16; ++r) v[r] = apply_eltwise(el, v[r]);
        } else if (c.flags & kChainGeluErf) {
          const itexhip_eltwise el{ITEXHIP_ELT_GELU_ERF, 0.0f, 0.0f};
#pragma unroll
          for (int r = 0; r < 16; ++r) v[r] = apply_eltwise(el, v[r]);
        } else {  // one of the other transcendental ones: a uniform switch around each 16-value loop
          const float al = c.other.alpha;
          switch (c.other.alg) {
            case ITEXHIP_ELT_ELU: {
              const itexhip_eltwise el{ITEXHIP_ELT_ELU, al, 0.0f};
#pragma unroll
              for (int r = 0; r < 16; ++r) v[r] = apply_eltwise(el, v[r]);
              break;
            }
            case ITEXHIP_ELT_LOGISTIC: {
              const itexhip_eltwise el{ITEXHIP_ELT_LOGISTIC, al, 0.0f};
#pragma unroll
              for (int r = 0; r < 16; ++r) v[r] = apply_eltwise(el, v[r]);
              break;
            }
            case ITEXHIP_ELT_TANH: {
              const itexhip_eltwise el{ITEXHIP_ELT_TANH, al, 0.0f};
#pragma unroll
              for (int r = 0; r < 16; ++r) v[r] = apply_eltwise(el, v[r]);
              break;
            }
            case ITEXHIP_ELT_SWISH: {
              const itexhip_eltwise el{ITEXHIP_ELT_SWISH, al, 0.0f};
#pragma unroll
              for (int r = 0; r < 16; ++r) v[r] = apply_eltwise(el, v[r]);
              break;
            }
            default: {
              const itexhip_eltwise el{ITEXHIP_ELT_MISH, al, 0.0f};
#pragma unroll
              for (int r = 0; r < 16; ++r) v[r] = apply_eltwise(el, v[r]);
              break;
            }
          }
        }
      } else {
        if (c.flags & kChainMax0) {
#pragma unroll
          for (int r = 0; r < 16; ++r) v[r] = fmaxf(v[r], 0.0f);
        }
        if (c.flags & kChainLeaky) {
#pragma unroll
          for (int r = 0; r < 16; ++r) v[r] = v[r] > 0.0f ? v[r] : v[r] * c.alpha;
        }
        if (c.flags & kChainClip) {
#pragma unroll
          for (int r = 0; r < 16; ++r) v[r] = fminf(fmaxf(v[r], c.lo), c.hi);
        }
      }
      if (c.flags & kChainSumLast) {
        if (staged) add_staged(v, ad); else add_sum(v, m, n0);
      }
      if (c.flags & kChainLinear) {
#pragma unroll
        for (int r = 0; r < 16; ++r) v[r] = c.lin_a * v[r] + c.lin_b;
      }
    };
    // A float addend (the MatMul's "Add" fusion with a float result) is read the way the result is written: every
    // wavefront load takes 8 rows x 128 contiguous bytes, whole memory lines, into the rows of the transposition buffer
    // that the results of the same 32 x 32 tile overwrite a moment later, and each lane picks its 16 values up from
    // there.  Read in the accumulator layout a wavefront load took 32 bytes of each of 32 rows and the addend cost
    // twice its bytes in fetches.  The loads of the next tile are in flight while the current one is worked on.
    constexpr bool CAN_STAGE = (ESZ == 4 && ACT >= 2 && JB == 1 && RPP == 8);
    const bool stage_addend = CAN_STAGE && e.addend_type == ITEXHIP_FLOAT &&
                              (e.canon.flags & (kChainSumFirst | kChainSumLast)) != 0;
    // AD tiles ahead, all of them in flight from the start of the epilogue: a tile is worked through in a fraction of a
    // memory round trip, so with one tile ahead every tile waited for its own round trip (BERT-base 3072 -> 768 with
    // the residual: 21.6 us against 13 us without the Add).
    constexpr int AD = CAN_STAGE ? (TM * TN < 4 ? TM * TN : 4) : 1;
    f4 ad_q[AD][4];
    auto fetch_addend = [&](auto slot, int i, int j) {  // rows of row tile i, channel tile j, flush layout
      const int n_col = n_base + (wn * TN + j) * 32 + f_piece * 4;
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int m = m_base + wm * WM + i * 32 + p * 8 + f_row;
        ad_q[decltype(slot)::value][p] = f4{0.0f, 0.0f, 0.0f, 0.0f};
        if (m < M && n_col < N)
          ad_q[decltype(slot)::value][p] = *reinterpret_cast<const f4*>(static_cast<const float*>(e.addend) + static_cast<int64_t>(m) * N + n_col);
      }
    };
    if constexpr (CAN_STAGE) {
      if (stage_addend)  // tiles in the order of the loops below: t = j * TM + i
        static_for<AD>([&](auto t) { fetch_addend(t, decltype(t)::value % TM, decltype(t)::value / TM); });
    }
    static_for<TN / JB>([&](auto jb) {
      static_for<JB>([&](auto jj) {
        constexpr int j = decltype(jb)::value * JB + decltype(jj)::value;
        auto put = [&](auto i, auto g, const v4i o) {
          uint8_t* dst = ebuf + (decltype(i)::value * 32 + lrow) * PITCH +
                         (decltype(jj)::value * 32 + decltype(g)::value * 8 + lgrp * 4) * ESZ;
          if constexpr (ESZ == 1) *reinterpret_cast<int*>(dst) = o.x;
          else if constexpr (ESZ == 2) *reinterpret_cast<int2*>(dst) = make_int2(o.x, o.y);
          else *reinterpret_cast<v4i*>(dst) = o;
        };
        if constexpr (ACT >= 2) {
          f4 sc[4], bi[4];
          static_for<4>([&](auto g) {
            const int col = (wn * TN + j) * 32 + decltype(g)::value * 8 + lgrp * 4;
            sc[decltype(g)::value] = *reinterpret_cast<const f4*>(panel_scale + col);
            bi[decltype(g)::value] = *reinterpret_cast<const f4*>(panel_bias + col);
          });
          static_for<TM>([&](auto i) {
            constexpr int ii = decltype(i)::value;
            constexpr int t = j * TM + ii;
            f4 ad[4] = {};
            if constexpr (CAN_STAGE) {
              if (stage_addend) {
#pragma unroll
                for (int p = 0; p < 4; ++p)
                  *reinterpret_cast<f4*>(ebuf + (ii * 32 + p * 8 + f_row) * PITCH + f_piece * 16) = ad_q[t % AD][p];
                if constexpr (t + AD < TM * TN)  // the tile AD further on takes the registers just emptied
                  fetch_addend(std::integral_constant<int, t % AD>{}, (t + AD) % TM, (t + AD) / TM);
#pragma unroll
                for (int g = 0; g < 4; ++g)
                  ad[g] = *reinterpret_cast<const f4*>(ebuf + (ii * 32 + lrow) * PITCH + (g * 8 + lgrp * 4) * 4);
              }
            }
            float v[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              v[r] = static_cast<float>(acc[t][r]) * sc[r >> 2][r & 3];
              v[r] = v[r] + bi[r >> 2][r & 3];
            }
            apply_chain(v, m_base + (wm * TM + ii) * 32 + lrow, n_base + (wn * TN + j) * 32 + lgrp * 4, ad,
                        CAN_STAGE && stage_addend);
            static_for<4>([&](auto g) {
              constexpr int r0 = decltype(g)::value * 4;
              put(i, g, epilogue_pack<OUT_T>(v4i{__float_as_int(v[r0]), __float_as_int(v[r0 + 1]), __float_as_int(v[r0 + 2]),
                                                 __float_as_int(v[r0 + 3])}));
            });
          });
        } else {
          static_for<4>([&](auto g) {
            const int col = (wn * TN + j) * 32 + decltype(g)::value * 8 + lgrp * 4;
            const f4 sc = *reinterpret_cast<const f4*>(panel_scale + col);
            const f4 bi = *reinterpret_cast<const f4*>(panel_bias + col);
            static_for<TM>([&](auto i) {
              constexpr int t = j * TM + decltype(i)::value;
              constexpr int r0 = decltype(g)::value * 4;
              const v4i part = v4i{acc[t][r0], acc[t][r0 + 1], acc[t][r0 + 2], acc[t][r0 + 3]};
              put(i, g, epilogue_convert<OUT_T, ACT>(part, sc, bi, e));
            });
          });
        }
      });
      // flush: lane -> (row, 16-byte piece); LDS operations of one wavefront complete in order
      const int n_col = n_base + (wn * TN + decltype(jb)::value * JB) * 32 + f_piece * (16 / ESZ);
#pragma unroll
      for (int pass = 0; pass < PASSES; ++pass) {
        const int row = min(pass * RPP + f_row, WM - 1);
        const v4i v = *reinterpret_cast<const v4i*>(ebuf + row * PITCH + f_piece * 16);
        const int m = m_base + wm * WM + row;
        const bool mine = (64 % LPR == 0 || f_row < RPP) && (WM % RPP == 0 || pass * RPP + f_row < WM);
        if (mine && m < M && n_col < N) {  // N * ESZ is a multiple of 16, so a piece is entirely inside or outside
          // Neither form leaves the output dirty in L2 until the flush at the end of the kernel.  32-bit outputs (the
          // store-bound epilogues: BERT-base 768 -> 3072 + ReLU 19.5 -> 17.6 us) go out as system-scope stores, written
          // through; 8- and 16-bit outputs, and the GELU epilogue whose stores trickle out between long runs of
          // arithmetic, measured 1-8 % faster as streaming (nontemporal) stores.
          uint8_t* const dst = reinterpret_cast<uint8_t*>(out) + (static_cast<int64_t>(m) * N + n_col) * ESZ;
          // (the s_nop: a store of more than 8 bytes reads its data registers for a cycle or two after it issues, and the
          // compiler, which cannot see a store inside the assembly, may let the next vector instruction overwrite them)
          if constexpr (ESZ == 4 && ACT != 3) asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(dst), "v"(v) : "memory");
          else __builtin_nontemporal_store(v, reinterpret_cast<v4i*>(dst));
        }
      }
    });
  } else {
    const bool has_bias = e.bias != nullptr || e.fused;
    static_for<TN>([&](auto j) {
      static_for<4>([&](auto g) {
        const int col = (wn * TN + j) * 32 + decltype(g)::value * 8 + lgrp * 4;
        const int n = n_base + col;
        if (n < N) {
          const f4 sc = *reinterpret_cast<const f4*>(panel_scale + col);
          const f4 bi = *reinterpret_cast<const f4*>(panel_bias + col);
          static_for<TM>([&](auto i) {
            constexpr int t = decltype(j)::value * TM + decltype(i)::value;
            constexpr int r0 = decltype(g)::value * 4;
            const int m = m_base + (wm * TM + i) * 32 + lrow;
            if (m < M) {
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                if (n + r < N) {
                  float v = static_cast<float>(acc[t][r0 + r]) * sc[r];
                  if (has_bias) v = v + bi[r];
                  const int64_t o = static_cast<int64_t>(m) * N + n + r;
                  for (int k = 0; k < e.n_eltwise; ++k) {
                    if (e.elt[k].alg == ITEXHIP_ELT_SUM) v = v + e.elt[k].alpha * load_addend(e, o);
                    else v = apply_eltwise(e.elt[k], v);
                  }
                  store_output<OUT_T>(out, o, v);
                }
              }
            }
          });
        }
      });
    });
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int OUT_T, int ACT, bool KALIGNED, bool CONV = false, bool ELEMENTWISE = false>
int launch_tile(const uint8_t* a, uint32_t amask, const uint8_t* bp, int M, int K, int N, const EpilogueArgs& e,
                void* out, hipStream_t st, typename conv_args_of<CONV>::type cv = {}) {
  const int KT = (K + 63) / 64, NT = (N + kChunkRows - 1) / kChunkRows;
  const int num_m = (M + BM - 1) / BM, num_n = (N + BN - 1) / BN;
  constexpr size_t lds_bytes = 4 * (BM / 16 + BN / 16) * kChunkBytes + 12 * BN + (CONV ? kMaxConvPieces * 8 : 0);  // the most
  const size_t lds_now = lds_bytes - (CONV ? (kMaxConvPieces - (K >> 4)) * 8 : 0);
  auto kern = qgemm_tile_kernel<BM, BN, WAVES_M, WAVES_N, OUT_T, ACT, KALIGNED, CONV, ELEMENTWISE>;
  static unsigned long long attr_done = 0;  // devices on which this instantiation's attribute is set
  if (!device_bit(&attr_done, false)) {
    hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (err != hipSuccess) return hip_fail(err, "hipFuncSetAttribute(qgemm_tile_kernel)");
    device_bit(&attr_done, true);
  }
  kern<<<dim3(static_cast<unsigned>(num_m * num_n)), dim3(64 * WAVES_M * WAVES_N), lds_now, st>>>(
      a, amask, bp, M, K, N, KT, NT, num_m, num_n, xcd_rectangles(num_m, num_n, BM, BN, K), e, out, cv);
  return ITEXHIP_OK;
}

// Tile shape: the one with the smallest estimated time = rounds of workgroups over the 256 CUs x
// tile area x a penalty for the operand traffic per MFMA of smaller tiles.
//
// long_epilogue_short_k: a transcendental activation (GELU ...) on a short K.  The epilogue is then a large part of the
// launch, and 128 x 128 tiles, two or three workgroups per CU, run one tile's epilogue under another's K loop: BERT-base
// 768 -> 3072 + GeluApproximate at 4096 tokens 22.4 -> 20.0 us (fp32), 20.8 -> 17.2 us (bfloat16); measured on 4096 x 3072,
// 2048 x 4096 and 4096 x 4096 outputs the small tiles win up to K = 1536 - 2048 and lose beyond (the K loop's operand
// traffic), and lose at any K when there are fewer than two tiles per CU (512 x 3072).  With any epilogue the same holds
// up to K = 256, where a launch is little more than its epilogue (100352 x 256 outputs, the last 1 x 1 convolution of a
// ResNet-50 block, K = 64: 18.7 -> 12.4 us, with the residual Sum 39.5 -> 20.5 us; 4096 x 3072, 16384 x 1024 and
// 2048 x 14336 outputs, 8-bit and fp32: 5 - 30 % faster at K = 64 - 256, mixed at 384, slower from 512 on).
inline int pick_tile_shape(int M, int N, bool wide_only, int first = 0, bool long_epilogue_short_k = false) {
  struct Shape { int bm, bn; double penalty; };
  static const Shape shapes[5] = {{256, 256, 1.0}, {256, 192, 1.03}, {256, 128, 1.08}, {128, 128, 1.2}, {64, 64, 1.8}};
  // itexhip_test_force_tile_shape forces a shape (tests exercise every shape on ragged problems with it)
  const int f = __atomic_load_n(&g_forced_tile_shape[0], __ATOMIC_RELAXED);
  if (f >= (wide_only ? 3 : first) && f < 5) return f;
  if (long_epilogue_short_k) {  // at least two 128 x 128 tiles per CU, at most 15 % of their area outside the output
    const int64_t t128 = static_cast<int64_t>((M + 127) / 128) * ((N + 127) / 128);
    if (t128 >= 512 && t128 * (128 * 128) * 100 <= static_cast<int64_t>(M) * N * 115) return 3;
  }
  int best = 3;
  double best_cost = 1e300;
  for (int i = wide_only ? 3 : first; i < 5; ++i) {
    const double tiles = static_cast<double>((M + shapes[i].bm - 1) / shapes[i].bm) * ((N + shapes[i].bn - 1) / shapes[i].bn);
    const double rounds = std::ceil(tiles / 256.0);
    const double cost = rounds * shapes[i].bm * shapes[i].bn * shapes[i].penalty;
    if (cost < best_cost) { best_cost = cost; best = i; }
  }
  return best;
}

template <int OUT_T, int ACT>
int dispatch_tile_shape(const uint8_t* a, uint32_t amask, const uint8_t* bp, int M, int K, int N,
                        const EpilogueArgs& e, void* out, hipStream_t st) {
  switch (pick_tile_shape(M, N, false, 0, (ACT == 3 && K <= 1536) || K <= 256)) {
    case 0: return launch_tile<256, 256, 2, 2, OUT_T, ACT, true>(a, amask, bp, M, K, N, e, out, st);
    case 1: return launch_tile<256, 192, 2, 2, OUT_T, ACT, true>(a, amask, bp, M, K, N, e, out, st);
    case 2: return launch_tile<256, 128, 2, 2, OUT_T, ACT, true>(a, amask, bp, M, K, N, e, out, st);
    // (128 x 128 with eight wavefronts of 32 x 64: two per SIMD cover each other's waits in the prologue and in the
    // epilogue - BERT-base 768 -> 768 6.85 -> 6.58 us, 3072 -> 768 with the residual Add 18.9 -> 17.4 us, the K loop of
    // 3072 -> 768 unchanged; the same split of the 256 x 128 tile changed nothing)
    case 3: return launch_tile<128, 128, 4, 2, OUT_T, ACT, true>(a, amask, bp, M, K, N, e, out, st);
    default: return launch_tile<64, 64, 2, 2, OUT_T, ACT, true>(a, amask, bp, M, K, N, e, out, st);
  }
}

// A bias vector, 16-byte aligned output rows and a post-op chain of the canonical form take the vector epilogue:
// with K a multiple of 64 the specialised kernels (uniform activation addresses) in every tile shape; other K:
// per-lane clamped activation loads, two tile shapes.
// A missing bias, an addend, other chains or unaligned outputs (rare) go to the element-wise epilogue, a kernel of
// its own in two shapes.
template <int OUT_T>
int dispatch_tile(const uint8_t* a, uint32_t a_xor, const uint8_t* bp, int M, int K, int N,
                  const EpilogueArgs& e_in, void* out, hipStream_t st) {
  constexpr int esz = (OUT_T == ITEXHIP_QINT8 || OUT_T == ITEXHIP_QUINT8) ? 1 : is_float16_type(OUT_T) ? 2 : 4;
  EpilogueArgs e = e_in;
  const int act = canon_chain(e, &e.canon);
  const bool has_sum = (e.canon.flags & (kChainSumFirst | kChainSumLast)) != 0;
  const bool sum_ok = !has_sum || (e.addend != nullptr && (N & 3) == 0 &&
                                   (reinterpret_cast<uintptr_t>(e.addend) &
                                    (e.addend_type == ITEXHIP_FLOAT ? 15 : is_float16_type(e.addend_type) ? 7 : 3)) == 0);
  const bool vec_epilogue = act >= 0 && sum_ok && (e.bias != nullptr || e.fused) &&
                            (reinterpret_cast<uintptr_t>(out) & 15) == 0 && ((static_cast<int64_t>(N) * esz) & 15) == 0;
  const bool wide = pick_tile_shape(M, N, true) == 3;
  if (vec_epilogue && (K & 63) == 0) {
    if (act == 0) return dispatch_tile_shape<OUT_T, 0>(a, a_xor, bp, M, K, N, e, out, st);
    if (act == 1) return dispatch_tile_shape<OUT_T, 1>(a, a_xor, bp, M, K, N, e, out, st);
    if (act == 2) return dispatch_tile_shape<OUT_T, 2>(a, a_xor, bp, M, K, N, e, out, st);
    return dispatch_tile_shape<OUT_T, 3>(a, a_xor, bp, M, K, N, e, out, st);
  }
  if (vec_epilogue && act == 3) {
    if (wide) return launch_tile<128, 128, 2, 2, OUT_T, 3, false>(a, a_xor, bp, M, K, N, e, out, st);
    return launch_tile<64, 64, 2, 2, OUT_T, 3, false>(a, a_xor, bp, M, K, N, e, out, st);
  }
  if (vec_epilogue) {  // the canonical chain covers "none" and "ReLU" too
    if (wide) return launch_tile<128, 128, 2, 2, OUT_T, 2, false>(a, a_xor, bp, M, K, N, e, out, st);
    return launch_tile<64, 64, 2, 2, OUT_T, 2, false>(a, a_xor, bp, M, K, N, e, out, st);
  }
  if (wide) return launch_tile<128, 128, 2, 2, OUT_T, 2, false, false, true>(a, a_xor, bp, M, K, N, e, out, st);
  return launch_tile<64, 64, 2, 2, OUT_T, 2, false, false, true>(a, a_xor, bp, M, K, N, e, out, st);
}

// Implicit GEMM of a Conv2D: `x` is the NHWC input, M = batch * out_h * out_w, K = k_h * k_w * in_c.  Run-time post-op
// chain in canonical form, vector epilogue (the host checks that the output allows it), three tile shapes (a
// 256 x 64 shape with four wavefronts stacked along M was slower than 64 x 64 tiles for 64 output channels).
template <int OUT_T>
int dispatch_tile_conv(const uint8_t* x, uint32_t a_xor, const uint8_t* bp, int M, int K, int N, const EpilogueArgs& e_in,
                       void* out, hipStream_t st, const ConvTileArgs& cv) {
  EpilogueArgs e = e_in;
  const int act = canon_chain(e, &e.canon);
  if (act < 0 || act == 3) {
    set_error("itexhip_qconv2d: the post-ops must be [sum] [ReLU / LeakyReLU / clip] [sum] [linear map], at most one sum");
    return ITEXHIP_INVALID_ARGUMENT;
  }
  if ((e.canon.flags & (kChainSumFirst | kChainSumLast)) &&
      (e.addend == nullptr || (N & 3) != 0 || (reinterpret_cast<uintptr_t>(e.addend) & (e.addend_type == ITEXHIP_FLOAT ? 15 : 3)) != 0)) {
    set_error("itexhip_qconv2d_sum: the summand must be 4-byte (8-bit types) or 16-byte (float) aligned and out_channels a multiple of 4");
    return ITEXHIP_INVALID_ARGUMENT;
  }
  struct Shape { int bm, bn; double penalty; };
  static const Shape shapes[3] = {{256, 128, 1.08}, {128, 128, 1.2}, {64, 64, 1.8}};
  int best = 0;
  double best_cost = 1e300;
  for (int i = 0; i < 3; ++i) {
    const double tiles = static_cast<double>((M + shapes[i].bm - 1) / shapes[i].bm) * ((N + shapes[i].bn - 1) / shapes[i].bn);
    const double cost = std::ceil(tiles / 256.0) * shapes[i].bm * shapes[i].bn * shapes[i].penalty;
    if (cost < best_cost) { best_cost = cost; best = i; }
  }
  const int f = __atomic_load_n(&g_forced_tile_shape[1], __ATOMIC_RELAXED);  // tests exercise every shape with it
  if (f >= 0 && f < 3) best = f;
  switch (best) {
    case 0: return launch_tile<256, 128, 2, 2, OUT_T, 2, false, true>(x, a_xor, bp, M, K, N, e, out, st, cv);
    case 1: return launch_tile<128, 128, 2, 2, OUT_T, 2, false, true>(x, a_xor, bp, M, K, N, e, out, st, cv);
    default: return launch_tile<64, 64, 2, 2, OUT_T, 2, false, true>(x, a_xor, bp, M, K, N, e, out, st, cv);
  }
}

}  // namespace itexhip
#endif  // ITEXHIP_QGEMM_TILE_HPP_
