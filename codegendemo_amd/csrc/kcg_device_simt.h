// kcg_device_simt.h — kernel family 1: the scalar-FMA register-tiled kernel that follows the tuning config literally.
#pragma once
#include "kcg_device_common.h"

namespace kcg {

// =============================================================================================
// Family 1: SIMT kernel — the literal schedule.
// =============================================================================================
template <class C>
__device__ __forceinline__ void gemm_simt(const typename C::TA* __restrict__ A, const typename C::TB* __restrict__ B,
                                          typename C::TC* __restrict__ Cm, char* smem, EpiArgs ep = EpiArgs{1.f, 0.f}) {
  typedef typename C::TA TA;
  typedef typename C::TB TB;
  typedef typename C::TC TC;
  typedef typename C::ACC ACC;
  constexpr int BM = C::BM, BN = C::BN, BK = C::BK, TM = C::TM, TN = C::TN, LSU = C::LSU;
  constexpr int M = C::M, N = C::N, K = C::K;
  constexpr int BX = BN / TN, BY = BM / TM, NTXY = BX * BY, NT = NTXY * LSU;
  constexpr int LDA = BM + C::SIMT_PAD_A, LDB = BN + C::SIMT_PAD_B;  // LDS rows: smA[BK][LDA], smB[BK][LDB]
  constexpr int STAGES = C::SHMP ? 2 : 1;
  constexpr int KT = cdiv(K, BK);
  constexpr bool EDGE = C::EDGE;

  constexpr int SMB_OFF = (STAGES * BK * LDA * (int)sizeof(TA) + 15) & ~15;
  TA* smA = reinterpret_cast<TA*>(smem);
  TB* smB = reinterpret_cast<TB*>(smem + SMB_OFF);

  const int tid = threadIdx.x;
  const int tz = tid / NTXY;                // split-U slice of this thread (Optimizer.cc:159-162)
  const int t = tid % NTXY;
  const int warp = t / C::WARP_SIZE, lane = t % C::WARP_SIZE;
  const int warp_y = warp / C::BLN, warp_x = warp % C::BLN;     // Utils.cc:250-256
  const int lane_y = lane / C::WLN, lane_x = lane % C::WLN;     // Utils.cc:262-268
  int by, bx;
  block_coords<C>(blockIdx.x, by, bx);
  const int m0 = by * BM, n0 = bx * BN;

  // ---- global -> register staging maps -------------------------------------------------------
  // A^T tile (IS_ATRANS=1): BK rows x BM cols, contiguous along m.  A tile (IS_ATRANS=0): BM rows x
  // BK cols, contiguous along k, transposed while it is written to smA[k][m].
  constexpr int GLW_A = C::GLW_A, GLW_B = C::GLW_B;
  constexpr bool LC_A = C::LC != 0 || (NT % BK != 0) || (BM % ((NT / BK) * GLW_A) != 0);
  constexpr bool LC_B = C::LC != 0 || (NT % BK != 0) || (BN % ((NT / BK) * GLW_B) != 0);
  typedef TileMap<BK, BM, GLW_A, NT, LC_A> MapAT;    // IS_ATRANS=1
  typedef TileMap<BM, BK, GLW_A, NT, true> MapAN;    // IS_ATRANS=0
  typedef TileMap<BK, BN, GLW_B, NT, LC_B> MapB;
  constexpr int ITERS_A = C::ATRANS ? MapAT::ITERS : MapAN::ITERS;
  constexpr bool AL_A = C::ATRANS ? (M % GLW_A == 0) : (K % GLW_A == 0);
  constexpr bool AL_B = (N % GLW_B == 0);

  TA tempA[ITERS_A][GLW_A];
  TB tempB[MapB::ITERS][GLW_B];

  auto load_global = [&](int kt) {
    const int k0 = kt * BK;
#pragma unroll
    for (int it = 0; it < ITERS_A; ++it) {
      int r, c;
      if constexpr (C::ATRANS) {
        if (MapAT::coords(tid, it, r, c)) gload<TA, GLW_A, EDGE, AL_A>(tempA[it], A, k0 + r, m0 + c, M, K, M);
      } else {
        if (MapAN::coords(tid, it, r, c)) gload<TA, GLW_A, EDGE, AL_A>(tempA[it], A, m0 + r, k0 + c, K, M, K);
      }
    }
#pragma unroll
    for (int it = 0; it < MapB::ITERS; ++it) {
      int r, c;
      if (MapB::coords(tid, it, r, c)) gload<TB, GLW_B, EDGE, AL_B>(tempB[it], B, k0 + r, n0 + c, N, K, N);
    }
  };
  auto store_lds = [&](int stage) {
    TA* sa = smA + stage * BK * LDA;
    TB* sb = smB + stage * BK * LDB;
#pragma unroll
    for (int it = 0; it < ITERS_A; ++it) {
      int r, c;
      if constexpr (C::ATRANS) {
        if (MapAT::coords(tid, it, r, c)) copy_bytes<GLW_A * (int)sizeof(TA)>(sa + r * LDA + c, tempA[it]);
      } else {
        if (MapAN::coords(tid, it, r, c)) {
#pragma unroll
          for (int e = 0; e < GLW_A; ++e) sa[(c + e) * LDA + r] = tempA[it][e];
        }
      }
    }
#pragma unroll
    for (int it = 0; it < MapB::ITERS; ++it) {
      int r, c;
      if (MapB::coords(tid, it, r, c)) copy_bytes<GLW_B * (int)sizeof(TB)>(sb + r * LDB + c, tempB[it]);
    }
  };

  // ---- LDS -> register fragments with the warp/thread scatter pattern (Optimizer.cc:151-183) ----
  constexpr int BRA = TM / C::WSW_A, WRA = C::WSW_A / C::TSW_A;
  constexpr int BRB = TN / C::WSW_B, WRB = C::WSW_B / C::TSW_B;
  auto load_frag = [&](int stage, int kk, TA* ra, TB* rb) {
    const TA* sa = smA + stage * BK * LDA + kk * LDA;
    const TB* sb = smB + stage * BK * LDB + kk * LDB;
#pragma unroll
    for (int i = 0; i < BRA; ++i)
#pragma unroll
      for (int j = 0; j < WRA; ++j)
        copy_bytes<C::TSW_A * (int)sizeof(TA)>(
            ra + i * C::WSW_A + j * C::TSW_A,
            sa + (i * C::BLM + warp_y) * C::WLM * C::WSW_A + (j * C::WLM + lane_y) * C::TSW_A);
#pragma unroll
    for (int i = 0; i < BRB; ++i)
#pragma unroll
      for (int j = 0; j < WRB; ++j)
        copy_bytes<C::TSW_B * (int)sizeof(TB)>(
            rb + i * C::WSW_B + j * C::TSW_B,
            sb + (i * C::BLN + warp_x) * C::WLN * C::WSW_B + (j * C::WLN + lane_x) * C::TSW_B);
  };

  ACC acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = ACC(0);

  auto fma_frag = [&](const TA* ra, const TB* rb) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] += (ACC)ra[i] * (ACC)rb[j];
  };

  constexpr int KSTEPS = BK / LSU;   // k values of one tile handled by this thread-z slice
  auto compute_tile = [&](int stage) {
    if constexpr (C::REGP) {
      // two k-steps per iteration with the two fragment buffers named explicitly: the compiler stops
      // unrolling very large bodies (TM*TN*BK beyond ~16k instructions), and a buffer chosen by a loop
      // counter that is no longer a constant would turn the register arrays into select chains
      TA ra0[TM], ra1[TM];
      TB rb0[TN], rb1[TN];
      load_frag(stage, tz, ra0, rb0);
#pragma unroll
      for (int s = 0; s < KSTEPS; s += 2) {
        if (s + 1 < KSTEPS) load_frag(stage, (s + 1) * LSU + tz, ra1, rb1);
        fma_frag(ra0, rb0);
        if (s + 1 < KSTEPS) {
          if (s + 2 < KSTEPS) load_frag(stage, (s + 2) * LSU + tz, ra0, rb0);
          fma_frag(ra1, rb1);
        }
      }
    } else {
      TA ra[TM];
      TB rb[TN];
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        load_frag(stage, s * LSU + tz, ra, rb);
        fma_frag(ra, rb);
      }
    }
  };

  // ---- K loop (Optimizer.cc:343-376; double buffer: Rewriter.cc:775-833) -----------------------
  if constexpr (C::SHMP) {
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < KT) load_global(kt + 1);
      compute_tile(cur);
      if (kt + 1 < KT) store_lds(cur ^ 1);
      __syncthreads();
    }
  } else {
    for (int kt = 0; kt < KT; ++kt) {
      load_global(kt);
      __syncthreads();
      store_lds(0);
      __syncthreads();
      compute_tile(0);
    }
  }

  // ---- epilogue -------------------------------------------------------------------------------
  if constexpr (LSU > 1) {
    ACC* smC = reinterpret_cast<ACC*>(smem);  // aliases smA/smB (Optimizer.cc:454-458)
    __syncthreads();
#pragma unroll
    for (int i0 = 0; i0 < BRA; ++i0)
#pragma unroll
      for (int i1 = 0; i1 < WRA; ++i1)
#pragma unroll
        for (int i2 = 0; i2 < C::TSW_A; ++i2) {
          const int row = (i0 * C::BLM + warp_y) * C::WLM * C::WSW_A + (i1 * C::WLM + lane_y) * C::TSW_A + i2;
          const int ri = i0 * C::WSW_A + i1 * C::TSW_A + i2;
#pragma unroll
          for (int j0 = 0; j0 < BRB; ++j0)
#pragma unroll
            for (int j1 = 0; j1 < WRB; ++j1) {
              const int col = (j0 * C::BLN + warp_x) * C::WLN * C::WSW_B + (j1 * C::WLN + lane_x) * C::TSW_B;
              const int rj = j0 * C::WSW_B + j1 * C::TSW_B;
#pragma unroll
              for (int j2 = 0; j2 < C::TSW_B; ++j2) smC[(tz * BM + row) * BN + col + j2] = acc[ri][rj + j2];
            }
        }
    __syncthreads();
    splitu_reduce_store<C, NT>(Cm, smC, tid, m0, n0, ep);
  } else {
    // direct store, TSW_B-wide pieces (Optimizer.cc:193-215,412-421)
    constexpr bool AL_C = (N % C::TSW_B == 0);
#pragma unroll
    for (int i0 = 0; i0 < BRA; ++i0)
#pragma unroll
      for (int i1 = 0; i1 < WRA; ++i1)
#pragma unroll
        for (int i2 = 0; i2 < C::TSW_A; ++i2) {
          const int row = (i0 * C::BLM + warp_y) * C::WLM * C::WSW_A + (i1 * C::WLM + lane_y) * C::TSW_A + i2;
          const int ri = i0 * C::WSW_A + i1 * C::TSW_A + i2;
#pragma unroll
          for (int j0 = 0; j0 < BRB; ++j0)
#pragma unroll
            for (int j1 = 0; j1 < WRB; ++j1) {
              const int col = (j0 * C::BLN + warp_x) * C::WLN * C::WSW_B + (j1 * C::WLN + lane_x) * C::TSW_B;
              const int rj = j0 * C::WSW_B + j1 * C::TSW_B;
              if constexpr (C::EPI) epi_apply<TC, ACC, C::TSW_B, EDGE, AL_C>(&acc[ri][rj], Cm, m0 + row, n0 + col, N, M, N, ep);
              gstore<TC, ACC, C::TSW_B, EDGE, AL_C>(Cm, &acc[ri][rj], m0 + row, n0 + col, N, M, N);
            }
        }
  }
}

}  // namespace kcg
