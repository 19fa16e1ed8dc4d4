// kcg_device_mfma.h — kernel family 2: the general wave-tiled matrix-core kernel.
#pragma once
#include "kcg_device_common.h"
#include "kcg_device_mfma_ops.h"
#include "kcg_device_direct.h"

namespace kcg {

// =============================================================================================
// Family 2: matrix-core kernel with register staging (global -> registers -> LDS): every flag
// combination, edge tiles, split-U, fp64.  Configs eligible for direct staging are handed on.
// =============================================================================================
template <class C>
__device__ __forceinline__ void gemm_mfma(const typename C::TA* __restrict__ A, const typename C::TB* __restrict__ B,
                                          typename C::TC* __restrict__ Cm, char* smem, EpiArgs ep = EpiArgs{1.f, 0.f}) {
  if constexpr (DirectPlan<C>::OK) {
    gemm_mfma_direct<C>(A, B, Cm, smem, ep);
    return;
  }
  typedef typename C::TA T;   // TA == TB for this family
  typedef typename C::TC TC;
  constexpr int BM = C::BM, BN = C::BN, BK = C::BK, LSU = C::LSU;
  constexpr int M = C::M, N = C::N, K = C::K;
  constexpr int ES = (int)sizeof(T);
  constexpr int G = 16 / ES;                  // k elements per 16-byte chunk
  constexpr int WM = BM / C::BLM, WN = BN / C::BLN;   // wave tile = (WLM*TM) x (WLN*TN)
  constexpr int MF = (ES != 8 && WM % 32 == 0 && WN % 32 == 0) ? 32 : 16;   // fp64 has the 16x16 shape only
  constexpr int KH = 64 / MF;                 // lane groups along k inside one instruction
  constexpr int KS = G * KH;                  // k covered by one fragment step
  constexpr int NSS = BK / KS;                // fragment steps per K tile
  constexpr int TMI = WM / MF, TNI = WN / MF; // matrix-core tiles per wave
  constexpr int CH = BK / G;                  // chunks per LDS row
  constexpr int NWXY = C::BLM * C::BLN;
  constexpr int NT = NWXY * 64 * LSU;
  constexpr int STAGES = C::SHMP ? 2 : 1;
  constexpr int KT = cdiv(K, BK);
  constexpr bool EDGE = C::EDGE;
  typedef Mfma<T, MF> MI;
  typedef typename MI::Acc Acc;
  typedef typename MI::Frag Frag;
  typedef typename AccOf<T>::type AccT;       // float, or double for fp64 inputs
  typedef LdsTile<CH> L;

  u32x4* smA = reinterpret_cast<u32x4*>(smem);               // [STAGES][BM*CH] chunks
  u32x4* smB = smA + STAGES * BM * CH;                       // [STAGES][BN*CH] chunks

  const int tid = threadIdx.x;
  const int wave = tid / 64, lane = tid % 64;
  const int wz = wave / NWXY;                 // split-U slice of this wave
  const int wxy = wave % NWXY;
  const int wy = wxy / C::BLN, wx = wxy % C::BLN;
  int by, bx;
  block_coords<C>(blockIdx.x, by, bx);
  const int m0 = by * BM, n0 = bx * BN;

  // ---- global -> registers -> LDS ------------------------------------------------------------
  // k-contiguous operand (A when IS_ATRANS=0): thread owns 16-byte chunks (row, c).
  constexpr int VK_A = cmin(C::GLW_A, G);
  typedef TileMap<BM, BK, G, NT, true> MapKA;
  // row(mn)-contiguous operand (B always, A when IS_ATRANS=1): thread owns a G(k) x VEC(mn) block,
  // loads G row vectors, transposes them in registers and writes VEC chunks.
  constexpr int VN_A = cmin(C::GLW_A, G);
  constexpr int VN_B = cmin(C::GLW_B, G);
  typedef BlockMap<CH, BM / VN_A, VN_A, NT, C::LC != 0> MapNA;
  typedef BlockMap<CH, BN / VN_B, VN_B, NT, C::LC != 0> MapNB;
  constexpr int ITERS_A = C::ATRANS ? MapNA::ITERS : MapKA::ITERS;
  constexpr int REGS_A = C::ATRANS ? G * VN_A : G;
  constexpr bool AL_A = C::ATRANS ? (M % VN_A == 0) : (K % VK_A == 0);
  constexpr bool AL_B = (N % VN_B == 0);

  T ga[ITERS_A][REGS_A];
  T gb[MapNB::ITERS][G * VN_B];

  // The staging work of one K tile is cut into items (one global vector load, or one 16-byte LDS
  // write, each) so that the pipelined loop below can place them one by one between matrix-core
  // instructions.  `idx` is a compile-time constant wherever these are called (unrolled loops).
  constexpr int LPA = C::ATRANS ? G : G / VK_A;   // global loads per A iteration
  constexpr int WPA = C::ATRANS ? VN_A : 1;       // LDS writes per A iteration
  constexpr int NLD_A = ITERS_A * LPA, NLD = NLD_A + MapNB::ITERS * G;
  constexpr int NWR_A = ITERS_A * WPA, NWR = NWR_A + MapNB::ITERS * VN_B;

  auto load_item = [&](int idx, int k0) {
    int r, c;
    if (idx < NLD_A) {
      const int it = idx / LPA, sub = idx % LPA;
      if constexpr (C::ATRANS) {   // r = k chunk, c = first m of the vector
        if (MapNA::coords(tid, it, r, c))
          gload<T, VN_A, EDGE, AL_A>(&ga[it][sub * VN_A], A, k0 + r * G + sub, m0 + c, M, K, M);
      } else {                     // r = m row, c = first k of the chunk
        if (MapKA::coords(tid, it, r, c))
          gload<T, VK_A, EDGE, AL_A>(&ga[it][sub * VK_A], A, m0 + r, k0 + c + sub * VK_A, K, M, K);
      }
    } else {
      const int it = (idx - NLD_A) / G, sub = (idx - NLD_A) % G;
      if (MapNB::coords(tid, it, r, c))
        gload<T, VN_B, EDGE, AL_B>(&gb[it][sub * VN_B], B, k0 + r * G + sub, n0 + c, N, K, N);
    }
  };
  auto write_item = [&](int idx, int stage) {
    u32x4* sa = smA + stage * BM * CH;
    u32x4* sb = smB + stage * BN * CH;
    int r, c;
    if (idx < NWR_A) {
      const int it = idx / WPA, e = idx % WPA;
      if constexpr (C::ATRANS) {
        if (MapNA::coords(tid, it, r, c)) {
          T chunk[G];
#pragma unroll
          for (int g = 0; g < G; ++g) chunk[g] = ga[it][g * VN_A + e];
          copy_bytes<16>(sa + L::slot(c + e, r), chunk);
        }
      } else {
        if (MapKA::coords(tid, it, r, c)) copy_bytes<16>(sa + L::slot(r, c / G), ga[it]);
      }
    } else {
      const int it = (idx - NWR_A) / VN_B, e = (idx - NWR_A) % VN_B;
      if (MapNB::coords(tid, it, r, c)) {
        T chunk[G];
#pragma unroll
        for (int g = 0; g < G; ++g) chunk[g] = gb[it][g * VN_B + e];
        copy_bytes<16>(sb + L::slot(c + e, r), chunk);
      }
    }
  };
  auto load_global = [&](int kt) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) load_item(i, kt * BK);
  };
  auto store_lds = [&](int stage) {
#pragma unroll
    for (int i = 0; i < NWR; ++i) write_item(i, stage);
  };

  // ---- fragments and matrix-core steps -------------------------------------------------------
  Acc acc[TMI][TNI];
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j)
#pragma unroll
      for (int e = 0; e < (int)(sizeof(Acc) / sizeof(AccT)); ++e) acc[i][j][e] = (AccT)0;

  const int frow = lane % MF;   // row of the MFMA tile this lane feeds
  const int fgrp = lane / MF;   // lane group along k
  auto load_frag = [&](int stage, int s, Frag* fa, Frag* fb) {
    const u32x4* sa = smA + stage * BM * CH;
    const u32x4* sb = smB + stage * BN * CH;
    const int c = s * KH + fgrp;
#pragma unroll
    for (int i = 0; i < TMI; ++i) copy_bytes<16>(&fa[i], sa + L::slot(wy * WM + i * MF + frow, c));
#pragma unroll
    for (int j = 0; j < TNI; ++j) copy_bytes<16>(&fb[j], sb + L::slot(wx * WN + j * MF + frow, c));
  };
  // fragment f of a step: f < TMI is the A fragment of tile row f, otherwise the B fragment f - TMI
  auto load_frag_item = [&](int stage, int s, int f, Frag* fa, Frag* fb) {
    const int c = s * KH + fgrp;
    if (f < TMI)
      copy_bytes<16>(&fa[f], smA + stage * BM * CH + L::slot(wy * WM + f * MF + frow, c));
    else
      copy_bytes<16>(&fb[f - TMI], smB + stage * BN * CH + L::slot(wx * WN + (f - TMI) * MF + frow, c));
  };
  auto mma_frag = [&](const Frag* fa, const Frag* fb) {
#pragma unroll
    for (int i = 0; i < TMI; ++i)
#pragma unroll
      for (int j = 0; j < TNI; ++j) MI::run(acc[i][j], fa[i], fb[j]);
  };

  constexpr int SPW = NSS / LSU;   // fragment steps of one tile handled by this wave's split-U slice
  constexpr int NM = TMI * TNI;    // matrix-core groups per step
  constexpr int NF = TMI + TNI;    // fragments per step
  constexpr int MT = SPW * NM;     // matrix-core groups per K tile: the time line of the pipelined loop
  constexpr bool PIPE_OK = MT >= 4;
  constexpr int BAR = (SPW - 1) * NM + NM / 2;                 // group in front of which the barrier stands
  constexpr int WEND = cmax(1, cmin(BAR, (MT * 3) / 8));       // LDS writes occupy groups [0, WEND)
  constexpr int LEND = cmin(MT, cmax(WEND + 1, (MT * 3) / 4)); // global loads occupy groups [WEND, LEND)
  constexpr int FSPAN = cmax(1, (NM * 3) / 4);                 // next-step fragment reads: first 3/4 of a step
  constexpr int NSPAN = cmax(1, ((MT - BAR) * 3) / 4);         // next-tile fragment reads: behind the barrier

  // ---- K loop ---------------------------------------------------------------------------------
  // SHARED_PREFETCH=1: two LDS stages, one barrier per K tile.  Registers carry tile kt+1 (fetched from
  // global memory during tile kt-1); it is written to the idle stage at the start of tile kt, under
  // the matrix-core work of that tile, and the fetch of tile kt+2 is issued right after.
  // REG_PREFETCH=1 additionally keeps fragments one step ahead: the barrier sits before the last
  // step's matrix-core work, and the first fragments of the next tile are read behind it, so their
  // LDS latency is covered by that work.
  if constexpr (C::SHMP) {
    load_global(0);
    store_lds(0);
    if (KT > 1) load_global(1);
    __syncthreads();
    if constexpr (C::REGP && PIPE_OK) {
      // Software pipeline: the tile's MT = SPW*NM matrix-core groups are the time line; LDS writes of
      // tile kt+1 go under the first groups, the global fetch of tile kt+2 under the following ones,
      // fragment reads of step s+1 under step s; the barrier stands in the middle of the last step
      // and the first fragments of tile kt+1 are read right behind it.  sched_barrier pins that order.
      Frag fa[2][TMI], fb[2][TNI];
      load_frag(0, wz, fa[0], fb[0]);
      auto tile = [&](int kt, auto has1, auto has2) {
        constexpr bool H1 = decltype(has1)::value, H2 = decltype(has2)::value;
        const int cur = kt & 1;
        // the step number is a compile-time constant (static_for, not a loop the compiler may decline to
        // unroll): it selects the half of the fragment double buffer
        static_for<0, SPW>([&](auto s_c) {
          constexpr int s = decltype(s_c)::value;
#pragma unroll
          for (int q = 0; q < NM; ++q) {
            const int slot = s * NM + q;
            if (slot == BAR) __syncthreads();
            MI::run(acc[q / TNI][q % TNI], fa[s & 1][q / TNI], fb[s & 1][q % TNI]);
            if constexpr (H1) {
#pragma unroll
              for (int i = 0; i < NWR; ++i)
                if ((i * WEND) / NWR == slot) write_item(i, cur ^ 1);
            }
            if constexpr (H2) {
#pragma unroll
              for (int i = 0; i < NLD; ++i)
                if (WEND + (i * (LEND - WEND)) / NLD == slot) load_item(i, (kt + 2) * BK);
            }
#pragma unroll
            for (int f = 0; f < NF; ++f) {
              if (s + 1 < SPW && (f * FSPAN) / NF == q)
                load_frag_item(cur, (s + 1) * LSU + wz, f, fa[(s + 1) & 1], fb[(s + 1) & 1]);
              if (H1 && BAR + (f * NSPAN) / NF == slot) load_frag_item(cur ^ 1, wz, f, fa[SPW & 1], fb[SPW & 1]);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        });
        if constexpr (SPW % 2 == 1) {   // odd step count: the prefetched fragments sit in slot 1
#pragma unroll
          for (int i = 0; i < TMI; ++i) fa[0][i] = fa[1][i];
#pragma unroll
          for (int j = 0; j < TNI; ++j) fb[0][j] = fb[1][j];
        }
      };
      for (int kt = 0; kt + 2 < KT; ++kt) tile(kt, BoolC<true>(), BoolC<true>());
      if (KT >= 2) tile(KT - 2, BoolC<true>(), BoolC<false>());
      tile(KT - 1, BoolC<false>(), BoolC<false>());
    } else {
      for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) store_lds(cur ^ 1);
        if (kt + 2 < KT) load_global(kt + 2);
        Frag fa[TMI], fb[TNI];
#pragma unroll
        for (int s = 0; s < SPW; ++s) {
          load_frag(cur, s * LSU + wz, fa, fb);
          mma_frag(fa, fb);
        }
        __syncthreads();
      }
    }
  } else {
    // single LDS stage (the reference's unpipelined order, Optimizer.cc:343-376)
    for (int kt = 0; kt < KT; ++kt) {
      load_global(kt);
      __syncthreads();
      store_lds(0);
      __syncthreads();
      if constexpr (C::REGP) {
        Frag fa[2][TMI], fb[2][TNI];
        load_frag(0, wz, fa[0], fb[0]);
        static_for<0, SPW>([&](auto s_c) {
          constexpr int s = decltype(s_c)::value;
          if constexpr (s + 1 < SPW) load_frag(0, (s + 1) * LSU + wz, fa[(s + 1) & 1], fb[(s + 1) & 1]);
          mma_frag(fa[s & 1], fb[s & 1]);
        });
      } else {
        Frag fa[TMI], fb[TNI];
#pragma unroll
        for (int s = 0; s < SPW; ++s) {
          load_frag(0, s * LSU + wz, fa, fb);
          mma_frag(fa, fb);
        }
      }
    }
  }

  // ---- epilogue -------------------------------------------------------------------------------
  // Accumulator layout of a 32x32 tile: lane holds column lane%32, rows 8*(e/4) + 4*(lane/32) + e%4
  // for e in 0..15; of a 16x16 tile: column lane%16, rows 4*(lane/16) + e for e in 0..3; of the fp64
  // 16x16 tile: column lane%16, rows lane/16 + 4*e (established on hardware; the parity tests pin it).
  constexpr int NACC = (int)(sizeof(Acc) / sizeof(AccT));
  const int ocol = lane % MF;
  const int orow = (lane / MF) * 4;
  auto acc_row = [&](int e) { return ES == 8 ? lane / MF + 4 * e : (e / 4) * 8 + orow + e % 4; };
  if constexpr (LSU > 1) {
    AccT* smC = reinterpret_cast<AccT*>(smem);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TMI; ++i)
#pragma unroll
      for (int j = 0; j < TNI; ++j)
#pragma unroll
        for (int e = 0; e < NACC; ++e) {
          const int row = wy * WM + i * MF + acc_row(e);
          const int col = wx * WN + j * MF + ocol;
          smC[(wz * BM + row) * BN + col] = acc[i][j][e];
        }
    __syncthreads();
    splitu_reduce_store<C, NT>(Cm, smC, tid, m0, n0, ep);
  } else {
#pragma unroll
    for (int i = 0; i < TMI; ++i)
#pragma unroll
      for (int j = 0; j < TNI; ++j)
#pragma unroll
        for (int e = 0; e < NACC; ++e) {
          const int row = m0 + wy * WM + i * MF + acc_row(e);
          const int col = n0 + wx * WN + j * MF + ocol;
          if (!EDGE || (row < M && col < N)) {
            AccT v = acc[i][j][e];
            if constexpr (C::EPI) epi_apply<TC, AccT, 1, false, true>(&v, Cm, row, col, N, M, N, ep);
            Cm[(long)row * N + col] = (TC)v;
          }
        }
  }
}

}  // namespace kcg
