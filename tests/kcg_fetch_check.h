// kcg_fetch_check.h — host-side walk through the fetch map of the direct-staging kernel (FetchMap in
// kcg_device_direct.h) for ONE instantiation: append this file to an instantiation stub (kcg_instantiation_source),
// compile for the host and run.  For every block, K tile, wave, fetch instruction and lane it checks that
//   * the 16 bytes fetched lie inside the operand's buffer (the kernel must never touch memory beyond A and B:
//     what follows a buffer may be another page), and
//   * every element of the tile that exists (row < M, column < N, k < K) ends up at the LDS position where the
//     fragment reads look for it (LdsTile::slot for the k-contiguous operand, chunk ^ swz_n(row) for the
//     row-contiguous ones), counting the shift that patch_final applies to a chunk fetched from further down.
// Needs no GPU.  Prints one line and returns 0 when all is well.
#pragma once
#include <cstdio>

// DirectPlan::AG: the wait counts of VmSchedule against an explicit list of the operations in the order the K loop issues
// them (prologue: the B fetches of the first tiles, then the A loads of the first steps; per slot of a tile: the B fetches whose
// position is that slot; behind a row's last slot: the A load of that row two steps on).  A wait for operation X with count n is
// right if at most n operations were issued after X at that point; it is tight if exactly n were (or 63, the counter's limit).
template <class P, class F>
int check_vm_schedule() {
  constexpr int SPW = P::SPW, TMI = P::WM / P::MF, TNI = P::WN / P::MF, NM = TMI * TNI, MT = SPW * NM;
  constexpr int NST = P::NST, NIB = F::NIB, KTT = F::KTT, D = P::AG_DEPTH, STEPS = KTT * SPW;
  constexpr int RB = 1, BAR = (SPW - 1) * NM + RB * TNI, SPREAD = NST >= 3 ? MT : MT - BAR;   // as in the kernel (A_AHEAD at its default)
  typedef kcg::VmSchedule<KTT, SPW, TMI, TNI, NIB, NST, BAR, SPREAD, D> VS;
  struct Op { int is_a, x, y; };                         // A load of (step x, row y) or B fetch of (tile x, item y)
  static Op ops[1 << 20];
  int n = 0;
  auto last_of = [&](int is_a, int x, int y) {           // index of that operation, -1 if it was never issued
    for (int k = n - 1; k >= 0; --k)
      if (ops[k].is_a == is_a && ops[k].x == x && (y < 0 || ops[k].y == y)) return k;
    return -1;
  };
  auto bad = [](const char* what, int t, int s, int i, int have, int allowed) {
    printf("FAILED: vm schedule: %s (tile %d, step %d, row %d): waits with %d, %d operations were issued behind it\n", what, t, s, i, have, allowed);
    return 1;
  };
  long loose = 0;
  const int npro = NST < KTT ? NST : KTT;
  for (int t = 0; t < npro; ++t)
    for (int f = 0; f < NIB; ++f) ops[n++] = Op{0, t, f};
  for (int gs = 0; gs < (D < STEPS ? D : STEPS); ++gs)
    for (int i = 0; i < TMI; ++i) ops[n++] = Op{1, gs, i};
  {
    const int allowed = n - 1 - last_of(0, 0, -1);
    if (VS::wait_pro() > allowed) return bad("B tile 0 at the end of the prologue", 0, 0, 0, VS::wait_pro(), allowed);
  }
  for (int t = 0; t < KTT; ++t)
    for (int s = 0; s < SPW; ++s)
      for (int i = 0; i < TMI; ++i) {
        const int ia = last_of(1, t * SPW + s, i);
        if (ia < 0) return bad("an A fragment that was never loaded", t, s, i, 0, 0);
        const int allowed_a = n - 1 - ia < 63 ? n - 1 - ia : 63;
        if (VS::wait_a(t, s, i) > allowed_a) return bad("A fragment", t, s, i, VS::wait_a(t, s, i), allowed_a);
        loose += allowed_a - VS::wait_a(t, s, i);
        if (s == SPW - 1 && i == RB && t + 1 < KTT) {
          int ib = -1;
          for (int f = 0; f < NIB; ++f) {
            const int k = last_of(0, t + 1, f);
            if (k < 0) return bad("a B fetch of the next tile that was never issued", t, s, f, 0, 0);
            ib = k > ib ? k : ib;
          }
          const int allowed_b = n - 1 - ib < 63 ? n - 1 - ib : 63;
          if (VS::wait_b(t) > allowed_b) return bad("B tile at the barrier", t, s, i, VS::wait_b(t), allowed_b);
          if (allowed_b - VS::wait_b(t) > NIB) return bad("B tile at the barrier waits for far more than it needs", t, s, i, VS::wait_b(t), allowed_b);
        }
        for (int j = 0; j < TNI; ++j) {
          const int q = s * NM + i * TNI + j;
          for (int f = 0; f < NIB; ++f) {
            const int pos = BAR + (f * SPREAD) / NIB;
            if (t + NST < KTT && pos == q) ops[n++] = Op{0, t + NST, f};
            if (t >= 1 && t - 1 + NST < KTT && SPREAD > MT - BAR && pos - MT == q) ops[n++] = Op{0, t - 1 + NST, f};
          }
        }
        if (t * SPW + s + D < STEPS) ops[n++] = Op{1, t * SPW + s + D, i};
        if (n > (1 << 20) - 64) return bad("too many operations for this check", t, s, i, n, 0);
      }
  if (loose != 0) return bad("A waits are not tight: summed slack", 0, 0, 0, (int)loose, 0);
  return 0;
}

// The counted waits for fragment reads (s_waitcnt lgkmcnt(n), n = StreamPlan::allowed(row)) against an explicit list of
// the LDS read instructions in the order the K loop issues them: prologue (the B fragments of step 0, the first DA A
// fragments, then a full wait); at the start of row i of a step the A fragment DA rows on (of this step, the next step or
// the next tile's first step), behind the matrix instruction of slot slot_b(j) the B fragment j of the next step.  LDS
// reads return in order: a wait with count n covers read X if at least n reads were issued after X.
template <class P, class F>
int check_lds_schedule() {
  constexpr int ES = P::ES, TMI = P::WM / P::MF, TNI = P::WN / P::MF, DA = TMI - 1;
  constexpr int RC = ES == 2 ? 2 : 4, NAI = P::AG ? 0 : (F::AK ? 1 : RC), NBI = RC;
  typedef kcg::StreamPlan<TMI, TNI, DA, NAI, NBI> SP;
  constexpr int KT = F::KT, KTT = F::KTT, SPW = P::SPW, SPWT = (F::KR + P::KS - 1) / P::KS;
  static int last_read[2][64][2];                       // [operand][fragment][step parity] -> index of its last read instruction
  int n = 0;                                            // read instructions issued so far
  auto issue = [&](int is_b, int frag, int gstep, int count) {
    n += count;
    last_read[is_b][frag][gstep & 1] = n - 1;
  };
  auto bad = [](const char* what, int t, int s, int i, int have, int behind) {
    printf("FAILED: lds schedule: %s (tile %d, step %d, row %d): waits with %d, %d reads were issued behind it\n", what, t, s, i, have, behind);
    return 1;
  };
  for (int j = 0; j < TNI; ++j) issue(1, j, 0, NBI);
  for (int i = 0; i < DA; ++i) issue(0, i, 0, NAI);
  int complete = n;                                     // a full wait: everything issued so far has arrived
  int gstep = 0;
  for (int t = 0; t < KTT; ++t) {
    const int ns = t < KT ? SPW : SPWT;
    const bool h1 = t + 1 < KTT;
    for (int s = 0; s < ns; ++s, ++gstep) {
      const bool last = s == ns - 1, next = !last || h1;
      for (int i = 0; i < TMI; ++i) {
        // the wait at the start of the row
        if (next) {
          const int have = SP::allowed(i);
          if (NAI > 0) {
            const int x = last_read[0][i][gstep & 1];
            if (x >= complete && n - 1 - x < have) return bad("A fragment", t, s, i, have, n - 1 - x);
          }
          if (i == 0)
            for (int j = 0; j < TNI; ++j) {
              const int x = last_read[1][j][gstep & 1];
              if (x >= complete && n - 1 - x < have) return bad("B fragment", t, s, j, have, n - 1 - x);
            }
          if (n - have > complete) complete = n - have;
        } else {
          complete = n;
        }
        if (last && i == SP::RB) complete = n;           // the full wait in front of the barrier
        // the A fragment DA rows on
        if (NAI > 0) {
          if (i + DA < TMI) issue(0, i + DA, gstep, NAI);
          else if (!last || h1) issue(0, i + DA - TMI, gstep + 1, NAI);
        }
        for (int j = 0; j < TNI; ++j)
          for (int jj = 0; jj < TNI; ++jj)
            if (SP::slot_b(jj) == i * TNI + j && (!last || h1)) issue(1, jj, gstep + 1, NBI);
      }
    }
  }
  return 0;
}

// The same for the global->LDS fetches of the ordinary build (both operands through LDS): at the barrier of tile t
// the kernel waits with vmcnt(tiles_ahead(t) * NFETCH) for tile t+1 to have landed; every fetch of tile t+1 must have at
// least that many fetches issued behind it (prologue: the first NST tiles, item by item; tile t: the items of tile t+NST
// whose position is a slot of this tile, and those of tile t-1+NST whose position lies a period further on).
template <class P, class F>
int check_fetch_schedule() {
  constexpr int SPW = P::SPW, TMI = P::WM / P::MF, TNI = P::WN / P::MF, NM = TMI * TNI, MT = SPW * NM;
  constexpr int NST = P::NST, NFETCH = P::NFETCH, KTT = F::KTT;
  constexpr int RB = 1, BAR = (SPW - 1) * NM + RB * TNI, SPREAD = NST >= 3 ? MT : MT - BAR;
  static int last_of_tile[1 << 16];
  if (KTT >= (1 << 16)) return 0;
  int n = 0;
  for (int t = 0; t < KTT; ++t) last_of_tile[t] = -1;
  const int npro = NST < KTT ? NST : KTT;
  for (int t = 0; t < npro; ++t) { n += NFETCH; last_of_tile[t] = n - 1; }
  if (n - 1 - last_of_tile[0] < (npro - 1) * NFETCH && (npro - 1) * NFETCH <= 63) {
    printf("FAILED: fetch schedule: the prologue's wait for tile 0 allows %d fetches in flight, %d were issued behind it\n", (npro - 1) * NFETCH, n - 1 - last_of_tile[0]);
    return 1;
  }
  for (int t = 0; t < KTT; ++t) {
    // slots in front of the barrier, the barrier's wait, then the rest (a partial last tile has fewer slots, but
    // issues no fetches: nothing is left to fetch)
    for (int q = 0; q < MT; ++q) {
      if (q == BAR && t + 1 < KTT) {
        const int newest = KTT - 1 < (t == 0 ? NST - 1 : t - 1 + NST) ? KTT - 1 : (t == 0 ? NST - 1 : t - 1 + NST);
        const int ahead = newest - (t + 1) > 0 ? newest - (t + 1) : 0;
        if (last_of_tile[t + 1] < 0 || n - 1 - last_of_tile[t + 1] < ahead * NFETCH) {
          printf("FAILED: fetch schedule: the barrier of tile %d waits with %d, %d fetches were issued behind tile %d\n", t, ahead * NFETCH,
                 last_of_tile[t + 1] < 0 ? -1 : n - 1 - last_of_tile[t + 1], t + 1);
          return 1;
        }
      }
      for (int f = 0; f < NFETCH; ++f) {
        const int pos = BAR + (f * SPREAD) / NFETCH;
        if (t + NST < KTT && pos == q) { ++n; last_of_tile[t + NST] = n - 1; }
        if (t >= 1 && t - 1 + NST < KTT && SPREAD > MT - BAR && pos - MT == q) { ++n; last_of_tile[t - 1 + NST] = n - 1; }
      }
    }
  }
  return 0;
}

int main() {
  typedef kcg::DirectPlan<Cfg> P;
  typedef kcg::FetchMap<Cfg> F;
  if (!P::OK) {
    printf("not a direct-staging instantiation\n");
    return 2;
  }
  if constexpr (P::AG) {
    if (check_vm_schedule<P, F>()) return 1;
  }
  if (check_lds_schedule<P, F>()) return 1;
  if constexpr (!P::AG) {
    if (check_fetch_schedule<P, F>()) return 1;
  }
  constexpr int M = F::M, N = F::N, K = F::K, BM = F::BM, BN = F::BN, BK = F::BK, G = F::G, ES = F::ES, NW = F::NW;
  const long a_bytes = (long)M * K * ES, b_bytes = (long)K * N * ES;
  const int gy = (M + BM - 1) / BM, gx = (N + BN - 1) / BN;
  long chunks = 0, moved = 0, misaligned = 0;
  // where the chunk in physical slot `phys` of an operand's stage comes from, after the shift of a moved chunk:
  // the element index (in the operand's buffer) that LDS position i of the chunk holds is first + i for i < count
  struct Got {
    long first;
    int count;
  };
  auto fail = [](const char* what, int by, int bx, int kt, int phys, long v) {
    printf("FAILED: %s (block row %d, block column %d, K tile %d, chunk slot %d, value %ld)\n", what, by, bx, kt, phys, v);
    return 1;
  };
  for (int by = 0; by < gy; ++by)
    for (int bx = 0; bx < gx; ++bx) {
      const int m0 = by * BM, n0 = bx * BN;
      for (int kt = 0; kt < F::KTT; ++kt) {
        const bool last = F::FINAL_SPECIAL && kt == F::KTF;
        const int kvalid = last ? F::KLAST : BK;
        auto fetched = [&](bool is_a, int phys, Got* g) -> int {
          const int ni = is_a ? F::NIA : F::NIB;
          const int wave = phys / (64 * ni), idx = (phys / 64) % ni, lane = phys % 64;
          if (wave >= NW) return fail("chunk slot beyond the stage", by, bx, kt, phys, wave);
          const typename F::Src s = is_a ? F::a(wave, lane, idx, m0, kvalid, last) : F::b(wave, lane, idx, n0, kvalid, last);
          const long addr = (is_a ? F::a_tile(m0, kt) : F::b_tile(n0, kt)) + (long)s.off;
          const long size = is_a ? a_bytes : b_bytes;
          if (addr < 0 || addr + 16 > size) return fail(is_a ? "fetch outside A" : "fetch outside B", by, bx, kt, phys, addr);
          if (addr % ES) return fail("fetch address not on an element boundary", by, bx, kt, phys, addr);
          const int sh = s.moved ? (is_a ? P::SH_A : P::SH_B) : 0;
          g->first = addr / ES + sh;
          g->count = G - sh;
          ++chunks;
          moved += s.moved;
          misaligned += (addr % 4) != 0;
          return 0;
        };
        // A, read straight from global memory into fragment registers (DirectPlan::AG): every load of every lane
        // stays inside A, and a lane whose row exists gets the 16 bytes of its row and k values
        if constexpr (P::AG) {
          for (int wy = 0; wy < Cfg::BLM; ++wy) {
            const int row0 = F::ag_row0(wy, m0);
            if (row0 < 0 || m0 + row0 >= M) return fail("AG: the wave's first row does not exist", by, bx, kt, wy, row0);
            for (int st = 0; st < P::SPW; ++st)
              for (int i = 0; i < P::WM / P::MF; ++i)
                for (int lane = 0; lane < 64; ++lane) {
                  const unsigned off = F::ag_lane(i, lane, m0, row0);
                  const long addr = F::a_tile(m0, kt) + (long)row0 * K * ES + (long)(unsigned long)off + (long)st * P::KS * ES;
                  if (addr < 0 || addr + 16 > a_bytes) return fail("AG load outside A", by, bx, kt, lane, addr);
                  const int row = m0 + wy * P::WM + i * P::MF + lane % P::MF, kk = kt * BK + st * P::KS + G * (lane / P::MF);
                  if (row < M && addr != ((long)row * K + kk) * ES) return fail("AG load is not the lane's fragment", by, bx, kt, lane, addr);
                  ++chunks;
                }
          }
        }
        // A
        for (int r = 0; r < (P::AG ? 0 : F::AK ? BM : BK); ++r)
          for (int c = 0; c < (F::AK ? F::CHK : F::NCHA); ++c) {
            const int phys = F::AK ? F::LK::slot(r, c) : r * F::NCHA + (c ^ F::swz_n(r, F::NCHA));
            Got g;
            if (fetched(true, phys, &g)) return 1;
            for (int i = 0; i < G; ++i) {
              const int row = F::AK ? m0 + r : m0 + c * G + i;            // m
              const int kk = F::AK ? kt * BK + c * G + i : kt * BK + r;   // k
              if (row >= M || row >= m0 + BM || kk >= K) continue;
              const long want = F::AK ? (long)row * K + kk : (long)kk * M + row;
              if (i >= g.count || g.first + i != want) return fail("A element not where the fragment reads look for it", by, bx, kt, phys, want);
            }
          }
        // B
        for (int r = 0; r < BK; ++r)
          for (int c = 0; c < F::NCHB; ++c) {
            const int phys = r * F::NCHB + (c ^ F::swz_n(r, F::NCHB));
            Got g;
            if (fetched(false, phys, &g)) return 1;
            for (int i = 0; i < G; ++i) {
              const int col = n0 + c * G + i, kk = kt * BK + r;
              if (col >= N || kk >= K) continue;
              const long want = (long)kk * N + col;
              if (i >= g.count || g.first + i != want) return fail("B element not where the fragment reads look for it", by, bx, kt, phys, want);
            }
          }
      }
    }
  printf("ok: %ld chunks, %ld fetched from further down, %ld from addresses off a 4-byte boundary\n", chunks, moved, misaligned);
  return 0;
}
