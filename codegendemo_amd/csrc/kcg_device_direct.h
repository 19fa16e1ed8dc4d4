// kcg_device_direct.h — kernel family 2b: matrix-core kernel with direct global->LDS staging and a
// row-streaming, hand-scheduled K loop (fp32, fp16, bf16 inputs).
#pragma once
#include "kcg_device_common.h"
#include "kcg_device_mfma_ops.h"

namespace kcg {

// Every lambda of this file is inlined by attribute.  The K loop is a forest of small generic lambdas (static_for
// bodies, one instantiation per tile, k-step, row and slot: thousands of functions); left to the optimiser's inliner
// they are inlined just the same, but only after argument promotion, attribute inference and the inliner's cost model
// have looked at each of them, which took most of the compile time of the large tiles.
#define KCG_INL __attribute__((always_inline))

// ---------------------------------------------------------------------------------------------
// In-kernel time line (diagnostic build, -DKCG_TIMELINE=1 or 2 through $KCG_EXTRA_FLAGS; 0 = off, no
// code).  Every wave of gemm_mfma_direct then writes one record of KCG_TL_WORDS 64-bit words to the buffer
// whose address the host has stored in the module's global `kcg_timeline_ptr` (hipModuleGetGlobal),
// record index = block * waves + wave:
//   [0] block start  [1] first K tile has landed  [2] K loop done  [3] C stores issued
//   [4] C stores acknowledged                    (constant 100 MHz clock, 10 ns units)
//   [5] shader-clock cycles spent in the K loop
//   [6] HW_ID (low half) and XCC_ID (high half) registers: which compute unit / XCD the wave ran on
//   [7] level 2 only: shader-clock cycles this wave spent between asking for and passing the K-loop
//       barriers (wait for its own fetches + LDS reads + the other waves); costs one extra scalar-memory
//       round trip per K tile, so the times of level 2 are a little longer than those of level 1
// kcg_runner --timeline builds such a kernel, runs it and prints the per-phase budget.
// ---------------------------------------------------------------------------------------------
#ifndef KCG_TIMELINE
#define KCG_TIMELINE 0
#endif
// Diagnostic builds only (never set by the library itself; C is then WRONG): the K loop of the direct-staging
// kernel without its global->LDS fetches (the stages keep the first tiles, which the prologue still fetches)
// resp. without its fragment reads (the matrix-core instructions keep running on the first fragments; 1: no fragment
// reads at all, 2: none of A, 3: none of B).  Timing such builds shows what each part of the data movement costs a launch.
#ifndef KCG_DIAG_NO_FETCH
#define KCG_DIAG_NO_FETCH 0
#endif
#ifndef KCG_DIAG_NO_LDS_READS
#define KCG_DIAG_NO_LDS_READS 0
#endif
// ... and with every fetch reading K tile 0 again (the fetches stay, but all of them hit in L2: what remains
// of their cost is the path from L2 into LDS, what disappears is the traffic between L2 and memory)
#ifndef KCG_DIAG_FETCH_TILE0
#define KCG_DIAG_FETCH_TILE0 0
#endif
// -DKCG_DIAG_EVEN_XCD_SLEEP=n (C stays correct): the blocks on even-numbered XCDs sleep n * 64 cycles in front of every
// K-tile barrier.  On a power-limited kernel the odd-numbered XCDs then run faster by about what the even ones lose:
// the XCDs share one power budget.
// Cache-policy bits of the global->LDS fetch instructions (bit 0: sc0, bit 1: nt, bit 4: sc1).  A block reads
// every operand byte exactly once, so nothing is gained by keeping the lines in the compute unit's vector cache.
#ifndef KCG_FETCH_AUX
#define KCG_FETCH_AUX 0
#endif
// 1: the direct-staging kernel writes C with non-temporal stores (C is written once and not read again by
// the kernel: the stores need not displace operand panels from L2)
#ifndef KCG_C_NT
#define KCG_C_NT 0
#endif
#if KCG_TIMELINE
#define KCG_TL_WORDS 8
extern "C" {
__device__ unsigned long long* kcg_timeline_ptr = nullptr;
}
__device__ __forceinline__ unsigned long long tl_realtime() {
  unsigned long long t;
  asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t)::"memory");
  return t;
}
__device__ __forceinline__ unsigned long long tl_cycles() {
  unsigned long long t;
  asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t)::"memory");
  return t;
}
#endif

// =============================================================================================
// Family 2b: matrix-core kernel with direct global->LDS staging.
//
// Every lane fetches one 16-byte chunk (G = 4 fp32 or 8 fp16/bf16 elements) with
// global_load_lds_dwordx4; a wave's 64 chunks land in 1 KiB of consecutive LDS, so no register, no
// ds_write and no vector ALU work is spent on staging, and with NST stages the fetch of a tile can be in
// flight for NST-1 K tiles.  The source address of a chunk need not be 16-byte aligned: where M, N or K is
// not a multiple of G the rows of A and B start anywhere (fp32: on 4-byte boundaries, fetched at the full
// rate; 16-bit rows of odd length: every other one 2 bytes off, fetched at about 40 % of it), and the chunk
// at the end of a row brings the first elements of the next row with it, which land in columns (or k values)
// that do not exist and are never used.  The LDS image keeps the orientation of global memory:
//   k-contiguous operand  (A, IS_ATRANS=0): rows = m, CH = BK/G chunks of G k values each; a fragment
//                                           is one ds_read_b128 (as in gemm_mfma)
//   row-contiguous operand (B; A^T)       : rows = k, NCH = BN/G (BM/G) chunks of G n values each.
//       16-bit: a fragment is two ds_read_b64_tr_b16: 16 lanes read a 4(k) x 16(n) block and each lane
//               receives one column of it, which is the k-packed layout the matrix core wants
//       32-bit: a fragment is four ds_read_b32, one per k value
// Edge tiles cost the K loop nothing: a lane whose chunk lies outside the matrix (rows or columns
// beyond M or N; k beyond K in the last, partial K tile) fetches a chunk of the same tile that does exist
// instead.  What lands in LDS for it only ever reaches accumulators of rows/columns that are not stored
// (M, N) or is not read at all (the partial K tile computes only the k-steps it has; where its last
// k-step is itself partial, the lanes that hold k values beyond K clear their fragments before use).
// The bank swizzle is applied on the fetch side: the lane that fills physical chunk c' of a row fetches
// logical chunk c' ^ swz(row), and readers look chunk c up at c ^ swz(row).
// =============================================================================================

// Static schedule of the fragment reads of one k-step of the direct-staging kernel (see its K loop):
// which slot reads which B fragment of the next step, and how many LDS read instructions issued after
// the fragments a row needs may still be in flight when that row starts.
template <int TMI, int TNI, int DA, int NAI, int NBI>
struct StreamPlan {
  static constexpr int NM = TMI * TNI;
  static constexpr int RB = TMI - DA;                              // first row whose side work belongs to the next step
  static constexpr int BW0 = RB * TNI;                             // B reads: slots [BW0, BW1)
  static constexpr int BW1 = DA > 1 ? (TMI - 1) * TNI : NM;
  static constexpr int slot_b(int j) { return BW0 + (j * (BW1 - BW0)) / TNI; }
  // (non-decreasing in j: the B fragments read behind slot q of a step are the range [first_b(q), first_b(q + 1)))
  static constexpr int first_b(int q) {
    int j = 0;
    while (j < TNI && slot_b(j) < q) ++j;
    return j;
  }
  // issue times in half slots: a row's A read comes first in its slot, a B read follows the
  // matrix-core instruction of its slot
  static constexpr int time_a(int step, int row) { return (step * NM + (row - DA) * TNI) * 2; }
  static constexpr int time_b(int step, int j) { return ((step - 1) * NM + slot_b(j)) * 2 + 1; }
  static constexpr int allowed(int row) {
    const int step = 2;
    const int now = (step * NM + row * TNI) * 2 - 1;               // just before this row's own A read
    int need = time_a(step, row);
    if (row == 0)
      for (int j = 0; j < TNI; ++j) need = cmax(need, time_b(step, j));
    int n = 0;
    for (int st = 0; st <= step + 1; ++st) {
      for (int r = 0; r < TMI; ++r) {
        const int t = time_a(st, r);
        if (t > need && t < now) n += NAI;
      }
      for (int j = 0; j < TNI; ++j) {
        const int t = time_b(st, j);
        if (t > need && t < now) n += NBI;
      }
    }
    return cmin(n, 15);                                            // the counter field has 4 bits; less is safe
  }
};

// Where on the time line of the K loop the NFETCH fetch instructions of a K tile are issued: item f behind the
// matrix-core instruction of slot pos(f), counted from the start of the tile that begins the fetch (a position of MT or
// more lies in the next tile).  pos is non-decreasing in f: the items of a slot are the range [lo(q), lo(q + 1)).
template <int NFETCH, int NIA, int BAR, int SPREAD>
struct FetchSlots {
  static constexpr int pos(int f) { return BAR + (f * SPREAD) / NFETCH; }
  static constexpr int lo(int q) {                                  // the first item whose position is q or later
    int f = 0;
    while (f < NFETCH && pos(f) < q) ++f;
    return f;
  }
  // (diagnostic builds: 1 drops every fetch of the K loop, 2 those of A only, 3 those of B only)
  static constexpr bool on(int f) {
    return KCG_DIAG_NO_FETCH == 0 || (KCG_DIAG_NO_FETCH == 2 && f >= NIA) || (KCG_DIAG_NO_FETCH == 3 && f < NIA);
  }
};

template <class C>
struct DirectPlan {
  typedef typename C::TA T;
  static constexpr int ES = (int)sizeof(T);
  static constexpr int WM = C::BM / C::BLM, WN = C::BN / C::BLN;
  // 16x16x32 instructions where the K tile allows: on fp16/bf16 data with realistic bit activity a
  // gfx950 sustains about 16 % more flops with them than with 32x32x16 at its power limit
#ifndef KCG_DIRECT_MF
#define KCG_DIRECT_MF 0               /* 16 or 32 forces the matrix-core tile of the direct-staging kernel */
#endif
  static constexpr int G = 16 / ES;                               // elements per 16-byte chunk
  // (the streaming K loop wants two rows of matrix-core tiles per wave: a 32-row wave tile takes 16x16 tiles)
  static constexpr bool FITS32 = WM % 32 == 0 && WN % 32 == 0 && WM / 32 >= 2;
  static constexpr int MF = KCG_DIRECT_MF ? KCG_DIRECT_MF
                            : ES == 2 ? ((C::BK % 32 == 0 || !FITS32) ? 16 : 32)
                                      : (FITS32 ? 32 : 16);       // fp32: no such difference, the larger tile reads less
  static constexpr int KS = G * (64 / MF);                        // k per step: one chunk per lane
  static constexpr int NW = C::BLM * C::BLN;
  static constexpr int NM = (WM / MF) * (WN / MF);
  static constexpr int SPW = (C::BK % KS == 0) ? C::BK / KS : 0;
  static constexpr bool pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }
  // block tile extents: a power of two, or a multiple of 16 chunks (the bank swizzle of a row-contiguous
  // tile exchanges chunks inside aligned groups of 16, so a row must consist of whole groups): 192, 320, ...
  static constexpr bool tile_ok(int x) { return pow2(x) || (x > 0 && x % (16 * G) == 0); }
  // The chunk at the end of the last row of a matrix whose rows are not whole chunks would reach up to 14 bytes
  // past the end of the buffer, which may be another page.  It is fetched from SH_x elements further down
  // instead (the last 16 bytes of the buffer), and the lane that fetched it moves the elements into place in LDS
  // (patch_final in the kernel).
  static constexpr int A_COLS = C::ATRANS ? C::M : C::K;          // row length of A as stored
  static constexpr int SH_A = (G - A_COLS % G) % G, SH_B = (G - C::N % G) % G;
  // A straight from global memory into the fragment registers (-DKCG_A_GLOBAL=1; "AG" below): a k-contiguous A
  // (IS_ATRANS=0) has the fragment layout of the matrix-core instructions in memory already - lane r + MF*g of a
  // fragment wants the 16 bytes A[row r][k0 + G*g ...] - so one global_load_dwordx4 per lane and fragment delivers
  // what the trip through LDS (a 1 KiB fetch into LDS + a ds_read_b128 per fragment) delivers, and the LDS that A
  // occupied goes to more B stages.  Every wave then loads its own rows of A (the waves of one block row load
  // the same ones).  Needs whole K tiles (no partial last tile: a fragment beyond K would read past a row).
#ifndef KCG_A_GLOBAL
#define KCG_A_GLOBAL 0
#endif
  static constexpr bool AG = KCG_A_GLOBAL != 0 && !C::ATRANS && C::K % C::BK == 0 && SPW > 0;
  static constexpr int AG_DEPTH = 2;                              // k-steps an A fragment is loaded ahead of its use
  static constexpr bool FIX_A = SH_A != 0 && !AG, FIX_B = SH_B != 0;
  static constexpr bool ELIGIBLE =
      (ES == 2 || (ES == 4 && sizeof(typename C::TC) == 4)) && C::SHMP && C::REGP && C::LC != 0 &&
      C::LSU == 1 && C::GLW_A == G && C::GLW_B == G &&
      // edge tiles in M and N are fine; K needs one full tile, and a row of A or B as stored at least one chunk (with
      // shorter rows several rows would share the chunk that reaches the end of the buffer)
      C::N >= G && A_COLS >= G &&
      SPW > 0 && C::K >= C::BK && WM / MF >= 2 && tile_ok(C::BM) && tile_ok(C::BN) && pow2(C::BK) && C::BM >= 32 && C::BN >= 32 &&
      (C::BM * C::BK / G) % (64 * NW) == 0 && (C::BN * C::BK / G) % (64 * NW) == 0 &&
      2 * (C::BM + C::BN) * C::BK * ES <= 160 * 1024 &&
      // fetch addresses are a scalar tile base + a 32-bit byte offset per lane
      (long)C::BM * C::K * ES < (1L << 31) && (long)C::BK * C::M * ES < (1L << 31) && (long)C::BK * C::N * ES < (1L << 31);
  // LDS stages: as many as fit in 160 KiB (or in half of it, see PAIR below), at most 4 (fetch distance =
  // NST-1 K tiles); an even number
  // when a tile is an odd number of k-steps (the B fragment double buffer alternates per step)
  static constexpr int A_STAGE_BYTES = AG ? 0 : C::BM * C::BK * ES;   // A's part of a stage (none when A bypasses LDS)
  static constexpr int STAGE_BYTES = A_STAGE_BYTES + C::BN * C::BK * ES;
  static constexpr int NST_FIT = (160 * 1024) / STAGE_BYTES;
  // and no more than the fetch counter can tell apart: the wait for tile kt+1 allows the fetches of
  // NST-2 younger tiles in flight (and, with AG, the A loads issued in that time), and that counter has 6 bits
  static constexpr int NFETCH = (((AG ? 0 : C::BM) + C::BN) * C::BK / G) / (64 * (NW > 0 ? NW : 1));   // per wave and tile
  static constexpr int VMOPS = NFETCH + (AG ? SPW * (WM / MF) : 0);                                    // ... all counted operations
  static constexpr int NST_VM = 2 + 63 / (VMOPS > 0 ? VMOPS : 1);
  static constexpr int NST_MAX = NST_FIT < NST_VM ? NST_FIT : NST_VM;
  // Two blocks on a compute unit beat one block with deeper staging when the launch has more blocks than the
  // chip has compute units (C::NUM_CU): one block's prologue, barrier waits and C stores run under the other's
  // matrix work (measured 2-5 % at 4096x1536x1000, 2048^3 and 4096^3 with 128x64 and 128x128 tiles).  Where
  // two blocks fit the register file (512 registers per lane and SIMD, a block's waves dealt evenly over
  // the four SIMDs: a wave holds WM*WN/64 accumulators and some 64 registers of fragments and addresses) the
  // stages are limited to half of the LDS.
#ifndef KCG_DIRECT_NST
#define KCG_DIRECT_NST 0              /* upper limit of the number of LDS stages; 0: the rule below */
#endif
  static constexpr int GRID_BLOCKS = ((C::M + C::BM - 1) / C::BM) * ((C::N + C::BN - 1) / C::BN);
  static constexpr bool PAIR = GRID_BLOCKS > C::NUM_CU && NW % 4 == 0 && (WM * WN / 64 + 64) * (NW / 2) <= 512 &&
                               2 * STAGE_BYTES <= 80 * 1024;
  static constexpr int NST_LIMIT = KCG_DIRECT_NST > 0 ? KCG_DIRECT_NST : (PAIR ? (80 * 1024) / STAGE_BYTES : 4);
  static constexpr int NST_TOP = NST_LIMIT > 4 ? 4 : NST_LIMIT;
  static constexpr int NST_CAP = NST_MAX < 2 ? 2 : (NST_MAX > NST_TOP ? NST_TOP : NST_MAX);
  static constexpr int NST = (SPW % 2 == 1 && NST_CAP % 2 == 1) ? NST_CAP - 1 : NST_CAP;
  // the host picks the path (it must size dynamic LDS accordingly): both sides have to agree on the
  // rule; the host may still decline an eligible config (a direct-staging build that would spill)
  static_assert(ELIGIBLE == C::DIRECT_ELIGIBLE, "host and device disagree on the direct-staging eligibility rule");
  static_assert(ELIGIBLE || !C::DIRECT, "direct staging asked for an ineligible config");
  static constexpr bool OK = C::DIRECT;
};

// Which 16 bytes of A and B the fetch instructions of a K tile bring to LDS: instruction idx of wave `wave` fills
// the 64 consecutive chunk slots 64*(wave*NI + idx) .. +63 of the operand's stage, one per lane.  Host-callable: a
// test walks every address of every tile of a problem through exactly this code.
template <class C>
struct FetchMap {
  typedef DirectPlan<C> P;
  static constexpr int ES = P::ES, G = P::G, NW = P::NW;
  static constexpr int BM = C::BM, BN = C::BN, BK = C::BK, M = C::M, N = C::N, K = C::K;
  static constexpr bool AK = !C::ATRANS;                          // A is k-contiguous in global memory
  static constexpr bool EDGE_M = M % BM != 0, EDGE_N = N % BN != 0;
  static constexpr int CHK = BK / G;                              // chunks per row of a k-contiguous tile
  static constexpr int NCHA = BM / G, NCHB = BN / G;              // chunks per row of a row-contiguous tile
  static constexpr int NIA = (BM * BK / G) / (64 * NW);           // fetch instructions per wave and tile, operand A
  static constexpr int NIB = (BN * BK / G) / (64 * NW);
  static constexpr int KT = K / BK;                               // full K tiles
  static constexpr int KR = K % BK;                               // the remainder: one more, partial tile
  static constexpr int KTT = KT + (KR > 0 ? 1 : 0);
  // The last tile computes its fetch offsets on the spot instead of taking the registers all other tiles share
  // when it is the partial one or holds a chunk that is fetched from another place (FIX_A / FIX_B).
  // KTF: tiles in front of it; KLAST: its k extent.
  static constexpr bool FINAL_SPECIAL = KR > 0 || P::FIX_A || P::FIX_B;
  static constexpr int KTF = FINAL_SPECIAL ? KTT - 1 : KTT;
  static constexpr int KLAST = KR > 0 ? KR : BK;
  typedef LdsTile<CHK> LK;
  // swizzle of a row-contiguous tile (chunk index ^= swz_n(row)).  16-bit: the rows that one pass of a
  // transposing read touches (k..k+3, and k+8..k+11 with 16-wide matrix-core tiles) must not share banks.
  // 32-bit: a fragment read is four 32-bit reads; in each, MF lanes read consecutive columns of one row
  // and the 64/MF lane groups read rows 4 apart, which must fall into different bank ranges.
  __host__ __device__ static constexpr int swz_n(int k, int nch) {
    const int mask = nch >= 16 ? 15 : nch - 1;          // nch: a power of two below 16, or a multiple of 16
    return (ES == 2 ? (((k & 3) << 2) ^ (((k >> 3) & 1) << 1)) : P::MF == 32 ? (((k >> 2) & 1) << 3) : (((k >> 2) & 3) << 2)) & mask;
  }
  // off: byte offset of the lane's chunk from the tile base.  moved: the chunk is the one at the end of the matrix and
  // is fetched from SH elements further down (last_tile says that the tile is the last one of the K loop); only
  // such a chunk can start in front of the tile base (off < 0).
  struct Src {
    int off;
    bool moved;
  };
  // kvalid: how many k rows / values of the tile exist (BK, or KR for the partial tile)
  __host__ __device__ static Src a(int wave, int lane, int idx, int m0, int kvalid, bool last_tile) {
    const int s = 64 * (wave * NIA + idx) + lane;       // physical chunk slot inside the A stage
    if constexpr (AK) {
      int row = s / CHK;
      const int cp = s % CHK;
      int k = (cp ^ ((row / LK::RDIV) % LK::SMOD)) * G;
      if constexpr (EDGE_M) row = cmin(row, M - 1 - m0);
      if (k >= kvalid) k = 0;
      const bool moved = P::FIX_A && last_tile && m0 + row == M - 1 && k + G > kvalid;
      return Src{(row * K + k - (moved ? P::SH_A : 0)) * ES, moved};
    } else {
      int k = s / NCHA;
      const int cp = s % NCHA;
      int m = (cp ^ swz_n(k, NCHA)) * G;
      if constexpr (EDGE_M) m = cmin(m, ((M - m0 - 1) / G) * G);   // the last chunk that starts inside the row
      if (k >= kvalid) k = 0;
      const bool moved = P::FIX_A && last_tile && k == kvalid - 1 && m0 + m + G > M;
      return Src{(k * M + m - (moved ? P::SH_A : 0)) * ES, moved};
    }
  }
  __host__ __device__ static Src b(int wave, int lane, int j, int n0, int kvalid, bool last_tile) {
    const int s = 64 * (wave * NIB + j) + lane;
    int k = s / NCHB;
    const int cp = s % NCHB;
    int n = (cp ^ swz_n(k, NCHB)) * G;
    if constexpr (EDGE_N) n = cmin(n, ((N - n0 - 1) / G) * G);
    if (k >= kvalid) k = 0;
    const bool moved = P::FIX_B && last_tile && k == kvalid - 1 && n0 + n + G > N;
    return Src{(k * N + n - (moved ? P::SH_B : 0)) * ES, moved};
  }
  // DirectPlan::AG: A fragments come straight from global memory.  The waves of wave row wy of the block at row m0
  // read from row ag_row0 of the block tile on (a wave whose rows all lie beyond M: from the last row that exists, so
  // that the lanes' offsets from there, unsigned 32-bit values, are never negative); for row block i of its fragments
  // a lane reads the 16 bytes at ag_lane from there (+ the k-step's KS elements): row i*MF + lane%MF (rows beyond M:
  // the last row; their results are not stored), k values G*(lane/MF) ...
  __host__ __device__ static int ag_row0(int wy, int m0) {
    int r = wy * P::WM;
    if constexpr (EDGE_M) r = cmin(r, M - 1 - m0);
    return r;
  }
  __host__ __device__ static unsigned ag_lane(int i, int lane, int m0, int row0) {
    int row = i * P::MF + lane % P::MF;
    if constexpr (EDGE_M) row = cmin(row, M - 1 - m0 - row0);
    return (unsigned)((row * K + G * (lane / P::MF)) * ES);
  }
  // byte offset of a block's tile kt from the start of A / B
  static constexpr long A_KT_BYTES = AK ? (long)BK * ES : (long)BK * M * ES;   // one K tile further
  static constexpr long B_KT_BYTES = (long)BK * N * ES;
  __host__ __device__ static constexpr long a_tile(int m0, int kt) { return (AK ? (long)m0 * K : (long)m0) * ES + kt * A_KT_BYTES; }
  __host__ __device__ static constexpr long b_tile(int n0, int kt) { return (long)n0 * ES + kt * B_KT_BYTES; }
};

// Order in which a wave of the direct-staging kernel issues the operations its vector-memory counter (vmcnt) counts
// when A bypasses LDS (DirectPlan::AG): the global->LDS fetches of B (NIB per K tile) and the A fragment loads (one per
// row of matrix-core tiles and k-step, issued D k-steps ahead).  The counter retires in order, so "operation X has
// completed" is "at most n operations issued after X are outstanding"; n is a property of this order, computed here at
// compile time for every place the K loop waits.  The K loop must issue in exactly this order:
//   prologue : B tiles 0..NPRO-1 | A steps 0..D-1
//   tile t, slot q (= matrix-core instruction (s, i, j), q = s*NM + i*TNI + j), after the instruction:
//              the B fetches whose position is q, ascending f (f of tile t+NST where pos(f) = q, f of tile t-1+NST
//              where pos(f) - MT = q), then, if j = TNI-1 and that step exists, the A load of (step t*SPW+s+D, row i)
template <int KTT, int SPW, int TMI, int TNI, int NIB, int NST, int BAR, int SPREAD, int D>
struct VmSchedule {
  static constexpr int NM = TMI * TNI, MT = SPW * NM, STEPS = KTT * SPW;
  static constexpr int NPRO = cmin(NST, KTT);
  static constexpr int PRO_A_STEPS = cmin(D, STEPS);
  static constexpr int PRO_OPS = NPRO * NIB + PRO_A_STEPS * TMI;
  static constexpr bool hn(int t) { return t + NST < KTT; }                              // tile t begins the fetch of tile t+NST
  static constexpr bool hp(int t) { return t >= 1 && t - 1 + NST < KTT && SPREAD > MT - BAR; }   // ... completes that of tile t-1+NST
  static constexpr int pos(int f) { return BAR + (f * SPREAD) / NIB; }                   // on the time line that starts at the issuing tile
  static constexpr bool a_issued(int t, int s) { return t * SPW + s + D < STEPS; }
  static constexpr int n_first() { int n = 0; for (int f = 0; f < NIB; ++f) n += pos(f) < MT ? 1 : 0; return n; }
  static constexpr int ops_in_tile(int t) {
    int n = (hn(t) ? n_first() : 0) + (hp(t) ? NIB - n_first() : 0);
    for (int s = 0; s < SPW; ++s) n += a_issued(t, s) ? TMI : 0;
    return n;
  }
  static constexpr int ops_in_slot(int t, int q) {
    int n = (q % TNI == TNI - 1 && a_issued(t, q / NM)) ? 1 : 0;
    for (int f = 0; f < NIB; ++f) n += ((hn(t) && pos(f) == q) ? 1 : 0) + ((hp(t) && pos(f) - MT == q) ? 1 : 0);
    return n;
  }
  // operations issued before the matrix-core instruction of slot q of tile t (q = MT: all of the tile)
  static constexpr int seq_at(int t, int q) {
    int n = PRO_OPS;
    for (int tt = 0; tt < t; ++tt) n += ops_in_tile(tt);
    for (int qq = 0; qq < q; ++qq) n += ops_in_slot(t, qq);
    return n;
  }
  // sequence number of the A load of (step gs, row i)
  static constexpr int seq_a(int gs, int i) {
    if (gs < D) return NPRO * NIB + gs * TMI + i;
    const int t = (gs - D) / SPW, s = (gs - D) % SPW;
    return seq_at(t, s * NM + i * TNI + TNI) - 1;                                        // the last operation of the row's last slot
  }
  // a sequence number by which every B fetch of tile u has been issued (the last operation of the slot of its last fetch)
  static constexpr int seq_b_done(int u) {
    if (u < NPRO) return (u + 1) * NIB - 1;
    const int p = pos(NIB - 1);
    return p < MT ? seq_at(u - NST, p + 1) - 1 : seq_at(u - NST + 1, p - MT + 1) - 1;
  }
  static constexpr int clamp(int n) { return n < 0 ? 0 : (n > 63 ? 63 : n); }
  // operations that may be outstanding when row i of step s of tile t starts (its A fragment has arrived) ...
  static constexpr int wait_a(int t, int s, int i) { return clamp(seq_at(t, s * NM + i * TNI) - 1 - seq_a(t * SPW + s, i)); }
  // ... and at the barrier of tile t (slot BAR of it has not been issued; tile t+1 has landed)
  static constexpr int wait_b(int t) { return clamp(seq_at(t, BAR) - 1 - seq_b_done(t + 1)); }
  // at the end of the prologue: B tile 0 has landed
  static constexpr int wait_pro() { return clamp(PRO_OPS - 1 - seq_b_done(0)); }
  // tiles t0 and t1 wait with the same counts everywhere (they can share their code)
  static constexpr bool same_waits(int t0, int t1) {
    if (wait_b(t0) != wait_b(t1)) return false;
    for (int s = 0; s < SPW; ++s)
      for (int i = 0; i < TMI; ++i)
        if (wait_a(t0, s, i) != wait_a(t1, s, i) || a_issued(t0, s) != a_issued(t1, s)) return false;
    return true;
  }
};

template <class C>
__device__ __forceinline__ void gemm_mfma_direct(const typename C::TA* __restrict__ A, const typename C::TB* __restrict__ B,
                                                 typename C::TC* __restrict__ Cm, char* smem, EpiArgs ep = EpiArgs{1.f, 0.f}) {
  typedef typename C::TA T;
  typedef typename C::TC TC;
  typedef DirectPlan<C> P;
  constexpr int BM = C::BM, BN = C::BN, BK = C::BK;
  constexpr int M = C::M, N = C::N, K = C::K;
  constexpr int WM = P::WM, WN = P::WN, MF = P::MF;
  constexpr int KH = 64 / MF, KS = P::KS, SPW = P::SPW;
  constexpr int TMI = WM / MF, TNI = WN / MF, NM = P::NM, NW = P::NW;
  typedef FetchMap<C> FM;
  constexpr int KT = FM::KT;                            // full K tiles
  constexpr int KR = FM::KR, SPWT = cdiv(KR, KS);       // the remainder: one more tile of SPWT k-steps (the last may be partial)
  constexpr int KTT = FM::KTT;
  constexpr bool FINAL_SPECIAL = FM::FINAL_SPECIAL;     // the last tile computes its fetch offsets on the spot
  constexpr int KTF = FM::KTF, KLAST = FM::KLAST;       // tiles in front of it; its k extent
  constexpr bool EDGE_M = M % BM != 0, EDGE_N = N % BN != 0;
  constexpr bool AK = !C::ATRANS;                       // A is k-contiguous in global memory
  constexpr int ES = P::ES, G = P::G;                   // element size; elements per 16-byte chunk
  constexpr int CHK = BK / G;                           // chunks per row of a k-contiguous tile
  constexpr int NCHA = BM / G, NCHB = BN / G;           // chunks per row of a row-contiguous tile
  constexpr bool AG = P::AG;                            // A goes from global memory straight into the fragment registers
  constexpr int A_BYTES = P::A_STAGE_BYTES, B_BYTES = BN * BK * ES, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int NIA = AG ? 0 : FM::NIA, NIB = FM::NIB;  // fetch instructions per wave and tile
  constexpr int FETCH_BYTES = 64 * 16;                  // LDS bytes one fetch instruction of a wave fills
  typedef Mfma<T, MF> MI;
  typedef typename MI::Acc Acc;
  typedef typename MI::Frag Frag;
  typedef LdsTile<CHK> LK;

  const int tid = threadIdx.x;
  // the wave number is the same in all lanes: saying so keeps everything derived from it (LDS fetch
  // destinations, which go through M0, and the wave's tile origin) in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
  const int wy = wave / C::BLN, wx = wave % C::BLN;
  int by, bx;
  block_coords<C>(blockIdx.x, by, bx);
  const int m0 = by * BM, n0 = bx * BN;
#if defined(KCG_DIAG_EVEN_XCD_SLEEP)
  const bool even_xcd = (__builtin_amdgcn_s_getreg(20 | (31 << 11)) & 1) == 0;
#endif
#if KCG_TIMELINE
  unsigned long long tl[KCG_TL_WORDS] = {};
  tl[0] = tl_realtime();
#endif

  // One LDS array holds the NST stages.  (No LDS access of this kernel is visible to the compiler as a
  // load: otherwise it would have to assume that the load may touch a stage a fetch is in flight to
  // and drain all fetches in front of it.)
  constexpr int NST = P::NST;
  __shared__ __attribute__((aligned(1024))) char lds_all[NST * STAGE_BYTES];
  (void)smem;
  auto stage_ptr = [&](auto stage_c) KCG_INL -> char* { return lds_all + decltype(stage_c)::value * STAGE_BYTES; };

  auto swz_n = [](int k, int nch) KCG_INL { return FM::swz_n(k, nch); };

  // ---- fetch: global -> LDS ------------------------------------------------------------------
  // Address = scalar tile base (advances with kt) + a 32-bit byte offset per lane and fetch item that
  // never changes (FetchMap): the K loop spends no vector instruction on addresses.
  auto off_a = [&](int idx) KCG_INL -> unsigned { return (unsigned)FM::a(wave, lane, idx, m0, BK, false).off; };
  auto off_b = [&](int j) KCG_INL -> unsigned { return (unsigned)FM::b(wave, lane, j, n0, BK, false).off; };
  unsigned voff_a[NIA > 0 ? NIA : 1], voff_b[NIB];
#pragma unroll
  for (int idx = 0; idx < NIA; ++idx) voff_a[idx] = off_a(idx);
#pragma unroll
  for (int j = 0; j < NIB; ++j) voff_b[j] = off_b(j);
  // AG: every wave reads its own WM rows of A, from ag_row0 on.  A wave whose rows all lie beyond M starts at the
  // last row that exists, so that the per-lane offsets from there (unsigned 32-bit) never have to be negative.
  const int ag_row0 = FM::ag_row0(wy, m0);
  const char* const a_base = (const char*)A + FM::a_tile(m0, 0) + (AG ? (long)ag_row0 * K * ES : 0L);
  const char* const b_base = (const char*)B + FM::b_tile(n0, 0);
  constexpr long A_KT_BYTES = FM::A_KT_BYTES, B_KT_BYTES = FM::B_KT_BYTES;   // one K tile further
  // The tile bases pass through an empty asm: the compiler must not fold the per-tile scalar part
  // into the per-lane part (it would hoist "base + lane offset" as a 64-bit vector value and add the
  // tile offset with vector instructions); kept apart, the fetch uses its scalar-base addressing form.
  struct TileBase { const char* a; const char* b; };
  auto tile_base = [&](int kt) KCG_INL {
    if constexpr (KCG_DIAG_FETCH_TILE0 != 0) kt = 0;
    TileBase t = {a_base + kt * A_KT_BYTES, b_base + kt * B_KT_BYTES};
    asm("" : "+s"(t.a), "+s"(t.b));
    return t;
  };
  // partial_c: the tile fetched is the last one and FINAL_SPECIAL
  auto fetch_item = [&](auto idx_c, const TileBase& tb, auto stage_c, auto partial_c) KCG_INL {
    constexpr bool PARTIAL = decltype(partial_c)::value;
    constexpr int idx = decltype(idx_c)::value;
    char* st = stage_ptr(stage_c);
    if constexpr (idx < NIA) {
      long off;
      if constexpr (PARTIAL) off = FM::a(wave, lane, idx, m0, KLAST, true).off;   // (signed: a moved chunk may start in front of the tile base)
      else {
        asm volatile("" : "+v"(voff_a[idx]));   // keeps the 32->64 bit extension next to the fetch (see tile_base)
        off = (long)(unsigned long)voff_a[idx];
      }
      const char* src = tb.a + off;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(st + FETCH_BYTES * (wave * NIA + idx)), 16, 0, KCG_FETCH_AUX);
    } else {
      constexpr int j = idx - NIA;
      long off;
      if constexpr (PARTIAL) off = FM::b(wave, lane, j, n0, KLAST, true).off;
      else {
        asm volatile("" : "+v"(voff_b[j]));
        off = (long)(unsigned long)voff_b[j];
      }
      const char* src = tb.b + off;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(st + A_BYTES + FETCH_BYTES * (wave * NIB + j)), 16, 0, KCG_FETCH_AUX);
    }
  };
  constexpr int NFETCH = NIA + NIB;
  // FIX_A / FIX_B: the chunk at the end of the matrix was fetched from SH elements further down, so its 16 bytes in
  // LDS hold the elements that exist in their upper part.  The lane that fetched it shifts them down (what the
  // upper part then stands for does not exist: columns beyond N, rows beyond M or k values beyond K).
  // Called by every wave once its own fetches of the last tile have landed, in front of the barrier that
  // publishes the tile.
  auto patch_final = [&](auto stage_c) KCG_INL {
    const unsigned st = (unsigned)(unsigned long)stage_ptr(stage_c);
    auto shift_down = [&](unsigned addr, auto bytes_c) KCG_INL {
      constexpr int SB = decltype(bytes_c)::value, WS = SB / 4, BS = (SB % 4) * 8;   // whole words; bits inside a word
      u32x4 w;
      asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(w) : "v"(addr) : "memory");
      const unsigned in[8] = {w.x, w.y, w.z, w.w, 0u, 0u, 0u, 0u};
      unsigned o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = BS ? (in[i + WS] >> BS) | (in[i + WS + 1] << ((32 - BS) % 32)) : in[i + WS];
      w = u32x4{o[0], o[1], o[2], o[3]};
      asm volatile("ds_write_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" ::"v"(addr), "v"(w) : "memory");
    };
    if constexpr (P::FIX_A) {
      if (m0 + BM >= M) {                       // (the block row with the last row of A, or its last column)
#pragma unroll
        for (int idx = 0; idx < NIA; ++idx)
          if (FM::a(wave, lane, idx, m0, KLAST, true).moved)
            shift_down(st + (unsigned)(FETCH_BYTES * (wave * NIA + idx) + lane * 16), IntC<P::SH_A * ES>());
      }
    }
    if constexpr (P::FIX_B) {
      if (n0 + BN >= N) {
#pragma unroll
        for (int j = 0; j < NIB; ++j)
          if (FM::b(wave, lane, j, n0, KLAST, true).moved)
            shift_down(st + (unsigned)(A_BYTES + FETCH_BYTES * (wave * NIB + j) + lane * 16), IntC<P::SH_B * ES>());
      }
    }
  };

  // ---- fragments -----------------------------------------------------------------------------
  // Every fragment read is issued as inline assembly.  As builtins or plain loads the compiler could
  // not tell that they do not touch the stage a fetch is in flight to and would drain all fetches
  // (vmcnt(0)) in front of them; it would also insert its own LDS waits, which know nothing of the
  // reads it cannot see.  The price: the compiler does not know that these reads are asynchronous, so
  // (1) the K loop counts the reads in flight itself and waits with s_waitcnt lgkmcnt(n) in front of the
  // matrix-core instructions that consume a fragment, and (2) a fragment stays in the very registers
  // the read instruction wrote (never a copy made before the data has arrived) until it is consumed.
  const int frow = lane % MF, fgrp = lane / MF;
  const int tx = lane % 16;                          // lane inside its 16-lane transposing group
  const int tsub = (lane / 16) % (MF / 16);          // which 16-column half of the matrix-core tile
  // a 32-bit word of two 16-bit k values of which the first `left` exist (K even: left is even, the middle case never occurs)
  struct Pair16 {
    __device__ __forceinline__ static unsigned keep(unsigned w, int left) {
      if constexpr (K % 2 == 0) return left > 0 ? w : 0u;
      else return left > 1 ? w : (left == 1 ? (w & 0xFFFFu) : 0u);
    }
  };
  struct FragTr {                                    // 16-bit, row-contiguous tile: two transposing 64-bit reads
    u32x2 h[2];
    __device__ __forceinline__ void pin() { asm volatile("" : "+v"(h[0]), "+v"(h[1])); }
    // nvalid: how many of the lane's G = 8 consecutive k values exist.  h[0] holds k values 0..3 of them (two per
    // 32-bit word, the earlier one in the lower half), h[1] the values 4..7.
    __device__ __forceinline__ void keep_first(int nvalid) {
      h[0].x = Pair16::keep(h[0].x, nvalid - 0); h[0].y = Pair16::keep(h[0].y, nvalid - 2);
      h[1].x = Pair16::keep(h[1].x, nvalid - 4); h[1].y = Pair16::keep(h[1].y, nvalid - 6);
    }
    __device__ __forceinline__ Frag get() const {
      const u32x4 v = {h[0].x, h[0].y, h[1].x, h[1].y};
      return __builtin_bit_cast(Frag, v);
    }
  };
  struct FragS4 {                                    // 32-bit, row-contiguous tile: four 32-bit reads
    unsigned w[4];
    __device__ __forceinline__ void pin() { asm volatile("" : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3])); }
    __device__ __forceinline__ void keep_first(int nvalid) {      // w[e] is the lane's e-th k value
#pragma unroll
      for (int e = 0; e < 4; ++e) w[e] = e < nvalid ? w[e] : 0u;
    }
    __device__ __forceinline__ Frag get() const {
      const u32x4 v = {w[0], w[1], w[2], w[3]};
      return __builtin_bit_cast(Frag, v);
    }
  };
  struct FragLd {                                    // k-contiguous tile: one 128-bit read
    u32x4 q;
    __device__ __forceinline__ void pin() { asm volatile("" : "+v"(q)); }
    __device__ __forceinline__ void keep_first(int nvalid) {
      if constexpr (ES == 4) {                                      // one k value per 32-bit word
        q.x = 0 < nvalid ? q.x : 0u; q.y = 1 < nvalid ? q.y : 0u; q.z = 2 < nvalid ? q.z : 0u; q.w = 3 < nvalid ? q.w : 0u;
      } else {                                                      // two k values per 32-bit word
        q.x = Pair16::keep(q.x, nvalid - 0); q.y = Pair16::keep(q.y, nvalid - 2); q.z = Pair16::keep(q.z, nvalid - 4); q.w = Pair16::keep(q.w, nvalid - 6);
      }
    }
    __device__ __forceinline__ Frag get() const { return __builtin_bit_cast(Frag, q); }
  };
  typedef typename Select<ES == 2, FragTr, FragS4>::type FragRc;
  typedef typename Select<AK, FragLd, FragRc>::type FragA;
  typedef FragRc FragB;
  constexpr int RC_READS = ES == 2 ? 2 : 4;          // LDS instructions per fragment of a row-contiguous tile
  // LDS address of a fragment read = a per-lane base that never changes (one register per fragment
  // column block of a row-contiguous tile, one per k-step of a k-contiguous tile) + a compile-time
  // offset (stage, k-step, fragment row block) that goes into the instruction's 16-bit offset field;
  // what does not fit the field is added to the base in units of 64 KiB.
  const unsigned lds0 = (unsigned)(unsigned long)lds_all;
  // Row-contiguous tile (nch chunks per row at byte offset toff of a stage): a lane reads the G k values
  // kb .. kb+G-1, kb = s*KS + G*fgrp, of column rowbase + lane%MF.
  //   16-bit: from two 4(k) x 16(n) blocks, each with one transposing read (16 lanes read a block and
  //           each receives a column);
  //   32-bit: one 32-bit read per k value.
  // The swizzle of a row depends on the lane only (swz_n looks at k bits that s and the read number do
  // not change).
  auto rc_lane_base = [&](int toff, int nch, int rowbase) KCG_INL {
    if constexpr (ES == 2) {
      const int n = rowbase + 16 * tsub + 4 * (tx % 4);
      const int k = 8 * fgrp + tx / 4;
      return lds0 + (unsigned)(toff + (k * nch + ((n / 8) ^ swz_n(k, nch))) * 16 + (n % 8) * 2);
    } else {
      const int n = rowbase + frow;
      const int k = 4 * fgrp;
      return lds0 + (unsigned)(toff + (k * nch + ((n / 4) ^ swz_n(k, nch))) * 16 + (n % 4) * 4);
    }
  };
  unsigned b_lane[TNI];
#pragma unroll
  for (int j = 0; j < TNI; ++j) b_lane[j] = rc_lane_base(A_BYTES, NCHB, wx * WN + j * MF);
  constexpr int NALANE = AG ? TMI : (AK ? SPW : TMI);
  unsigned a_lane[NALANE];
  if constexpr (AG) {
    // byte offset of the lane's 16 bytes of fragment row block i from the wave's part of the K tile
#pragma unroll
    for (int i = 0; i < TMI; ++i) a_lane[i] = FM::ag_lane(i, lane, m0, ag_row0);
  } else if constexpr (AK) {
#pragma unroll
    for (int st = 0; st < SPW; ++st)
      a_lane[st] = lds0 + (unsigned)(LK::slot(wy * WM + frow, st * KH + fgrp) * 16);   // swizzle: row%16 = frow%16 only
  } else {
#pragma unroll
    for (int i = 0; i < TMI; ++i) a_lane[i] = rc_lane_base(0, NCHA, wy * WM + i * MF);
  }
  auto split_base = [](unsigned lane_base, int imm) KCG_INL { return lane_base + (unsigned)(imm / 65536) * 65536u; };
  auto read_rc = [&](unsigned lane_base, auto imm_c, auto nch_c, FragRc* dst) KCG_INL {
    constexpr int IMM0 = decltype(imm_c)::value, ROW = decltype(nch_c)::value * 16;   // bytes per tile row
    if constexpr (ES == 2) {
      constexpr int IMM1 = IMM0 + 4 * ROW;                              // second block: four rows further
      const unsigned base0 = split_base(lane_base, IMM0), base1 = split_base(lane_base, IMM1);
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst->h[0]) : "v"(base0), "n"(IMM0 % 65536));
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst->h[1]) : "v"(base1), "n"(IMM1 % 65536));
    } else {
      constexpr int IMM1 = IMM0 + ROW, IMM2 = IMM0 + 2 * ROW, IMM3 = IMM0 + 3 * ROW;   // one tile row per k value
      const unsigned base0 = split_base(lane_base, IMM0), base1 = split_base(lane_base, IMM1);
      const unsigned base2 = split_base(lane_base, IMM2), base3 = split_base(lane_base, IMM3);
      asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(dst->w[0]) : "v"(base0), "n"(IMM0 % 65536));
      asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(dst->w[1]) : "v"(base1), "n"(IMM1 % 65536));
      asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(dst->w[2]) : "v"(base2), "n"(IMM2 % 65536));
      asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(dst->w[3]) : "v"(base3), "n"(IMM3 % 65536));
    }
  };
  // fragment f of k-step s of the stage: s, f and the stage are compile-time constants (IntC)
  auto load_a = [&](auto stage_c, auto s_c, auto f_c, FragA* dst) KCG_INL {
    constexpr int ST = decltype(stage_c)::value, S = decltype(s_c)::value, F = decltype(f_c)::value;
    if constexpr (AK) {
      constexpr int IMM = ST * STAGE_BYTES + F * MF * CHK * 16;
      const unsigned base = split_base(a_lane[S], IMM);
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst->q) : "v"(base), "n"(IMM % 65536));
    } else {
      read_rc(a_lane[F], IntC<ST * STAGE_BYTES + S * KS * NCHA * 16>(), IntC<NCHA>(), dst);
    }
  };
  // AG: fragment f of k-step s of the K tile at `base` (scalar), straight from global memory.  Like the LDS reads
  // an instruction the compiler does not see as a load: the K loop waits for it itself (VmSchedule).
  auto load_ag = [&](const char* base, auto s_c, auto f_c, FragLd* dst) KCG_INL {
    constexpr int S = decltype(s_c)::value, F = decltype(f_c)::value;
    const unsigned off = a_lane[F];
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(dst->q) : "v"(off), "s"(base), "n"(S * KS * ES));
  };
  auto load_b = [&](auto stage_c, auto s_c, auto f_c, FragB* dst) KCG_INL {
    constexpr int ST = decltype(stage_c)::value, S = decltype(s_c)::value, F = decltype(f_c)::value;
    read_rc(b_lane[F], IntC<ST * STAGE_BYTES + S * KS * NCHB * 16>(), IntC<NCHB>(), dst);
  };
  // lgkmcnt(0): every LDS read issued so far has returned
  auto wait_lds = [&]() KCG_INL { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); };

  // prologue, first half: the first NST tiles go out together (the wait further down is for tile 0
  // alone: its successors' memory latency overlaps with it instead of following it), and before
  // anything else that takes time: clearing the accumulators runs under that latency
  static_for<0, NST>([&](auto t) KCG_INL {
    if constexpr (decltype(t)::value < KTT) {
      const TileBase tb = tile_base(decltype(t)::value);
      static_for<0, NFETCH>([&](auto i) KCG_INL { fetch_item(i, tb, t, BoolC<(FINAL_SPECIAL && decltype(t)::value == KTF)>()); });
    }
  });

  Acc acc[TMI][TNI];
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j)
#pragma unroll
      for (int e = 0; e < (int)(sizeof(Acc) / sizeof(float)); ++e) acc[i][j][e] = 0.0f;
  // The zeros must be in their registers here and now: left alone the compiler writes them right in
  // front of the first matrix-core instruction of each accumulator, and that instruction (which the
  // compiler does not recognise as one, see Mfma::run_tied) would need wait states after such a write.
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j) asm volatile("" : "+a"(acc[i][j]));
  asm volatile("s_nop 7" ::: "memory");

  // ---- K loop ----------------------------------------------------------------------------------
  // Time line of a k-step: its NM = TMI x TNI matrix-core instructions, row by row (row i: fragment
  // A_i against B_0..B_TNI-1).  Side work is pinned to slots of that time line:
  //   * the A fragment that row i+DA needs is read when row i starts (rows >= TMI: rows of the next
  //     step); it replaces the fragment of a row that is done, so A takes TMI fragments of registers;
  //   * the B fragments of the next step are read into the other half of a double buffer in the slots
  //     slot_b(j) of rows RB..TMI-2 (RB = TMI-DA);
  //   * in the last step of a tile the barrier stands where row RB starts: all reads of this stage
  //     have been issued by then, and everything read from there on belongs to the next tile;
  //   * fetches: see below.
  // LDS reads return in order, so "fragment X has arrived" is "at most n reads issued after X are
  // still in flight"; n is a compile-time property of this schedule (StreamPlan::allowed).
#ifndef KCG_SCHED_A_AHEAD
#define KCG_SCHED_A_AHEAD 0           /* rows an A fragment is read ahead of its use; 0 = TMI-1 */
#endif
  // (the further ahead, the earlier the barrier stands in the last step and the more room the fetches
  // behind it have; measured best at the maximum)
  constexpr int DA = cmax(1, cmin(TMI - 1, KCG_SCHED_A_AHEAD > 0 ? KCG_SCHED_A_AHEAD : TMI - 1));
  typedef StreamPlan<TMI, TNI, DA, (AG ? 0 : AK ? 1 : RC_READS), RC_READS> SP;
  constexpr int RB = SP::RB;
  constexpr int MT = SPW * NM;
  constexpr int BAR = (SPW - 1) * NM + RB * TNI;
  constexpr int TAIL = MT - BAR;
  static_assert(TMI >= 2, "the streaming schedule needs two rows of matrix-core tiles per wave");
  static_assert((NST * SPW) % 2 == 0, "B double buffer: the parity of a step must follow from its stage");
  // s_waitcnt vmcnt(n), everything else unconstrained: n fetches of this wave may still be in flight
  static_assert((NST - 2) * P::VMOPS < 64, "vmcnt has 6 bits");
  constexpr int SPREAD = NST >= 3 ? MT : TAIL;                            // see "One K tile" below
  constexpr int AGD = P::AG_DEPTH;
  typedef VmSchedule<KTT, SPW, TMI, TNI, NIB, NST, BAR, SPREAD, AGD> VS;  // AG only
  static_assert(!AG || ((NST * SPW) % AGD == 0 && KR == 0), "AG: the ring slot of a fragment must follow from stage and step");
  auto vmcnt_only = [](int n) KCG_INL { return 0x0F70 | (n & 15) | ((n >> 4) << 14); };
  auto tiles_ahead = [](int t) KCG_INL {
    const int last = cmin(KTT - 1, t == 0 ? NST - 1 : t - 1 + NST);  // newest tile whose fetch has been issued
    return cmax(0, last - (t + 1));
  };

  // prologue, second half
  constexpr int NPRO = cmin(NST, KTT);                                    // tiles the prologue has issued
  // AG: A fragments live in a ring of AGD k-steps, fa[(step % AGD) * TMI + row]; the first AGD steps are loaded here
  FragA fa[AG ? AGD * TMI : TMI];
  if constexpr (AG) {
    static_for<0, cmin(AGD, KTT * SPW)>([&](auto gs_c) KCG_INL {
      constexpr int GS = decltype(gs_c)::value;
      const TileBase tb = tile_base(GS / SPW);
      static_for<0, TMI>([&](auto i) KCG_INL { load_ag(tb.a, IntC<GS % SPW>(), i, &fa[(GS % AGD) * TMI + decltype(i)::value]); });
    });
    __builtin_amdgcn_s_waitcnt(vmcnt_only(VS::wait_pro()));
  } else {
    __builtin_amdgcn_s_waitcnt(vmcnt_only(cmin(63, (NPRO - 1) * NFETCH)));  // this wave's chunks of tile 0 are in LDS
  }
  asm volatile("" ::: "memory");
  if constexpr ((P::FIX_A || P::FIX_B) && KTT == 1) patch_final(IntC<0>());
  __builtin_amdgcn_s_barrier();                                            // ... and everyone's (bare barrier: see the K loop)
  asm volatile("" ::: "memory");
#if KCG_TIMELINE
  tl[1] = tl_realtime();
  const unsigned long long tl_c0 = tl_cycles();
#endif
  FragB fb[2][TNI];
  constexpr bool NO_READS_A = KCG_DIAG_NO_LDS_READS == 1 || KCG_DIAG_NO_LDS_READS == 2;   // diagnostic builds
  constexpr bool NO_READS_B = KCG_DIAG_NO_LDS_READS == 1 || KCG_DIAG_NO_LDS_READS == 3;
  static_for<0, TNI>([&](auto j) KCG_INL { load_b(IntC<0>(), IntC<0>(), j, &fb[0][decltype(j)::value]); });
  if constexpr (!AG)
    static_for<0, (NO_READS_A ? TMI : DA)>([&](auto i) KCG_INL { load_a(IntC<0>(), IntC<0>(), i, &fa[decltype(i)::value]); });
  if constexpr (NO_READS_B && SPW > 1)
    static_for<0, TNI>([&](auto j) KCG_INL { load_b(IntC<0>(), IntC<1>(), j, &fb[1][decltype(j)::value]); });
  wait_lds();   // the counted waits of the loop assume that nothing older than its own reads is in flight

  // One K tile.  CUR: the stage it computes from; H1: tile kt+1 exists; HN: tile kt+NST exists; HP: the
  // fetch of tile kt-1+NST, begun behind the previous tile's barrier, is still being issued.  NS: k-steps
  // of this tile (SPW, fewer for the partial tile); PN / PP: the tile fetched under HN / HP is the partial one.
  //
  // A stage is free once the barrier of the tile that computed from it has been passed, and the tile
  // fetched into it is needed NST-1 barriers later.  With three or more stages its NFETCH fetch
  // instructions are spread over the whole period up to the next barrier (the memory pipeline of a CU
  // takes 16 cycles per 1 KiB fetch instruction; four waves issuing all of theirs right behind the
  // barrier would stall on it); with two stages they must all be issued in the rest of this tile.
  // AG: tsim_c is the tile's number in the operation order of VmSchedule (its own number, or for the tiles of the
  // run-time loop that of the first tile that executes the same code).
  typedef FetchSlots<NFETCH, NIA, BAR, SPREAD> FS;
  auto tile = [&](int kt, auto cur_c, auto has1, auto hasn, auto hasp, auto ahead_c, auto ns_c, auto pn_c, auto pp_c, auto fixn_c,
                  auto tsim_c) KCG_INL {
    constexpr int TSIM = decltype(tsim_c)::value;
    constexpr int CUR = decltype(cur_c)::value, NS = decltype(ns_c)::value;
    constexpr int NXT = (CUR + 1) % NST, PRV = (CUR + NST - 1) % NST;
    constexpr bool H1 = decltype(has1)::value, HN = decltype(hasn)::value;
    constexpr bool HP = decltype(hasp)::value && SPREAD > TAIL;
    const TileBase tbn = tile_base(HN ? kt + NST : 0);
    const TileBase tbp = tile_base(HP ? kt - 1 + NST : 0);
    // In the partial K tile a k-step may reach beyond K: every fragment layout of this kernel gives a lane
    // the G consecutive k values that start at S*KS + G*(lane/MF); those of them that are >= K (what was
    // fetched in their place is arbitrary) are cleared before use.
    constexpr bool PARTIAL = KR > 0 && NS == SPWT && decltype(has1)::value == false && (KR % KS != 0);
    static_for<0, NS>([&](auto s_c) KCG_INL {
      constexpr int S = decltype(s_c)::value;
      constexpr bool LAST = (S == NS - 1);
      constexpr bool MASK = PARTIAL && LAST;
      const int nvalid = KR - (S * KS + G * fgrp);   // how many of this lane's G consecutive k values lie below K
      constexpr int PB = (CUR * SPW + S) & 1;       // half of the B double buffer this step computes from
      constexpr bool NEXT = !LAST || H1;            // a next step exists, its fragments are read under this one
      constexpr int RING = AG ? ((CUR * SPW + S) % AGD) * TMI : 0;     // AG: this step's slots in the ring of A fragments
      // AG: the load issued behind row I fetches row I of the step AGD further on, into the registers this row frees
      constexpr bool A_NEXT = AG && (TSIM * SPW + S + AGD < KTT * SPW);
      const char* a_next = nullptr;
      if constexpr (A_NEXT) a_next = tile_base(kt + (S + AGD) / SPW).a;
      static_for<0, TMI>([&](auto i_c) KCG_INL {
        constexpr int I = decltype(i_c)::value;
        constexpr int FI = RING + I;
        // AG: this row's A fragment has arrived (vmcnt counts fetches and A loads alike, in order)
        if constexpr (AG) __builtin_amdgcn_s_waitcnt(vmcnt_only(VS::wait_a(TSIM, S, I)));
        // the fragments of this row have arrived.  Without a next step the reads the count relies on
        // are not issued: wait for everything instead.
        if constexpr (NEXT) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(SP::allowed(I)) : "memory");
        else wait_lds();
        if constexpr (LAST && I == RB) {
          // tile kt+1 has landed (this wave's part): of the fetches issued so far only those of the
          // tiles behind it may still be in flight
#if KCG_TIMELINE >= 2
          wait_lds();        // (level 2: the stamp's own wait must not count as barrier wait)
          const unsigned long long tl_b0 = tl_cycles();
#endif
          if constexpr (H1 && AG) __builtin_amdgcn_s_waitcnt(vmcnt_only(VS::wait_b(TSIM)));
          else if constexpr (H1) __builtin_amdgcn_s_waitcnt(vmcnt_only(decltype(ahead_c)::value * NFETCH));
          wait_lds();        // this wave's reads of stage CUR have all returned
          if constexpr (decltype(fixn_c)::value) patch_final(IntC<NXT>());   // tile kt+1 is the last one (nothing behind it in flight)
          // ... everyone's part; and every wave is done reading stage CUR.  The bare barrier instruction:
          // __syncthreads() comes with a fence in front of which the compiler drains every fetch in
          // flight (vmcnt(0)), which would expose the whole memory latency at each tile.  What has
          // to be complete at this point is exactly what the two waits above ask for.
          asm volatile("" ::: "memory");
#if defined(KCG_DIAG_EVEN_XCD_SLEEP)
          if (even_xcd) __builtin_amdgcn_s_sleep(KCG_DIAG_EVEN_XCD_SLEEP);
#endif
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
#if KCG_TIMELINE >= 2
          tl[7] += tl_cycles() - tl_b0;
#endif
        }
        // the empty asm statements make the fragments "outputs" of the wait: the matrix-core
        // instructions that consume them cannot be scheduled in front of it
        fa[FI].pin();
        if constexpr (I == 0) {
#pragma unroll
          for (int j = 0; j < TNI; ++j) fb[PB][j].pin();
        }
        if constexpr (MASK) {
          // (pinned again behind the selects: they must have been issued before the wait state that
          // separates them from the matrix-core instruction reading their results)
          fa[FI].keep_first(nvalid);
          fa[FI].pin();
          if constexpr (I == 0) {
#pragma unroll
            for (int j = 0; j < TNI; ++j) {
              fb[PB][j].keep_first(nvalid);
              fb[PB][j].pin();
            }
          }
          asm volatile("s_nop 1" ::: "memory");
        }
        if constexpr (NO_READS_A || AG) {
        } else if constexpr (I + DA < TMI) load_a(IntC<CUR>(), IntC<S>(), IntC<I + DA>(), &fa[I + DA]);
        else if constexpr (!LAST) load_a(IntC<CUR>(), IntC<S + 1>(), IntC<I + DA - TMI>(), &fa[I + DA - TMI]);
        else if constexpr (H1) load_a(IntC<NXT>(), IntC<0>(), IntC<I + DA - TMI>(), &fa[I + DA - TMI]);
        static_for<0, TNI>([&](auto j_c) KCG_INL {
          constexpr int J = decltype(j_c)::value;
          constexpr int slot = S * NM + I * TNI + J;
          // operands swapped (B fragment first): the accumulator then holds C^T tiles, i.e. each lane owns
          // one row m and groups of four consecutive n, which the epilogue stores as 128-bit vectors
          // odd rows run right to left: neighbours on the time line always share one operand
          constexpr int JC = (I & 1) ? TNI - 1 - J : J;
          MI::run_tied(acc[I][JC], fb[PB][JC].get(), fa[FI].get());
          static_for<SP::first_b(I * TNI + J), SP::first_b(I * TNI + J + 1)>([&](auto jj_c) KCG_INL {
            constexpr int JJ = decltype(jj_c)::value;
            if constexpr (!NO_READS_B) {
              if constexpr (!LAST) load_b(IntC<CUR>(), IntC<S + 1>(), jj_c, &fb[PB ^ 1][JJ]);
              else if constexpr (H1) load_b(IntC<NXT>(), IntC<0>(), jj_c, &fb[PB ^ 1][JJ]);
            }
          });
          // the fetch items whose position on the time line (FetchSlots::pos, counted from the start of the tile that
          // begins the fetch) is this slot: of tile kt+NST, and, a period later, of tile kt-1+NST; ascending f
          if constexpr (HN)
            static_for<FS::lo(slot), FS::lo(slot + 1)>([&](auto f_c) KCG_INL {
              if constexpr (FS::on(decltype(f_c)::value)) fetch_item(f_c, tbn, IntC<CUR>(), pn_c);
            });
          if constexpr (HP)
            static_for<FS::lo(slot + MT), FS::lo(slot + MT + 1)>([&](auto f_c) KCG_INL {
              if constexpr (FS::on(decltype(f_c)::value)) fetch_item(f_c, tbp, IntC<PRV>(), pp_c);
            });
          __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (A_NEXT) {
          load_ag(a_next, IntC<(S + AGD) % SPW>(), i_c, &fa[FI]);
          __builtin_amdgcn_sched_barrier(0);
        }
      });
    });
  };
  // Tile 0 first (nothing of an earlier period to continue); then groups of NST tiles that have every
  // neighbour; the rest is unrolled with the right flags at compile time (KT is a constant).
  // tiles_ahead(T): how many tiles behind tile T+1 have been issued when tile T reaches its barrier
  // (the prologue issued tiles 0..NST-1, tile t issues or completes the issue of tile t-1+NST)
  typedef BoolC<false> No;
  constexpr bool FIX = P::FIX_A || P::FIX_B;
  tile(0, IntC<0>(), BoolC<(1 < KTT)>(), BoolC<(NST < KTT)>(), No(), IntC<tiles_ahead(0)>(), IntC<(0 < KT ? SPW : SPWT)>(),
       BoolC<(FINAL_SPECIAL && NST == KTF)>(), No(), BoolC<(FIX && 2 == KTT)>(), IntC<0>());
  auto static_tile = [&](auto tc) KCG_INL {
    constexpr int T = decltype(tc)::value;
    tile(T, IntC<T % NST>(), BoolC<(T + 1 < KTT)>(), BoolC<(T + NST < KTT)>(), BoolC<(T - 1 + NST < KTT)>(), IntC<tiles_ahead(T)>(),
         IntC<(T < KT ? SPW : SPWT)>(), BoolC<(FINAL_SPECIAL && T + NST == KTF)>(), BoolC<(FINAL_SPECIAL && T - 1 + NST == KTF)>(),
         BoolC<(FIX && T + 2 == KTT)>(), tc);
  };
  // The run-time loop starts at tile L0.  AG: the wait counts of a tile depend on what was issued up to NST-1
  // tiles earlier, and the prologue issued the first NST tiles in another order than the loop does: the tiles in
  // front of L0 = NST are unrolled with their own counts.
  constexpr int L0 = AG ? cmax(NST, 2) : 1;
  static_for<1, cmin(L0, KTT)>(static_tile);
  constexpr int NFULL = KTF - NST - L0 > 0 ? KTF - NST - L0 : 0;   // tiles L0 .. KTF-NST-1 have kt+NST < KTF: ordinary tiles all round
  constexpr int NG = NFULL / NST;
  for (int g = 0; g < NG; ++g) {
    static_for<0, NST>([&](auto sc) KCG_INL {
      constexpr int S = decltype(sc)::value;
      static_assert(!AG || NG == 0 || VS::same_waits(L0 + S, L0 + (NG > 0 ? NG - 1 : 0) * NST + S), "AG: the loop's tiles must wait alike");
      tile(L0 + g * NST + S, IntC<(L0 + S) % NST>(), BoolC<true>(), BoolC<true>(), BoolC<true>(), IntC<NST - 2>(), IntC<SPW>(), No(), No(), No(),
           IntC<L0 + S>());
    });
  }
  static_for<cmax(L0, 1) + NG * NST, KTT>(static_tile);

  // the last matrix-core results must have left the pipeline before the epilogue reads them (the
  // compiler, which normally inserts these wait states, does not know the instructions above)
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#if KCG_TIMELINE
  tl[5] = tl_cycles() - tl_c0;
  tl[2] = tl_realtime();
#endif
  // ... and the epilogue's reads must stay behind those wait states: an accumulator is an ordinary
  // register value to the compiler, free to be read (converted, moved) ahead of an asm statement that does
  // not mention it.  Passing every accumulator through an empty asm statement behind the wait states
  // makes each read depend on it (asm volatile statements keep their order).
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j) asm volatile("" : "+a"(acc[i][j]));
  // ---- epilogue --------------------------------------------------------------------------------
  // With swapped operands a 32x32 accumulator holds, per lane, row m = lane%32 and columns
  // n = 8*g + 4*(lane/32) + {0..3} for g = 0..3 (16x16: row lane%16, columns 4*(lane/16) + {0..3}).
  constexpr int NACC = (int)(sizeof(Acc) / sizeof(float));
  const int orow = lane % MF;
  const int ocol = (lane / MF) * 4;
  // Diagnostic builds only (never set by the library itself): -DKCG_DIAG_STORE_ROWS=n stores just the first n
  // rows of matrix-core tiles of every wave tile, so C is INCOMPLETE; timing such a build shows how much of a
  // launch the C stores cost (n = 0) and what hiding a part of them under matrix work could gain at best.
#ifndef KCG_DIAG_STORE_ROWS
#define KCG_DIAG_STORE_ROWS -1
#endif
  constexpr int STORE_ROWS = KCG_DIAG_STORE_ROWS < 0 ? TMI : cmin(TMI, KCG_DIAG_STORE_ROWS);
#pragma unroll
  for (int i = 0; i < STORE_ROWS; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j)
#pragma unroll
      for (int g = 0; g < NACC / 4; ++g) {
        const int row = m0 + wy * WM + i * MF + orow;
        const int col = n0 + wx * WN + j * MF + g * 8 + ocol;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][g * 4 + e];
        // (N a multiple of 4: every group of four columns is one aligned 16-byte vector, inside or outside as a whole)
        if constexpr (C::EPI) epi_apply<TC, float, 4, (EDGE_M || EDGE_N), (N % 4 == 0)>(v, Cm, row, col, N, M, N, ep);
#if defined(KCG_DIAG_STORE_LINES)
        // diagnostic build (C WRONG: values land in other places): the same 64 store instructions per wave, each writing
        // KCG_DIAG_STORE_LINES*64 contiguous bytes per row (2: whole 128-byte lines of 8 rows, 4: 256 bytes of 4 rows)
        // instead of 64 bytes of 16 rows
        {
          constexpr int LPR = 4 * KCG_DIAG_STORE_LINES, RPI = 64 / LPR;      // lanes per row; rows per instruction
          const int t = (i * TNI + j) * (NACC / 4) + g;
          constexpr int CG = WN / (LPR * 4);                                  // column groups per wave tile
          const int drow = m0 + wy * WM + (t / CG) * RPI + lane % RPI;
          const int dcol = n0 + wx * WN + (t % CG) * (LPR * 4) + (lane / RPI) * 4;
          gstore<TC, float, 4, (EDGE_M || EDGE_N), (N % 4 == 0), (KCG_C_NT != 0)>(Cm, v, drow, dcol, N, M, N);
        }
#else
        gstore<TC, float, 4, (EDGE_M || EDGE_N), (N % 4 == 0), (KCG_C_NT != 0)>(Cm, v, row, col, N, M, N);
#endif
      }
#if KCG_TIMELINE
  asm volatile("" ::: "memory");
  tl[3] = tl_realtime();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  tl[4] = tl_realtime();
  tl[6] = (unsigned long long)__builtin_amdgcn_s_getreg(4 | (31 << 11)) |            // HW_REG_HW_ID
          ((unsigned long long)__builtin_amdgcn_s_getreg(20 | (31 << 11)) << 32);     // HW_REG_XCC_ID
  if (kcg_timeline_ptr != nullptr && lane == 0) {
    unsigned long long* rec = kcg_timeline_ptr + ((size_t)blockIdx.x * NW + wave) * KCG_TL_WORDS;
#pragma unroll
    for (int w = 0; w < KCG_TL_WORDS; ++w) rec[w] = tl[w];
  }
#endif
}

}  // namespace kcg
