// kcg_gemm_device.h — hand-written gfx950 (CDNA4, wave64) GEMM kernel templates.
//
// This header is embedded into libkcg_gemm.so and handed to hiprtc together with a generated
// instantiation stub that defines one `struct Cfg` (all tuning parameters as constexpr members) and
// one `extern "C" __global__` entry named like the reference kernel.  It replaces what the reference
// obtains by rewriting affine MLIR (src/lib/Conversion/Optimizer.cc:285-469) and lowering it to
// AMDGCN: here the same schedule parameters select code paths of a fixed template at compile time.
//
// Semantics of the product (Matmul.cc:41-65):  C[i,j] = sum_{k=0..K-1} A(i,k) * B[k,j]
//   IS_ATRANS=1 : A buffer is [K,M] row-major (A(i,k) = A[k*M+i])   — the layout of every shipped JSON
//   IS_ATRANS=0 : A buffer is [M,K] row-major (A(i,k) = A[i*K+k])
//   B buffer is [K,N] row-major, C buffer is [M,N] row-major; M,N,K are compile-time constants and
//   the kernel takes three raw global pointers (Matmul.cc:115-120).
//
// Two kernel families:
//   gemm_simt : scalar-FMA register-tiled kernel that follows the tuning config literally
//               (thread tile TMxTN, warp/lane scatter, split-U across thread-z, optional LDS and
//               register double buffering).  It is the fallback for configs whose wave tile cannot
//               be covered by matrix-core tiles.
//   gemm_mfma : wave-tiled matrix-core kernel (v_mfma_f32_32x32x2_f32 / 16x16x4_f32,
//               v_mfma_f32_32x32x16_{f16,bf16} / 16x16x32_{f16,bf16}); operands are staged in LDS
//               as [row][k] with 16-byte chunks XOR-swizzled so that every fragment is a single
//               conflict-free ds_read_b128.
//
// No host headers are available under hiprtc; only compiler builtins are used.
#pragma once

namespace kcg {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef double doublex2 __attribute__((ext_vector_type(2)));
typedef double doublex4 __attribute__((ext_vector_type(4)));
typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <int BYTES> struct RawVec;
template <> struct RawVec<1> { typedef unsigned char type; };
template <> struct RawVec<2> { typedef unsigned short type; };
template <> struct RawVec<4> { typedef unsigned int type; };
template <> struct RawVec<8> { typedef u32x2 type; };
template <> struct RawVec<16> { typedef u32x4 type; };

template <class T> struct AccOf { typedef float type; };
template <> struct AccOf<double> { typedef double type; };

constexpr int cdiv(int a, int b) { return (a + b - 1) / b; }
constexpr int cmin(int a, int b) { return a < b ? a : b; }
constexpr int cmax(int a, int b) { return a > b ? a : b; }
constexpr int lowbit(int a) { return a & (-a); }
template <bool B> struct BoolC { static constexpr bool value = B; };
template <bool B, class X, class Y> struct Select { typedef X type; };
template <class X, class Y> struct Select<false, X, Y> { typedef Y type; };
template <int I> struct IntC { static constexpr int value = I; };
// f(IntC<Begin>()), ..., f(IntC<End-1>()) — a loop whose index is a compile-time constant in the body
template <int Begin, int End, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (Begin < End) {
    f(IntC<Begin>());
    static_for<Begin + 1, End>(f);
  }
}

// Copy NBYTES (power of two, <= 16) between two suitably aligned addresses as one access.
template <int NBYTES>
__device__ __forceinline__ void copy_bytes(void* dst, const void* src) {
  typedef typename RawVec<NBYTES>::type V;
  *reinterpret_cast<V*>(dst) = *reinterpret_cast<const V*>(src);
}

// ---------------------------------------------------------------------------------------------
// Block id -> (by, bx).  Rewriter::BlockMapping (Rewriter.cc:726-761): groups of BLOCK_MAPPING block
// rows are walked column by column so that concurrently resident blocks share B panels in L2.
// On top of it, when the block count is a multiple of 8, consecutive hardware ids (which the
// dispatcher deals round-robin to the 8 XCDs, each with a private L2) are remapped so that every XCD
// walks one contiguous eighth of that order.
// ---------------------------------------------------------------------------------------------
template <class C>
__device__ __forceinline__ void block_coords(int bid, int& by, int& bx) {
  constexpr int GY = cdiv(C::M, C::BM);
  constexpr int GX = cdiv(C::N, C::BN);
  constexpr int NB = GY * GX;
  if constexpr (C::XCD_REMAP && (NB % 8 == 0)) {
    bid = (bid % 8) * (NB / 8) + bid / 8;
  }
  if constexpr (C::BLOCK_MAPPING > 0 && (GY % (C::BLOCK_MAPPING > 0 ? C::BLOCK_MAPPING : 1) == 0)) {
    constexpr int G = C::BLOCK_MAPPING;
    constexpr int GN = G * GX;
    by = (bid / GN) * G + bid % G;
    bx = (bid % GN) / G;
  } else {
    by = bid / GX;
    bx = bid % GX;
  }
}

// ---------------------------------------------------------------------------------------------
// Thread -> vector map over a ROWS x COLS tile whose COLS dimension is contiguous in memory.
//   CONT=1 ("LOAD_CONTINUOUS", Optimizer.cc:79-83):  v = tid + it*NT, row = v / VPR, col = (v % VPR)*VEC
//   CONT=0 (Optimizer.cc:84-88): row = tid / (NT/ROWS), col = it*(NT/ROWS*VEC) + (tid % (NT/ROWS))*VEC
// ---------------------------------------------------------------------------------------------
template <int ROWS, int COLS, int VEC, int NT, bool CONT>
struct TileMap {
  static constexpr int VPR = COLS / VEC;
  static constexpr int NV = ROWS * VPR;
  static constexpr int TPR = CONT ? 1 : NT / ROWS;
  static constexpr int ITERS = CONT ? cdiv(NV, NT) : COLS / (TPR * VEC);
  static constexpr bool FULL = CONT ? (NV % NT == 0) : true;
  __device__ __forceinline__ static bool coords(int tid, int it, int& r, int& c) {
    if constexpr (CONT) {
      int v = tid + it * NT;
      r = v / VPR;
      c = (v % VPR) * VEC;
      return FULL || v < NV;
    } else {
      r = tid / TPR;
      c = it * (TPR * VEC) + (tid % TPR) * VEC;
      return true;
    }
  }
};

// Thread -> (k chunk, first row) map for an operand tile that is contiguous along m/n in global memory
// and is transposed into [row][k chunk] LDS layout: NCH k-chunks x NVEC row vectors of VEC rows.
//   ROWS_FAST=1: consecutive threads take consecutive row vectors (widest global coalescing)
//   ROWS_FAST=0: consecutive threads take consecutive k chunks of one row vector, so the 16-byte LDS
//                writes of 8 neighbouring lanes land in 8 different bank groups
template <int NCH, int NVEC, int VEC, int NT, bool ROWS_FAST>
struct BlockMap {
  static constexpr int NB = NCH * NVEC;
  static constexpr int ITERS = cdiv(NB, NT);
  static constexpr bool FULL = (NB % NT == 0);
  __device__ __forceinline__ static bool coords(int tid, int it, int& chunk, int& row) {
    int v = tid + it * NT;
    if constexpr (ROWS_FAST) {
      chunk = v / NVEC;
      row = (v % NVEC) * VEC;
    } else {
      chunk = v % NCH;
      row = (v / NCH) * VEC;
    }
    return FULL || v < NB;
  }
};

// Load VEC consecutive elements T from row r, column c of a row-major matrix with leading dimension
// LD into dst[0..VEC).  With EDGE, elements outside [0,RMAX) x [0,CMAX) read as zero.  ALIGNED says
// every such vector is naturally aligned to VEC*sizeof(T) so one wide load is legal.
template <class T, int VEC, bool EDGE, bool ALIGNED>
__device__ __forceinline__ void gload(T* dst, const T* __restrict__ base, int r, int c, int LD, int RMAX, int CMAX) {
  if constexpr (!EDGE) {
    if constexpr (ALIGNED) {
      copy_bytes<VEC * (int)sizeof(T)>(dst, base + (long)r * LD + c);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) dst[e] = base[(long)r * LD + c + e];
    }
  } else {
    if (ALIGNED && r < RMAX && c + VEC <= CMAX) {
      copy_bytes<VEC * (int)sizeof(T)>(dst, base + (long)r * LD + c);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        dst[e] = (r < RMAX && c + e < CMAX) ? base[(long)r * LD + c + e] : T(0);
      }
    }
  }
}

// Store VEC consecutive output elements (converted from the accumulator type) with the same rules.
template <class TC, class ACC, int VEC, bool EDGE, bool ALIGNED>
__device__ __forceinline__ void gstore(TC* __restrict__ base, const ACC* src, int r, int c, int LD, int RMAX, int CMAX) {
  TC tmp[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) tmp[e] = (TC)src[e];
  if constexpr (!EDGE) {
    if constexpr (ALIGNED) {
      copy_bytes<VEC * (int)sizeof(TC)>(base + (long)r * LD + c, tmp);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) base[(long)r * LD + c + e] = tmp[e];
    }
  } else {
    if (ALIGNED && r < RMAX && c + VEC <= CMAX) {
      copy_bytes<VEC * (int)sizeof(TC)>(base + (long)r * LD + c, tmp);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        if (r < RMAX && c + e < CMAX) base[(long)r * LD + c + e] = tmp[e];
    }
  }
}

// Split-U epilogue shared by both families (Rewriter::splitUReduce / splitUWrite, Rewriter.cc:603-663):
// smC is [LSU][BM][BN] accumulators; slice 0 is copied, slices 1..LSU-1 are added in order, and the
// sum is written to C with GLOB_STORE_WIDTH-wide vectors using the (non-)continuous map selected by
// REDUCE_C_CONTINUOUS (Optimizer.cc:241-282).
template <class C, int NT>
__device__ __forceinline__ void splitu_reduce_store(typename C::TC* __restrict__ Cm, const typename C::ACC* smC,
                                                    int tid, int m0, int n0) {
  typedef typename C::ACC ACC;
  constexpr int GSW = C::GSW;
  constexpr bool CONT = C::RC != 0 || (NT % C::BM != 0) || (C::BN % ((NT / C::BM) * GSW) != 0);
  typedef TileMap<C::BM, C::BN, GSW, NT, CONT> Map;
  constexpr bool ALIGNED = (C::N % GSW == 0);
#pragma unroll
  for (int it = 0; it < Map::ITERS; ++it) {
    int r, c;
    if (Map::coords(tid, it, r, c)) {
      ACC sum[GSW];
#pragma unroll
      for (int e = 0; e < GSW; ++e) sum[e] = smC[r * C::BN + c + e];
#pragma unroll
      for (int z = 1; z < C::LSU; ++z) {
#pragma unroll
        for (int e = 0; e < GSW; ++e) sum[e] += smC[(z * C::BM + r) * C::BN + c + e];
      }
      gstore<typename C::TC, ACC, GSW, C::EDGE, ALIGNED>(Cm, sum, m0 + r, n0 + c, C::N, C::M, C::N);
    }
  }
}

// =============================================================================================
// Family 1: SIMT kernel — the literal schedule.
// =============================================================================================
template <class C>
__device__ __forceinline__ void gemm_simt(const typename C::TA* __restrict__ A, const typename C::TB* __restrict__ B,
                                          typename C::TC* __restrict__ Cm, char* smem) {
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
      TA ra[2][TM];
      TB rb[2][TN];
      load_frag(stage, tz, ra[0], rb[0]);
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        if (s + 1 < KSTEPS) load_frag(stage, (s + 1) * LSU + tz, ra[(s + 1) & 1], rb[(s + 1) & 1]);
        fma_frag(ra[s & 1], rb[s & 1]);
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
    splitu_reduce_store<C, NT>(Cm, smC, tid, m0, n0);
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
              gstore<TC, ACC, C::TSW_B, EDGE, AL_C>(Cm, &acc[ri][rj], m0 + row, n0 + col, N, M, N);
            }
        }
  }
}

// =============================================================================================
// Family 2: MFMA kernel.
// =============================================================================================

// One matrix-core step on a 16-byte fragment pair.  For 4-byte inputs a fragment holds four k values
// and feeds four 32x32x2 (16x16x4) instructions; for 2-byte inputs it holds eight k values and feeds
// one 32x32x16 (16x16x32) instruction.  The k value a given (lane group, element) stands for is the
// same for the A and the B fragment, which is all the contraction needs.
template <class T, int MF> struct Mfma;

template <> struct Mfma<float, 32> {
  typedef floatx16 Acc;
  typedef floatx4 Frag;
  __device__ __forceinline__ static void run(Acc& c, const Frag& a, const Frag& b) {
#pragma unroll
    for (int t = 0; t < 4; ++t) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b[t], c, 0, 0, 0);
  }
  // accumulator tied in place, see the 16-bit variants below.  Four dependent instructions in a row on
  // one accumulator need no wait states between them (the compiler emits none for the builtin form either).
  __device__ __forceinline__ static void run_tied(Acc& c, const Frag& a, const Frag& b) {
#pragma unroll
    for (int t = 0; t < 4; ++t) asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+a"(c) : "v"(a[t]), "v"(b[t]));
  }
};
template <> struct Mfma<float, 16> {
  typedef floatx4 Acc;
  typedef floatx4 Frag;
  __device__ __forceinline__ static void run(Acc& c, const Frag& a, const Frag& b) {
#pragma unroll
    for (int t = 0; t < 4; ++t) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[t], b[t], c, 0, 0, 0);
  }
  // accumulator tied in place, see the 16-bit variants below.  Four dependent instructions in a row on
  // one accumulator need no wait states between them (the compiler emits none for the builtin form either).
  __device__ __forceinline__ static void run_tied(Acc& c, const Frag& a, const Frag& b) {
#pragma unroll
    for (int t = 0; t < 4; ++t) asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0" : "+a"(c) : "v"(a[t]), "v"(b[t]));
  }
};
// fp64: one instruction shape, 16x16x4 (lane: row/column lane%16, k = lane/16); a 16-byte chunk holds two
// consecutive k values, so a fragment step is two instructions
template <> struct Mfma<double, 16> {
  typedef doublex4 Acc;
  typedef doublex2 Frag;
  __device__ __forceinline__ static void run(Acc& c, const Frag& a, const Frag& b) {
#pragma unroll
    for (int t = 0; t < 2; ++t) c = __builtin_amdgcn_mfma_f64_16x16x4f64(a[t], b[t], c, 0, 0, 0);
  }
};
template <> struct Mfma<_Float16, 32> {
  typedef floatx16 Acc;
  typedef halfx8 Frag;
  __device__ __forceinline__ static void run(Acc& c, const Frag& a, const Frag& b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  // the same instruction with the accumulator tied to its own registers (accumulation registers):
  // left to itself the register allocator gives some of these instructions a fresh destination and
  // copies accumulators around the loop.  The compiler does not see a matrix-core instruction here:
  // the caller keeps dependent uses of c (as accumulator input or as plain data) far enough away.
  __device__ __forceinline__ static void run_tied(Acc& c, const Frag& a, const Frag& b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
template <> struct Mfma<_Float16, 16> {
  typedef floatx4 Acc;
  typedef halfx8 Frag;
  __device__ __forceinline__ static void run(Acc& c, const Frag& a, const Frag& b) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  // the same instruction with the accumulator tied to its own registers (accumulation registers):
  // left to itself the register allocator gives some of these instructions a fresh destination and
  // copies accumulators around the loop.  The compiler does not see a matrix-core instruction here:
  // the caller keeps dependent uses of c (as accumulator input or as plain data) far enough away.
  __device__ __forceinline__ static void run_tied(Acc& c, const Frag& a, const Frag& b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
template <> struct Mfma<__bf16, 32> {
  typedef floatx16 Acc;
  typedef bf16x8 Frag;
  __device__ __forceinline__ static void run(Acc& c, const Frag& a, const Frag& b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  // the same instruction with the accumulator tied to its own registers (accumulation registers):
  // left to itself the register allocator gives some of these instructions a fresh destination and
  // copies accumulators around the loop.  The compiler does not see a matrix-core instruction here:
  // the caller keeps dependent uses of c (as accumulator input or as plain data) far enough away.
  __device__ __forceinline__ static void run_tied(Acc& c, const Frag& a, const Frag& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
template <> struct Mfma<__bf16, 16> {
  typedef floatx4 Acc;
  typedef bf16x8 Frag;
  __device__ __forceinline__ static void run(Acc& c, const Frag& a, const Frag& b) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  // the same instruction with the accumulator tied to its own registers (accumulation registers):
  // left to itself the register allocator gives some of these instructions a fresh destination and
  // copies accumulators around the loop.  The compiler does not see a matrix-core instruction here:
  // the caller keeps dependent uses of c (as accumulator input or as plain data) far enough away.
  __device__ __forceinline__ static void run_tied(Acc& c, const Frag& a, const Frag& b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};

// LDS operand tile: rows (m or n) of CH 16-byte chunks (k).  The LDS of gfx950 has 64 dword banks, i.e.
// 16 bank groups of 16 bytes; a 128-bit access of a wave costs as many passes as the largest number
// of lanes (out of every 16) that meet in one group.  Chunk c of row r lives at chunk slot
// r*CH + (c ^ swz(r)); swz is chosen so that 16 consecutive rows at equal c (a fragment read) fall
// into 16 different groups.
template <int CH>
struct LdsTile {
  static constexpr int SMOD = cmin(16, lowbit(CH));
  static constexpr int RDIV = cmax(1, 16 / SMOD);
  __device__ __forceinline__ static int slot(int r, int c) { return r * CH + (c ^ ((r / RDIV) % SMOD)); }
};

// =============================================================================================
// Family 2b: matrix-core kernel with direct global->LDS staging (16-bit inputs).
//
// Every lane fetches one 16-byte chunk with global_load_lds_dwordx4; a wave's 64 chunks land in 1 KiB of
// consecutive LDS, so no register, no ds_write and no VALU work is spent on staging and the fetch of
// tile kt+2 can be in flight for a whole K tile.  The LDS image keeps the orientation of global memory:
//   k-contiguous operand  (A, IS_ATRANS=0): rows = m, CH = BK/8 chunks of 8 k values each; a fragment
//                                           is one ds_read_b128 (as in gemm_mfma)
//   row-contiguous operand (B; A^T)       : rows = k, NCH = BN/8 (BM/8) chunks of 8 n values each; a
//                                           fragment is two ds_read_b64_tr_b16: 16 lanes read a 4(k) x
//                                           16(n) block and each lane receives one column of it, which
//                                           is the k-packed layout the matrix core wants
// The bank swizzle is applied on the fetch side: the lane that fills physical chunk c' of a row fetches
// logical chunk c' ^ swz(row), and readers look chunk c up at c ^ swz(row).
// =============================================================================================
typedef short short4v __attribute__((ext_vector_type(4)));

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
  static constexpr bool FITS32 = WM % 32 == 0 && WN % 32 == 0;
  static constexpr int MF = KCG_DIRECT_MF ? KCG_DIRECT_MF
                            : ES == 2 ? ((C::BK % 32 == 0 || !FITS32) ? 16 : 32)
                                      : (FITS32 ? 32 : 16);       // fp32: no such difference, the larger tile reads less
  static constexpr int KS = G * (64 / MF);                        // k per step: one chunk per lane
  static constexpr int NW = C::BLM * C::BLN;
  static constexpr int NM = (WM / MF) * (WN / MF);
  static constexpr int SPW = (C::BK % KS == 0) ? C::BK / KS : 0;
  static constexpr bool pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }
  static constexpr bool ELIGIBLE =
      (ES == 2 || (ES == 4 && sizeof(typename C::TC) == 4)) && !C::EDGE && C::SHMP && C::REGP && C::LC != 0 &&
      C::LSU == 1 && C::GLW_A == G && C::GLW_B == G &&
      SPW > 0 && WM / MF >= 2 && pow2(C::BM) && pow2(C::BN) && pow2(C::BK) && C::BM >= 64 && C::BN >= 64 &&
      (C::BM * C::BK / G) % (64 * NW) == 0 && (C::BN * C::BK / G) % (64 * NW) == 0 && (C::M % G == 0) &&
      (C::N % G == 0) && (C::K % G == 0) && 2 * (C::BM + C::BN) * C::BK * ES <= 160 * 1024;
  // LDS stages: as many as fit in 160 KiB, at most 4 (fetch distance = NST-1 K tiles); an even number
  // when a tile is an odd number of k-steps (the B fragment double buffer alternates per step)
  static constexpr int STAGE_BYTES = (C::BM + C::BN) * C::BK * ES;
  static constexpr int NST_FIT = (160 * 1024) / STAGE_BYTES;
  // and no more than the fetch counter can tell apart: the wait for tile kt+1 allows the fetches of
  // NST-2 younger tiles in flight, and that counter has 6 bits
  static constexpr int NFETCH = ((C::BM + C::BN) * C::BK / G) / (64 * (NW > 0 ? NW : 1));   // per wave and tile
  static constexpr int NST_VM = 2 + 63 / (NFETCH > 0 ? NFETCH : 1);
  static constexpr int NST_MAX = NST_FIT < NST_VM ? NST_FIT : NST_VM;
  static constexpr int NST_CAP = NST_MAX < 2 ? 2 : (NST_MAX > 4 ? 4 : NST_MAX);
  static constexpr int NST = (SPW % 2 == 1 && NST_CAP % 2 == 1) ? NST_CAP - 1 : NST_CAP;
  // the host picks the path (it must size dynamic LDS accordingly); both sides have to agree
  static_assert(ELIGIBLE == C::DIRECT, "host and device disagree on the direct-staging eligibility rule");
  static constexpr bool OK = C::DIRECT;
};

template <class C>
__device__ __forceinline__ void gemm_mfma_direct(const typename C::TA* __restrict__ A, const typename C::TB* __restrict__ B,
                                                 typename C::TC* __restrict__ Cm, char* smem) {
  typedef typename C::TA T;
  typedef typename C::TC TC;
  typedef DirectPlan<C> P;
  constexpr int BM = C::BM, BN = C::BN, BK = C::BK;
  constexpr int M = C::M, N = C::N, K = C::K;
  constexpr int WM = P::WM, WN = P::WN, MF = P::MF;
  constexpr int KH = 64 / MF, KS = P::KS, SPW = P::SPW;
  constexpr int TMI = WM / MF, TNI = WN / MF, NM = P::NM, NW = P::NW;
  constexpr int KT = K / BK;
  constexpr bool AK = !C::ATRANS;                       // A is k-contiguous in global memory
  constexpr int ES = P::ES, G = P::G;                   // element size; elements per 16-byte chunk
  constexpr int CHK = BK / G;                           // chunks per row of a k-contiguous tile
  constexpr int NCHA = BM / G, NCHB = BN / G;           // chunks per row of a row-contiguous tile
  constexpr int A_BYTES = BM * BK * ES, B_BYTES = BN * BK * ES, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int NIA = (BM * BK / G) / (64 * NW);        // fetch instructions per wave and tile, operand A
  constexpr int NIB = (BN * BK / G) / (64 * NW);
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

  // One LDS array holds the NST stages.  (No LDS access of this kernel is visible to the compiler as a
  // load: otherwise it would have to assume that the load may touch a stage a fetch is in flight to
  // and drain all fetches in front of it.)
  constexpr int NST = P::NST;
  __shared__ __attribute__((aligned(1024))) char lds_all[NST * STAGE_BYTES];
  (void)smem;
  auto stage_ptr = [&](auto stage_c) -> char* { return lds_all + decltype(stage_c)::value * STAGE_BYTES; };

  // swizzle of a row-contiguous tile (chunk index ^= swz_n(row)).  16-bit: the rows that one pass of a
  // transposing read touches (k..k+3, and k+8..k+11 with 16-wide matrix-core tiles) must not share banks.
  // 32-bit: a fragment read is four 32-bit reads; in each, MF lanes read consecutive columns of one row
  // and the 64/MF lane groups read rows 4 apart, which must fall into different bank ranges.
  auto swz_n = [](int k, int nch) {
    if constexpr (ES == 2) return (((k & 3) << 2) ^ (((k >> 3) & 1) << 1)) & (nch - 1);
    else if constexpr (MF == 32) return (((k >> 2) & 1) << 3) & (nch - 1);
    else return (((k >> 2) & 3) << 2) & (nch - 1);
  };

  // ---- fetch: global -> LDS ------------------------------------------------------------------
  // Address = scalar tile base (advances with kt) + a 32-bit byte offset per lane and fetch item that
  // never changes: the K loop spends no vector instruction on addresses.
  static_assert((long)BM * K * ES < (1L << 31) && (long)BK * M * ES < (1L << 31) && (long)BK * N * ES < (1L << 31),
                "32-bit lane offsets");
  unsigned voff_a[NIA], voff_b[NIB];
#pragma unroll
  for (int idx = 0; idx < NIA; ++idx) {
    const int s = 64 * (wave * NIA + idx) + lane;     // physical chunk slot inside the A stage
    if constexpr (AK) {
      const int row = s / CHK, cp = s % CHK;
      const int c = cp ^ ((row / LK::RDIV) % LK::SMOD);
      voff_a[idx] = (unsigned)((row * K + c * G) * ES);
    } else {
      const int k = s / NCHA, cp = s % NCHA;
      const int c = cp ^ swz_n(k, NCHA);
      voff_a[idx] = (unsigned)((k * M + c * G) * ES);
    }
  }
#pragma unroll
  for (int j = 0; j < NIB; ++j) {
    const int s = 64 * (wave * NIB + j) + lane;
    const int k = s / NCHB, cp = s % NCHB;
    const int c = cp ^ swz_n(k, NCHB);
    voff_b[j] = (unsigned)((k * N + c * G) * ES);
  }
  const char* const a_base = (const char*)(AK ? A + (long)m0 * K : A + m0);
  const char* const b_base = (const char*)(B + n0);
  constexpr long A_KT_BYTES = AK ? (long)BK * ES : (long)BK * M * ES;   // one K tile further
  constexpr long B_KT_BYTES = (long)BK * N * ES;
  // The tile bases pass through an empty asm: the compiler must not fold the per-tile scalar part
  // into the per-lane part (it would hoist "base + lane offset" as a 64-bit vector value and add the
  // tile offset with vector instructions); kept apart, the fetch uses its scalar-base addressing form.
  struct TileBase { const char* a; const char* b; };
  auto tile_base = [&](int kt) {
    TileBase t = {a_base + kt * A_KT_BYTES, b_base + kt * B_KT_BYTES};
    asm("" : "+s"(t.a), "+s"(t.b));
    return t;
  };
  auto fetch_item = [&](int idx, const TileBase& tb, auto stage_c) {
    char* st = stage_ptr(stage_c);
    if (idx < NIA) {
      asm volatile("" : "+v"(voff_a[idx]));   // keeps the 32->64 bit extension next to the fetch (see tile_base)
      const char* src = tb.a + (unsigned long)voff_a[idx];
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(st + 1024 * (wave * NIA + idx)), 16, 0, 0);
    } else {
      const int j = idx - NIA;
      asm volatile("" : "+v"(voff_b[j]));
      const char* src = tb.b + (unsigned long)voff_b[j];
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(st + A_BYTES + 1024 * (wave * NIB + j)), 16, 0, 0);
    }
  };
  constexpr int NFETCH = NIA + NIB;

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
  struct FragTr {                                    // 16-bit, row-contiguous tile: two transposing 64-bit reads
    u32x2 h[2];
    __device__ __forceinline__ void pin() { asm volatile("" : "+v"(h[0]), "+v"(h[1])); }
    __device__ __forceinline__ Frag get() const {
      const u32x4 v = {h[0].x, h[0].y, h[1].x, h[1].y};
      return __builtin_bit_cast(Frag, v);
    }
  };
  struct FragS4 {                                    // 32-bit, row-contiguous tile: four 32-bit reads
    unsigned w[4];
    __device__ __forceinline__ void pin() { asm volatile("" : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3])); }
    __device__ __forceinline__ Frag get() const {
      const u32x4 v = {w[0], w[1], w[2], w[3]};
      return __builtin_bit_cast(Frag, v);
    }
  };
  struct FragLd {                                    // k-contiguous tile: one 128-bit read
    u32x4 q;
    __device__ __forceinline__ void pin() { asm volatile("" : "+v"(q)); }
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
  auto rc_lane_base = [&](int toff, int nch, int rowbase) {
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
  constexpr int NALANE = AK ? SPW : TMI;
  unsigned a_lane[NALANE];
  if constexpr (AK) {
#pragma unroll
    for (int st = 0; st < SPW; ++st)
      a_lane[st] = lds0 + (unsigned)(LK::slot(wy * WM + frow, st * KH + fgrp) * 16);   // swizzle: row%16 = frow%16 only
  } else {
#pragma unroll
    for (int i = 0; i < TMI; ++i) a_lane[i] = rc_lane_base(0, NCHA, wy * WM + i * MF);
  }
  auto split_base = [](unsigned lane_base, int imm) { return lane_base + (unsigned)(imm / 65536) * 65536u; };
  auto read_rc = [&](unsigned lane_base, auto imm_c, auto nch_c, FragRc* dst) {
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
  auto load_a = [&](auto stage_c, auto s_c, auto f_c, FragA* dst) {
    constexpr int ST = decltype(stage_c)::value, S = decltype(s_c)::value, F = decltype(f_c)::value;
    if constexpr (AK) {
      constexpr int IMM = ST * STAGE_BYTES + F * MF * CHK * 16;
      const unsigned base = split_base(a_lane[S], IMM);
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst->q) : "v"(base), "n"(IMM % 65536));
    } else {
      read_rc(a_lane[F], IntC<ST * STAGE_BYTES + S * KS * NCHA * 16>(), IntC<NCHA>(), dst);
    }
  };
  auto load_b = [&](auto stage_c, auto s_c, auto f_c, FragB* dst) {
    constexpr int ST = decltype(stage_c)::value, S = decltype(s_c)::value, F = decltype(f_c)::value;
    read_rc(b_lane[F], IntC<ST * STAGE_BYTES + S * KS * NCHB * 16>(), IntC<NCHB>(), dst);
  };
  // lgkmcnt(0): every LDS read issued so far has returned
  auto wait_lds = [&]() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); };

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
  typedef StreamPlan<TMI, TNI, DA, (AK ? 1 : RC_READS), RC_READS> SP;
  constexpr int RB = SP::RB;
  constexpr int MT = SPW * NM;
  constexpr int BAR = (SPW - 1) * NM + RB * TNI;
  constexpr int TAIL = MT - BAR;
  static_assert(TMI >= 2, "the streaming schedule needs two rows of matrix-core tiles per wave");
  static_assert((NST * SPW) % 2 == 0, "B double buffer: the parity of a step must follow from its stage");
  // s_waitcnt vmcnt(n), everything else unconstrained: n fetches of this wave may still be in flight
  static_assert((NST - 2) * NFETCH < 64, "vmcnt has 6 bits");
  auto vmcnt_only = [](int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); };
  auto tiles_ahead = [](int t) {
    const int last = cmin(KT - 1, t == 0 ? NST - 1 : t - 1 + NST);   // newest tile whose fetch has been issued
    return cmax(0, last - (t + 1));
  };

  // prologue: tile 0 -> stage 0, wait for it; then tiles 1..NST-1 in flight
#pragma unroll
  for (int i = 0; i < NFETCH; ++i) fetch_item(i, tile_base(0), IntC<0>());
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's chunks of tile 0 are in LDS
  __syncthreads();
  static_for<1, NST>([&](auto t) {
    if (decltype(t)::value < KT) {
#pragma unroll
      for (int i = 0; i < NFETCH; ++i) fetch_item(i, tile_base(decltype(t)::value), t);
    }
  });
  FragA fa[TMI];
  FragB fb[2][TNI];
  static_for<0, TNI>([&](auto j) { load_b(IntC<0>(), IntC<0>(), j, &fb[0][decltype(j)::value]); });
  static_for<0, DA>([&](auto i) { load_a(IntC<0>(), IntC<0>(), i, &fa[decltype(i)::value]); });
  wait_lds();   // the counted waits of the loop assume that nothing older than its own reads is in flight

  // One K tile.  CUR: the stage it computes from; H1: tile kt+1 exists; HN: tile kt+NST exists; HP: the
  // fetch of tile kt-1+NST, begun behind the previous tile's barrier, is still being issued.
  //
  // A stage is free once the barrier of the tile that computed from it has been passed, and the tile
  // fetched into it is needed NST-1 barriers later.  With three or more stages its NFETCH fetch
  // instructions are spread over the whole period up to the next barrier (the memory pipeline of a CU
  // takes 16 cycles per 1 KiB fetch instruction; four waves issuing all of theirs right behind the
  // barrier would stall on it); with two stages they must all be issued in the rest of this tile.
  constexpr int SPREAD = NST >= 3 ? MT : TAIL;
  auto tile = [&](int kt, auto cur_c, auto has1, auto hasn, auto hasp, auto ahead_c) {
    constexpr int CUR = decltype(cur_c)::value;
    constexpr int NXT = (CUR + 1) % NST, PRV = (CUR + NST - 1) % NST;
    constexpr bool H1 = decltype(has1)::value, HN = decltype(hasn)::value;
    constexpr bool HP = decltype(hasp)::value && SPREAD > TAIL;
    const TileBase tbn = tile_base(HN ? kt + NST : 0);
    const TileBase tbp = tile_base(HP ? kt - 1 + NST : 0);
    static_for<0, SPW>([&](auto s_c) {
      constexpr int S = decltype(s_c)::value;
      constexpr bool LAST = (S == SPW - 1);
      constexpr int PB = (CUR * SPW + S) & 1;       // half of the B double buffer this step computes from
      constexpr bool NEXT = !LAST || H1;            // a next step exists, its fragments are read under this one
      static_for<0, TMI>([&](auto i_c) {
        constexpr int I = decltype(i_c)::value;
        // the fragments of this row have arrived.  Without a next step the reads the count relies on
        // are not issued: wait for everything instead.
        if constexpr (NEXT) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(SP::allowed(I)) : "memory");
        else wait_lds();
        if constexpr (LAST && I == RB) {
          // tile kt+1 has landed (this wave's part): of the fetches issued so far only those of the
          // tiles behind it may still be in flight
          if constexpr (H1) __builtin_amdgcn_s_waitcnt(vmcnt_only(decltype(ahead_c)::value * NFETCH));
          wait_lds();        // this wave's reads of stage CUR have all returned
          // ... everyone's part; and every wave is done reading stage CUR.  The bare barrier instruction:
          // __syncthreads() comes with a fence in front of which the compiler drains every fetch in
          // flight (vmcnt(0)), which would expose the whole memory latency at each tile.  What has
          // to be complete at this point is exactly what the two waits above ask for.
          asm volatile("" ::: "memory");
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
        }
        // the empty asm statements make the fragments "outputs" of the wait: the matrix-core
        // instructions that consume them cannot be scheduled in front of it
        fa[I].pin();
        if constexpr (I == 0) {
#pragma unroll
          for (int j = 0; j < TNI; ++j) fb[PB][j].pin();
        }
        if constexpr (I + DA < TMI) load_a(IntC<CUR>(), IntC<S>(), IntC<I + DA>(), &fa[I + DA]);
        else if constexpr (!LAST) load_a(IntC<CUR>(), IntC<S + 1>(), IntC<I + DA - TMI>(), &fa[I + DA - TMI]);
        else if constexpr (H1) load_a(IntC<NXT>(), IntC<0>(), IntC<I + DA - TMI>(), &fa[I + DA - TMI]);
        static_for<0, TNI>([&](auto j_c) {
          constexpr int J = decltype(j_c)::value;
          constexpr int slot = S * NM + I * TNI + J;
          // operands swapped (B fragment first): the accumulator then holds C^T tiles, i.e. each lane owns
          // one row m and groups of four consecutive n, which the epilogue stores as 128-bit vectors
          // odd rows run right to left: neighbours on the time line always share one operand
          constexpr int JC = (I & 1) ? TNI - 1 - J : J;
          MI::run_tied(acc[I][JC], fb[PB][JC].get(), fa[I].get());
          static_for<0, TNI>([&](auto jj_c) {
            constexpr int JJ = decltype(jj_c)::value;
            if constexpr (SP::slot_b(JJ) == I * TNI + J) {
              if constexpr (!LAST) load_b(IntC<CUR>(), IntC<S + 1>(), jj_c, &fb[PB ^ 1][JJ]);
              else if constexpr (H1) load_b(IntC<NXT>(), IntC<0>(), jj_c, &fb[PB ^ 1][JJ]);
            }
          });
#pragma unroll
          for (int f = 0; f < NFETCH; ++f) {
            const int pos = BAR + (f * SPREAD) / NFETCH;          // position on the time line that starts at this tile
            if (HN && pos == slot) fetch_item(f, tbn, IntC<CUR>());
            if (HP && pos - MT == slot) fetch_item(f, tbp, IntC<PRV>());
          }
          __builtin_amdgcn_sched_barrier(0);
        });
      });
    });
  };
  // Tile 0 first (nothing of an earlier period to continue); then groups of NST tiles that have every
  // neighbour; the rest is unrolled with the right flags at compile time (KT is a constant).
  // tiles_ahead(T): how many tiles behind tile T+1 have been issued when tile T reaches its barrier
  // (the prologue issued tiles 0..NST-1, tile t issues or completes the issue of tile t-1+NST)
  tile(0, IntC<0>(), BoolC<(1 < KT)>(), BoolC<(NST < KT)>(), BoolC<false>(), IntC<tiles_ahead(0)>());
  constexpr int NFULL = KT - NST - 1 > 0 ? KT - NST - 1 : 0;   // tiles 1 .. KT-NST-1 have kt+NST < KT
  constexpr int NG = NFULL / NST;
  for (int g = 0; g < NG; ++g) {
    static_for<0, NST>([&](auto sc) {
      constexpr int S = decltype(sc)::value;
      tile(1 + g * NST + S, IntC<(1 + S) % NST>(), BoolC<true>(), BoolC<true>(), BoolC<true>(), IntC<NST - 2>());
    });
  }
  static_for<1 + NG * NST, KT>([&](auto tc) {
    constexpr int T = decltype(tc)::value;
    tile(T, IntC<T % NST>(), BoolC<(T + 1 < KT)>(), BoolC<(T + NST < KT)>(), BoolC<(T - 1 + NST < KT)>(), IntC<tiles_ahead(T)>());
  });

  // the last matrix-core results must have left the pipeline before the epilogue reads them (the
  // compiler, which normally inserts these wait states, does not know the instructions above)
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  // ---- epilogue --------------------------------------------------------------------------------
  // With swapped operands a 32x32 accumulator holds, per lane, row m = lane%32 and columns
  // n = 8*g + 4*(lane/32) + {0..3} for g = 0..3 (16x16: row lane%16, columns 4*(lane/16) + {0..3}).
  constexpr int NACC = (int)(sizeof(Acc) / sizeof(float));
  const int orow = lane % MF;
  const int ocol = (lane / MF) * 4;
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j)
#pragma unroll
      for (int g = 0; g < NACC / 4; ++g) {
        const int row = m0 + wy * WM + i * MF + orow;
        const int col = n0 + wx * WN + j * MF + g * 8 + ocol;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][g * 4 + e];
        gstore<TC, float, 4, false, true>(Cm, v, row, col, N, M, N);
      }
}

template <class C>
__device__ __forceinline__ void gemm_mfma(const typename C::TA* __restrict__ A, const typename C::TB* __restrict__ B,
                                          typename C::TC* __restrict__ Cm, char* smem) {
  if constexpr (DirectPlan<C>::OK) {
    gemm_mfma_direct<C>(A, B, Cm, smem);
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
#pragma unroll
        for (int s = 0; s < SPW; ++s) {
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
        }
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
#pragma unroll
        for (int s = 0; s < SPW; ++s) {
          if (s + 1 < SPW) load_frag(0, (s + 1) * LSU + wz, fa[(s + 1) & 1], fb[(s + 1) & 1]);
          mma_frag(fa[s & 1], fb[s & 1]);
        }
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
    splitu_reduce_store<C, NT>(Cm, smC, tid, m0, n0);
  } else {
#pragma unroll
    for (int i = 0; i < TMI; ++i)
#pragma unroll
      for (int j = 0; j < TNI; ++j)
#pragma unroll
        for (int e = 0; e < NACC; ++e) {
          const int row = m0 + wy * WM + i * MF + acc_row(e);
          const int col = n0 + wx * WN + j * MF + ocol;
          if (!EDGE || (row < M && col < N)) Cm[(long)row * N + col] = (TC)acc[i][j][e];
        }
  }
}

}  // namespace kcg
