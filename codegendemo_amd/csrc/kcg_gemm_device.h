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
};
template <> struct Mfma<float, 16> {
  typedef floatx4 Acc;
  typedef floatx4 Frag;
  __device__ __forceinline__ static void run(Acc& c, const Frag& a, const Frag& b) {
#pragma unroll
    for (int t = 0; t < 4; ++t) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[t], b[t], c, 0, 0, 0);
  }
};
template <> struct Mfma<_Float16, 32> {
  typedef floatx16 Acc;
  typedef halfx8 Frag;
  __device__ __forceinline__ static void run(Acc& c, const Frag& a, const Frag& b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma<_Float16, 16> {
  typedef floatx4 Acc;
  typedef halfx8 Frag;
  __device__ __forceinline__ static void run(Acc& c, const Frag& a, const Frag& b) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma<__bf16, 32> {
  typedef floatx16 Acc;
  typedef bf16x8 Frag;
  __device__ __forceinline__ static void run(Acc& c, const Frag& a, const Frag& b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma<__bf16, 16> {
  typedef floatx4 Acc;
  typedef bf16x8 Frag;
  __device__ __forceinline__ static void run(Acc& c, const Frag& a, const Frag& b) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

// LDS operand tile: ROWS rows (m or n) of CH 16-byte chunks (k).  Chunk c of row r lives at chunk
// slot r*CH + (c ^ swz(r)); swz makes 8 consecutive rows hit 8 different 16-byte bank groups.
template <int CH>
struct LdsTile {
  static constexpr int SMOD = cmin(8, lowbit(CH));
  static constexpr int RDIV = cmax(1, 8 / SMOD);
  __device__ __forceinline__ static int slot(int r, int c) { return r * CH + (c ^ ((r / RDIV) % SMOD)); }
};

template <class C>
__device__ __forceinline__ void gemm_mfma(const typename C::TA* __restrict__ A, const typename C::TB* __restrict__ B,
                                          typename C::TC* __restrict__ Cm, char* smem) {
  typedef typename C::TA T;   // TA == TB for this family
  typedef typename C::TC TC;
  constexpr int BM = C::BM, BN = C::BN, BK = C::BK, LSU = C::LSU;
  constexpr int M = C::M, N = C::N, K = C::K;
  constexpr int ES = (int)sizeof(T);
  constexpr int G = 16 / ES;                  // k elements per 16-byte chunk
  constexpr int WM = BM / C::BLM, WN = BN / C::BLN;   // wave tile = (WLM*TM) x (WLN*TN)
  constexpr int MF = (WM % 32 == 0 && WN % 32 == 0) ? 32 : 16;
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
  typedef TileMap<CH, BM, VN_A, NT, true> MapNA;
  typedef TileMap<CH, BN, VN_B, NT, true> MapNB;
  constexpr int ITERS_A = C::ATRANS ? MapNA::ITERS : MapKA::ITERS;
  constexpr int REGS_A = C::ATRANS ? G * VN_A : G;
  constexpr bool AL_A = C::ATRANS ? (M % VN_A == 0) : (K % VK_A == 0);
  constexpr bool AL_B = (N % VN_B == 0);

  T ga[ITERS_A][REGS_A];
  T gb[MapNB::ITERS][G * VN_B];

  auto load_global = [&](int kt) {
    const int k0 = kt * BK;
#pragma unroll
    for (int it = 0; it < ITERS_A; ++it) {
      int r, c;
      if constexpr (C::ATRANS) {
        if (MapNA::coords(tid, it, r, c)) {   // r = k chunk, c = first m of the vector
#pragma unroll
          for (int g = 0; g < G; ++g)
            gload<T, VN_A, EDGE, AL_A>(&ga[it][g * VN_A], A, k0 + r * G + g, m0 + c, M, K, M);
        }
      } else {
        if (MapKA::coords(tid, it, r, c)) {   // r = m row, c = first k of the chunk
#pragma unroll
          for (int v = 0; v < G / VK_A; ++v)
            gload<T, VK_A, EDGE, AL_A>(&ga[it][v * VK_A], A, m0 + r, k0 + c + v * VK_A, K, M, K);
        }
      }
    }
#pragma unroll
    for (int it = 0; it < MapNB::ITERS; ++it) {
      int r, c;
      if (MapNB::coords(tid, it, r, c)) {
#pragma unroll
        for (int g = 0; g < G; ++g)
          gload<T, VN_B, EDGE, AL_B>(&gb[it][g * VN_B], B, k0 + r * G + g, n0 + c, N, K, N);
      }
    }
  };
  auto store_lds = [&](int stage) {
    u32x4* sa = smA + stage * BM * CH;
    u32x4* sb = smB + stage * BN * CH;
#pragma unroll
    for (int it = 0; it < ITERS_A; ++it) {
      int r, c;
      if constexpr (C::ATRANS) {
        if (MapNA::coords(tid, it, r, c)) {
#pragma unroll
          for (int e = 0; e < VN_A; ++e) {
            T chunk[G];
#pragma unroll
            for (int g = 0; g < G; ++g) chunk[g] = ga[it][g * VN_A + e];
            copy_bytes<16>(sa + L::slot(c + e, r), chunk);
          }
        }
      } else {
        if (MapKA::coords(tid, it, r, c)) copy_bytes<16>(sa + L::slot(r, c / G), ga[it]);
      }
    }
#pragma unroll
    for (int it = 0; it < MapNB::ITERS; ++it) {
      int r, c;
      if (MapNB::coords(tid, it, r, c)) {
#pragma unroll
        for (int e = 0; e < VN_B; ++e) {
          T chunk[G];
#pragma unroll
          for (int g = 0; g < G; ++g) chunk[g] = gb[it][g * VN_B + e];
          copy_bytes<16>(sb + L::slot(c + e, r), chunk);
        }
      }
    }
  };

  // ---- fragments and matrix-core steps -------------------------------------------------------
  Acc acc[TMI][TNI];
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j)
#pragma unroll
      for (int e = 0; e < (int)(sizeof(Acc) / sizeof(float)); ++e) acc[i][j][e] = 0.0f;

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
  auto mma_frag = [&](const Frag* fa, const Frag* fb) {
#pragma unroll
    for (int i = 0; i < TMI; ++i)
#pragma unroll
      for (int j = 0; j < TNI; ++j) MI::run(acc[i][j], fa[i], fb[j]);
  };

  constexpr int SPW = NSS / LSU;   // fragment steps of one tile handled by this wave's split-U slice
  auto compute_tile = [&](int stage) {
    if constexpr (C::REGP) {
      Frag fa[2][TMI], fb[2][TNI];
      load_frag(stage, wz, fa[0], fb[0]);
#pragma unroll
      for (int s = 0; s < SPW; ++s) {
        if (s + 1 < SPW) load_frag(stage, (s + 1) * LSU + wz, fa[(s + 1) & 1], fb[(s + 1) & 1]);
        mma_frag(fa[s & 1], fb[s & 1]);
      }
    } else {
      Frag fa[TMI], fb[TNI];
#pragma unroll
      for (int s = 0; s < SPW; ++s) {
        load_frag(stage, s * LSU + wz, fa, fb);
        mma_frag(fa, fb);
      }
    }
  };

  // ---- K loop ---------------------------------------------------------------------------------
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
  // Accumulator layout of a 32x32 tile: lane holds column lane%32, rows 8*(e/4) + 4*(lane/32) + e%4
  // for e in 0..15; of a 16x16 tile: column lane%16, rows 4*(lane/16) + e for e in 0..3.
  constexpr int NACC = (int)(sizeof(Acc) / sizeof(float));
  const int ocol = lane % MF;
  const int orow = (lane / MF) * 4;
  if constexpr (LSU > 1) {
    float* smC = reinterpret_cast<float*>(smem);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TMI; ++i)
#pragma unroll
      for (int j = 0; j < TNI; ++j)
#pragma unroll
        for (int e = 0; e < NACC; ++e) {
          const int row = wy * WM + i * MF + (e / 4) * 8 + orow + e % 4;
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
          const int row = m0 + wy * WM + i * MF + (e / 4) * 8 + orow + e % 4;
          const int col = n0 + wx * WN + j * MF + ocol;
          if (!EDGE || (row < M && col < N)) Cm[(long)row * N + col] = (TC)acc[i][j][e];
        }
  }
}

}  // namespace kcg
