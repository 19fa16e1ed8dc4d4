// kcg_device_common.h — vector types, compile-time helpers, block scheduling, global load/store helpers
// and the split-U reduce shared by all kernel families of kcg_gemm_device.h.
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

// Raw 1..16-byte carriers for copy_bytes.  They are declared may_alias: copy_bytes moves floats, halves
// and doubles through them, and without the attribute the compiler is entitled to assume that a store
// through `unsigned int` cannot change a `float` object (type-based alias analysis) and to reorder the
// typed accesses around the copy.
template <int BYTES> struct RawVec;
template <> struct RawVec<1> { typedef unsigned char type; };
template <> struct RawVec<2> { typedef unsigned short __attribute__((may_alias)) type; };
template <> struct RawVec<4> { typedef unsigned int __attribute__((may_alias)) type; };
template <> struct RawVec<8> { typedef u32x2 __attribute__((may_alias)) type; };
template <> struct RawVec<16> { typedef u32x4 __attribute__((may_alias)) type; };

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
// The same where the addresses are aligned to ALIGN bytes only (ALIGN < NBYTES): still one access.  Global memory
// takes vector accesses at element alignment; rows of C whose length is not a multiple of the vector are the case.
template <int NBYTES, int ALIGN>
__device__ __forceinline__ void copy_bytes_unaligned(void* dst, const void* src) {
  typedef typename RawVec<NBYTES>::type V;
  typedef V __attribute__((aligned(ALIGN))) VU;
  *reinterpret_cast<VU*>(dst) = *reinterpret_cast<const VU*>(src);
}
// the same with a non-temporal store (streaming data that the kernel does not read again)
template <int NBYTES>
__device__ __forceinline__ void copy_bytes_nt(void* dst, const void* src) {
  typedef typename RawVec<NBYTES>::type V;
  __builtin_nontemporal_store(*reinterpret_cast<const V*>(src), reinterpret_cast<V*>(dst));
}

// ---------------------------------------------------------------------------------------------
// Block id -> (by, bx).  Rewriter::BlockMapping (Rewriter.cc:726-761): groups of BLOCK_MAPPING block
// rows are walked column by column so that concurrently resident blocks share B panels in L2.
// On top of it, when the block count is a multiple of the number of XCDs (C::NUM_XCD, 8 on an MI355X),
// consecutive hardware ids (which the dispatcher deals round-robin to the XCDs, each with a private L2)
// are remapped so that every XCD walks one contiguous part of that order.
// ---------------------------------------------------------------------------------------------
template <class C>
__device__ __forceinline__ void block_coords(int bid, int& by, int& bx) {
  constexpr int GY = cdiv(C::M, C::BM);
  constexpr int GX = cdiv(C::N, C::BN);
  constexpr int NB = GY * GX;
  constexpr int NX = C::NUM_XCD;
  if constexpr (C::XCD_REMAP && NX > 1 && (NB % NX == 0)) {
    bid = (bid % NX) * (NB / NX) + bid / NX;
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
// every such vector is naturally aligned to VEC*sizeof(T) so one wide load is legal: LD (which is CMAX
// at every call site, the matrices being dense) and c are multiples of VEC.
template <class T, int VEC, bool EDGE, bool ALIGNED>
__device__ __forceinline__ void gload(T* dst, const T* __restrict__ base, int r, int c, int LD, int RMAX, int CMAX) {
  if constexpr (!EDGE) {
    if constexpr (ALIGNED) {
      copy_bytes<VEC * (int)sizeof(T)>(dst, base + (long)r * LD + c);
    } else {
      copy_bytes_unaligned<VEC * (int)sizeof(T), (int)sizeof(T)>(dst, base + (long)r * LD + c);
    }
  } else if constexpr (ALIGNED) {
    // c and CMAX are multiples of VEC: the vector lies inside or outside as a whole.  No branch: a lane
    // whose vector lies outside loads element 0 of the matrix instead and then drops it.
    const bool in = r < RMAX && c < CMAX;
    copy_bytes<VEC * (int)sizeof(T)>(dst, base + (in ? (long)r * LD + c : 0L));
#pragma unroll
    for (int e = 0; e < VEC; ++e) dst[e] = in ? dst[e] : T(0);
  } else if constexpr (VEC == 1) {
    const bool in = r < RMAX && c < CMAX;
    const T v = base[in ? (long)r * LD + c : 0L];
    dst[0] = in ? v : T(0);
  } else {
    // rows that do not start on vector boundaries: a vector that lies inside its row is still one access (at element
    // alignment, branch-free like the aligned case); only the vector across the end of a row goes element by element
    const bool whole = r < RMAX && c + VEC <= CMAX;
    copy_bytes_unaligned<VEC * (int)sizeof(T), (int)sizeof(T)>(dst, base + (whole ? (long)r * LD + c : 0L));
    if (!whole) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const bool in = r < RMAX && c + e < CMAX;
        const T v = base[in ? (long)r * LD + c + e : 0L];
        dst[e] = in ? v : T(0);
      }
    }
  }
}

// Store VEC consecutive output elements (converted from the accumulator type) with the same rules.
template <class TC, class ACC, int VEC, bool EDGE, bool ALIGNED, bool NT = false>
__device__ __forceinline__ void gstore(TC* __restrict__ base, const ACC* src, int r, int c, int LD, int RMAX, int CMAX) {
  TC tmp[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) tmp[e] = (TC)src[e];
  if constexpr (!EDGE) {
    if constexpr (ALIGNED && NT) {
      copy_bytes_nt<VEC * (int)sizeof(TC)>(base + (long)r * LD + c, tmp);
    } else if constexpr (ALIGNED) {
      copy_bytes<VEC * (int)sizeof(TC)>(base + (long)r * LD + c, tmp);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) base[(long)r * LD + c + e] = tmp[e];
    }
  } else if constexpr (ALIGNED) {
    if (r < RMAX && c < CMAX) copy_bytes<VEC * (int)sizeof(TC)>(base + (long)r * LD + c, tmp);
  } else {
    // a vector that lies inside the row goes out as one access at element alignment; the one across the end of
    // the row element by element
    if (VEC > 1 && r < RMAX && c + VEC <= CMAX) {
      copy_bytes_unaligned<VEC * (int)sizeof(TC), (int)sizeof(TC)>(base + (long)r * LD + c, tmp);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        if (r < RMAX && c + e < CMAX) base[(long)r * LD + c + e] = tmp[e];
    }
  }
}

// Epilogue C = alpha * (A B) + beta * C (the call shape of the vendor sgemm the reference profiles against,
// runRoc.cpp:27-28,53-66), compiled in only when the instantiation asks for it (C::EPI).  As in BLAS, beta == 0
// means that C is not read at all (whatever it held, NaN included, does not reach the result).
struct EpiArgs {
  float alpha, beta;
};
template <class TC, class ACC, int VEC, bool EDGE, bool ALIGNED>
__device__ __forceinline__ void epi_apply(ACC* v, const TC* base, int r, int c, int LD, int RMAX, int CMAX, EpiArgs ep) {
  const ACC alpha = (ACC)ep.alpha, beta = (ACC)ep.beta;
  if (ep.beta != 0.f) {
    TC old[VEC];
    gload<TC, VEC, EDGE, ALIGNED>(old, base, r, c, LD, RMAX, CMAX);
#pragma unroll
    for (int e = 0; e < VEC; ++e) v[e] = alpha * v[e] + beta * (ACC)old[e];
  } else {
#pragma unroll
    for (int e = 0; e < VEC; ++e) v[e] = alpha * v[e];
  }
}

// Split-U epilogue shared by both families (Rewriter::splitUReduce / splitUWrite, Rewriter.cc:603-663):
// smC is [LSU][BM][BN] accumulators; slice 0 is copied, slices 1..LSU-1 are added in order, and the
// sum is written to C with GLOB_STORE_WIDTH-wide vectors using the (non-)continuous map selected by
// REDUCE_C_CONTINUOUS (Optimizer.cc:241-282).
template <class C, int NT>
__device__ __forceinline__ void splitu_reduce_store(typename C::TC* __restrict__ Cm, const typename C::ACC* smC,
                                                    int tid, int m0, int n0, EpiArgs ep) {
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
      if constexpr (C::EPI) epi_apply<typename C::TC, ACC, GSW, C::EDGE, ALIGNED>(sum, Cm, m0 + r, n0 + c, C::N, C::M, C::N, ep);
      gstore<typename C::TC, ACC, GSW, C::EDGE, ALIGNED>(Cm, sum, m0 + r, n0 + c, C::N, C::M, C::N);
    }
  }
}

}  // namespace kcg
