// kcg_device_mfma_ops.h — matrix-core instruction wrappers (one fragment step per call) and the swizzled LDS
// operand tile used by both matrix-core kernels.
#pragma once
#include "kcg_device_common.h"

namespace kcg {

// =============================================================================================
// Matrix-core building blocks shared by gemm_mfma and gemm_mfma_direct.
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
  __host__ __device__ __forceinline__ static int slot(int r, int c) { return r * CH + (c ^ ((r / RDIV) % SMOD)); }
};

}  // namespace kcg
