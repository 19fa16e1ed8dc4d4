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
// Kernel families (one header each):
//   gemm_simt : scalar-FMA register-tiled kernel that follows the tuning config literally
//               (thread tile TMxTN, warp/lane scatter, split-U across thread-z, optional LDS and
//               register double buffering).  It is the fallback for configs whose wave tile cannot
//               be covered by matrix-core tiles.
//   gemm_mfma : wave-tiled matrix-core kernel (v_mfma_f32_32x32x2_f32 / 16x16x4_f32,
//               v_mfma_f32_32x32x16_{f16,bf16} / 16x16x32_{f16,bf16}); operands are staged in LDS
//               as [row][k] with 16-byte chunks XOR-swizzled so that every fragment is a single
//               conflict-free ds_read_b128 (kcg_device_mfma.h); configs with both prefetch flags,
//               LOAD_CONTINUOUS and 128-bit loads run gemm_mfma_direct (kcg_device_direct.h): operands
//               go global -> LDS directly and the K loop is scheduled by hand.
//
// No host headers are available under hiprtc; only compiler builtins are used.
#pragma once

#include "kcg_device_common.h"
#include "kcg_device_simt.h"
#include "kcg_device_mfma_ops.h"
#include "kcg_device_direct.h"
#include "kcg_device_mfma.h"
