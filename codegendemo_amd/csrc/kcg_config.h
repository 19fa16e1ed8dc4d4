// kcg_config.h — host-side meaning of the 31-integer KCG matmul tuning config: named fields, derived
// quantities, validity predicates, kernel name, launch geometry, LDS bytes and the block swizzle.
// Pure C++17, no HIP: usable from CPU-only tests.
#pragma once
#include <cstdint>
#include <string>

#include "../../include/kcg_gemm.h"

namespace kcg {

// Named view of kcg_matmul_cfg (argument order of src/main.cc:64-96).
struct MatmulConfig {
  int BM, BN, BK, TM, TN, WARP_SIZE, BLM, BLN, WLM, WLN;
  int GLW_A, GLW_B, WSW_A, WSW_B, TSW_A, TSW_B, LSU, BLOCK_MAPPING, GSW;
  int UNROLL, REGP, SHMP, LC, RC;
  int dtA, dtB, dtC;
  int M, N, K;
  int ATRANS;

  static MatmulConfig from(const kcg_matmul_cfg& c);
  kcg_matmul_cfg raw() const;

  // MatmulConfigUtils (Optimizer.cc:10-36)
  int block_x() const { return BN / TN; }
  int block_y() const { return BM / TM; }
  int thread_num() const { return block_x() * block_y() * LSU; }
  int grid_y() const { return (M + BM - 1) / BM; }
  int grid_x() const { return (N + BN - 1) / BN; }
  bool edge() const { return (M % BM) || (N % BN) || (K % BK); }
};

const char* dtype_name(int dt);  // "float32" … as KcgDtypeToStr (src/lib/Common/Utils.cc:146-162)
const char* dtype_ctype(int dt); // HIP element type spelled in the instantiation stub
int dtype_size(int dt);

// MFMA tiling the wave tile resolves to; valid only if ok.
struct MfmaPlan {
  bool ok = false;
  int WM = 0, WN = 0;  // wave tile
  int MF = 0;          // 32 or 16
  int G = 0;           // k elements per 16-byte LDS chunk
  int KS = 0;          // k covered by one fragment step
  std::string why;     // reason when !ok
};
MfmaPlan plan_mfma(const MatmulConfig& c);

// Reasons are human-readable; empty string == valid.
std::string check_common(const MatmulConfig& c);
std::string check_simt(const MatmulConfig& c);
std::string check_mfma(const MatmulConfig& c);

std::string kernel_name(const MatmulConfig& c);
int reference_lds_bytes(const MatmulConfig& c);
int simt_pad_a(const MatmulConfig& c);
bool mfma_direct(const MatmulConfig& c);      // matrix-core kernel stages operands with direct global->LDS loads
int lds_bytes(const MatmulConfig& c, int kind, bool allow_direct = true);  // what the chosen kernel really needs
void block_mapping(const MatmulConfig& c, int bid, bool xcd_remap, int* by, int* bx);

int num_cus();    // compute units / XCDs of the (partition of the) GPU the kernels are built for: 256 / 8,
int num_xcds();   // or $KCG_NUM_CUS / $KCG_NUM_XCDS

// HIP text of the instantiation stub for (config, kind, xcd_remap).  ex < 0: the reference's kernel form (three
// pointers); ex = 0 / 1: the batched-strided form, without / with the alpha-beta epilogue (kernel_name_ex).
std::string instantiation_source(const MatmulConfig& c, int kind, bool xcd_remap, bool allow_direct = true, int ex = -1);
std::string kernel_name_ex(const MatmulConfig& c, int epilogue);

constexpr int kMaxLdsBytes = 160 * 1024;  // gfx950: 160 KiB LDS per CU, one workgroup may take all
constexpr int kMaxThreads = 1024;

}  // namespace kcg
