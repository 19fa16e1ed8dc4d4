// kcg_config.cc — see kcg_config.h.
#include "kcg_config.h"

#include <cstdlib>
#include <sstream>

namespace kcg {

MatmulConfig MatmulConfig::from(const kcg_matmul_cfg& r) {
  MatmulConfig c;
  const int32_t* v = r.v;
  c.BM = v[KCG_BLOCK_SIZE_M]; c.BN = v[KCG_BLOCK_SIZE_N]; c.BK = v[KCG_BLOCK_SIZE_K];
  c.TM = v[KCG_THREAD_SIZE_M]; c.TN = v[KCG_THREAD_SIZE_N]; c.WARP_SIZE = v[KCG_WARP_SIZE];
  c.BLM = v[KCG_BLOCK_LAYOUT_M]; c.BLN = v[KCG_BLOCK_LAYOUT_N];
  c.WLM = v[KCG_WARP_LAYOUT_M]; c.WLN = v[KCG_WARP_LAYOUT_N];
  c.GLW_A = v[KCG_GLOB_LOAD_WIDTH_A]; c.GLW_B = v[KCG_GLOB_LOAD_WIDTH_B];
  c.WSW_A = v[KCG_WARP_SCATTER_WIDTH_A]; c.WSW_B = v[KCG_WARP_SCATTER_WIDTH_B];
  c.TSW_A = v[KCG_THREAD_SCATTER_WIDTH_A]; c.TSW_B = v[KCG_THREAD_SCATTER_WIDTH_B];
  c.LSU = v[KCG_LOCAL_SPLIT_U]; c.BLOCK_MAPPING = v[KCG_BLOCK_MAPPING]; c.GSW = v[KCG_GLOB_STORE_WIDTH];
  c.UNROLL = v[KCG_UNROLL_NUM]; c.REGP = v[KCG_REG_PREFETCH]; c.SHMP = v[KCG_SHARED_PREFETCH];
  c.LC = v[KCG_LOAD_CONTINUOUS]; c.RC = v[KCG_REDUCE_C_CONTINUOUS];
  c.dtA = v[KCG_DTYPE_A]; c.dtB = v[KCG_DTYPE_B]; c.dtC = v[KCG_DTYPE_C];
  c.M = v[KCG_M]; c.N = v[KCG_N]; c.K = v[KCG_K];
  c.ATRANS = v[KCG_IS_ATRANS];
  return c;
}

kcg_matmul_cfg MatmulConfig::raw() const {
  kcg_matmul_cfg r;
  int32_t* v = r.v;
  v[KCG_BLOCK_SIZE_M] = BM; v[KCG_BLOCK_SIZE_N] = BN; v[KCG_BLOCK_SIZE_K] = BK;
  v[KCG_THREAD_SIZE_M] = TM; v[KCG_THREAD_SIZE_N] = TN; v[KCG_WARP_SIZE] = WARP_SIZE;
  v[KCG_BLOCK_LAYOUT_M] = BLM; v[KCG_BLOCK_LAYOUT_N] = BLN;
  v[KCG_WARP_LAYOUT_M] = WLM; v[KCG_WARP_LAYOUT_N] = WLN;
  v[KCG_GLOB_LOAD_WIDTH_A] = GLW_A; v[KCG_GLOB_LOAD_WIDTH_B] = GLW_B;
  v[KCG_WARP_SCATTER_WIDTH_A] = WSW_A; v[KCG_WARP_SCATTER_WIDTH_B] = WSW_B;
  v[KCG_THREAD_SCATTER_WIDTH_A] = TSW_A; v[KCG_THREAD_SCATTER_WIDTH_B] = TSW_B;
  v[KCG_LOCAL_SPLIT_U] = LSU; v[KCG_BLOCK_MAPPING] = BLOCK_MAPPING; v[KCG_GLOB_STORE_WIDTH] = GSW;
  v[KCG_UNROLL_NUM] = UNROLL; v[KCG_REG_PREFETCH] = REGP; v[KCG_SHARED_PREFETCH] = SHMP;
  v[KCG_LOAD_CONTINUOUS] = LC; v[KCG_REDUCE_C_CONTINUOUS] = RC;
  v[KCG_DTYPE_A] = dtA; v[KCG_DTYPE_B] = dtB; v[KCG_DTYPE_C] = dtC;
  v[KCG_M] = M; v[KCG_N] = N; v[KCG_K] = K;
  v[KCG_IS_ATRANS] = ATRANS;
  return r;
}

const char* dtype_name(int dt) {
  switch (dt) {
    case KCG_DT_FLOAT16: return "float16";
    case KCG_DT_BFLOAT16: return "bfloat16";
    case KCG_DT_FLOAT32: return "float32";
    case KCG_DT_FLOAT64: return "float64";
    default: return "";
  }
}

const char* dtype_ctype(int dt) {
  switch (dt) {
    case KCG_DT_FLOAT16: return "_Float16";
    case KCG_DT_BFLOAT16: return "__bf16";
    case KCG_DT_FLOAT32: return "float";
    case KCG_DT_FLOAT64: return "double";
    default: return "void";
  }
}

int dtype_size(int dt) {
  switch (dt) {
    case KCG_DT_FLOAT16: return 2;
    case KCG_DT_BFLOAT16: return 2;
    case KCG_DT_FLOAT32: return 4;
    case KCG_DT_FLOAT64: return 8;
    default: return 0;
  }
}

static bool is_pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }

static std::string fmt(const char* what, int a) {
  std::ostringstream s;
  s << what << " (got " << a << ")";
  return s.str();
}

std::string check_common(const MatmulConfig& c) {
  if (c.M <= 0 || c.N <= 0 || c.K <= 0) return "M_SIZE, N_SIZE, K_SIZE must be positive";
  // (the kernels index rows, columns and blocks with 32-bit integers; element offsets are 64-bit)
  if (c.M > (1 << 30) || c.N > (1 << 30) || c.K > (1 << 30)) return "M_SIZE, N_SIZE, K_SIZE must not exceed 2^30";
  if (c.BM <= 0 || c.BN <= 0 || c.BK <= 0) return "BLOCK_SIZE_M/N/K must be positive";
  if ((long)((c.M + c.BM - 1) / c.BM) * ((c.N + c.BN - 1) / c.BN) > 0x7fffffffL) return "more than 2^31 - 1 blocks";
  if (c.TM <= 0 || c.TN <= 0) return "THREAD_SIZE_M/N must be positive";
  if (c.WARP_SIZE != 64) return fmt("WARP_SIZE must be 64 on gfx950", c.WARP_SIZE);
  if (c.BLM <= 0 || c.BLN <= 0 || c.WLM <= 0 || c.WLN <= 0) return "BLOCK_LAYOUT / WARP_LAYOUT must be positive";
  if (c.WLM * c.WLN != c.WARP_SIZE) return "WARP_LAYOUT_M * WARP_LAYOUT_N != WARP_SIZE";           // matmul.py:190,267-274
  if (c.BM % c.TM || c.BN % c.TN) return "BLOCK_SIZE_M/N not divisible by THREAD_SIZE_M/N";         // matmul.py:186-187
  if (c.BLM * c.WLM * c.TM != c.BM) return "BLOCK_LAYOUT_M * WARP_LAYOUT_M * THREAD_SIZE_M != BLOCK_SIZE_M";  // matmul.py:188,300-303
  if (c.BLN * c.WLN * c.TN != c.BN) return "BLOCK_LAYOUT_N * WARP_LAYOUT_N * THREAD_SIZE_N != BLOCK_SIZE_N";
  if (c.LSU < 1) return fmt("LOCAL_SPLIT_U must be >= 1", c.LSU);
  if (c.BK % c.LSU) return "BLOCK_SIZE_K not divisible by LOCAL_SPLIT_U";                          // Optimizer.cc:310
  if (c.thread_num() > kMaxThreads) return fmt("threads per block exceed 1024", c.thread_num());
  if (c.BLOCK_MAPPING < 0) return "BLOCK_MAPPING must be >= 0";
  if (!dtype_size(c.dtA) || !dtype_size(c.dtB) || !dtype_size(c.dtC)) return "unsupported DATATYPE code";
  if (c.dtA != c.dtB) return "DATATYPE_A and DATATYPE_B must be equal";
  const bool same = (c.dtC == c.dtA);
  const bool widen = (c.dtC == KCG_DT_FLOAT32) && (c.dtA == KCG_DT_FLOAT16 || c.dtA == KCG_DT_BFLOAT16);
  if (!same && !widen) return "DATATYPE_C must equal DATATYPE_A, or be float32 for 16-bit inputs";
  const int sz = dtype_size(c.dtA);
  if (!is_pow2(c.GLW_A) || !is_pow2(c.GLW_B)) return "GLOB_LOAD_WIDTH_A/B must be a power of two >= 1";
  if (c.GLW_A * sz > 16 || c.GLW_B * sz > 16) return "GLOB_LOAD_WIDTH_A/B wider than 128 bits";
  if (!is_pow2(c.GSW) || c.GSW * dtype_size(c.dtC) > 16) return "GLOB_STORE_WIDTH must be a power of two, at most 128 bits";
  // a lane whose vector lies outside the matrix reads the first vector of the buffer instead and drops it: every
  // operand must hold at least one 16-byte vector
  if ((long)c.M * c.K * sz < 16 || (long)c.K * c.N * sz < 16 || (long)c.M * c.N * dtype_size(c.dtC) < 16)
    return "A, B and C must each hold at least 16 bytes";
  return "";
}

int simt_pad_a(const MatmulConfig& c) {
  if (c.ATRANS) return 0;
  return c.TSW_A > 4 ? c.TSW_A : 4;
}

std::string check_simt(const MatmulConfig& c) {
  std::string e = check_common(c);
  if (!e.empty()) return e;
  const int szA = dtype_size(c.dtA);
  if (!is_pow2(c.TSW_A) || !is_pow2(c.TSW_B) || !is_pow2(c.WSW_A) || !is_pow2(c.WSW_B))
    return "WARP/THREAD_SCATTER_WIDTH must be powers of two >= 1";
  if (c.WSW_A < c.TSW_A || c.WSW_B < c.TSW_B) return "WARP_SCATTER_WIDTH < THREAD_SCATTER_WIDTH";     // matmul.py:309-310
  if (c.WSW_A % c.TSW_A || c.WSW_B % c.TSW_B) return "WARP_SCATTER_WIDTH not a multiple of THREAD_SCATTER_WIDTH";  // matmul.py:311-312
  if (c.TM % c.WSW_A || c.TN % c.WSW_B) return "THREAD_SIZE not a multiple of WARP_SCATTER_WIDTH";     // Optimizer.cc:21-24
  if (c.TSW_A * szA > 16 || c.TSW_B * szA > 16 || c.TSW_B * dtype_size(c.dtC) > 16)
    return "THREAD_SCATTER_WIDTH wider than 128 bits";
  if (c.ATRANS) {
    if (c.BM % c.GLW_A) return "BLOCK_SIZE_M not divisible by GLOB_LOAD_WIDTH_A";                   // matmul.cpp:2481-2483
  } else {
    if (c.BK % c.GLW_A) return "BLOCK_SIZE_K not divisible by GLOB_LOAD_WIDTH_A (A is [M,K])";
  }
  if (c.BN % c.GLW_B) return "BLOCK_SIZE_N not divisible by GLOB_LOAD_WIDTH_B";
  if (c.LSU > 1 && (c.BN % c.GSW)) return "BLOCK_SIZE_N not divisible by GLOB_STORE_WIDTH";
  if (c.TM * c.TN > 256) return "thread tile larger than 256 accumulators";
  if (lds_bytes(c, KCG_KIND_SIMT) > kMaxLdsBytes) return "LDS footprint exceeds 160 KiB";
  return "";
}

MfmaPlan plan_mfma(const MatmulConfig& c) {
  MfmaPlan p;
  if (c.BLM <= 0 || c.BLN <= 0 || c.BM % c.BLM || c.BN % c.BLN) {
    p.why = "block tile not divisible by BLOCK_LAYOUT";
    return p;
  }
  p.WM = c.BM / c.BLM;
  p.WN = c.BN / c.BLN;
  if (p.WM % 16 || p.WN % 16) {
    p.why = "wave tile (WARP_LAYOUT*THREAD_SIZE) is not a multiple of the 16x16 matrix-core tile";
    return p;
  }
  const int sz = dtype_size(c.dtA);
  if (sz != 2 && sz != 4 && sz != 8) {
    p.why = "matrix-core kernel supports float64, float32, float16 and bfloat16 inputs";
    return p;
  }
  p.MF = (sz != 8 && p.WM % 32 == 0 && p.WN % 32 == 0) ? 32 : 16;   // fp64: 16x16x4 only
  p.G = 16 / sz;
  p.KS = p.G * (64 / p.MF);
  p.ok = true;
  return p;
}

std::string check_mfma(const MatmulConfig& c) {
  std::string e = check_common(c);
  if (!e.empty()) return e;
  MfmaPlan p = plan_mfma(c);
  if (!p.ok) return p.why;
  if (c.BK % (p.KS * c.LSU)) {
    std::ostringstream s;
    s << "BLOCK_SIZE_K must be a multiple of " << p.KS << "*LOCAL_SPLIT_U for the " << p.MF << "x" << p.MF
      << " matrix-core tile";
    return s.str();
  }
  if ((p.WM / p.MF) * (p.WN / p.MF) * (p.MF * p.MF / 64) * (dtype_size(c.dtA) == 8 ? 2 : 1) > 256)
    return "wave tile needs more than 256 accumulator registers";
  if (c.LSU > 1 && (c.BN % c.GSW)) return "BLOCK_SIZE_N not divisible by GLOB_STORE_WIDTH";
  if (lds_bytes(c, KCG_KIND_MFMA) > kMaxLdsBytes) return "LDS footprint exceeds 160 KiB";
  if ((c.SHMP ? 2 : 1) * (c.BM + c.BN) * c.BK * dtype_size(c.dtA) > kMaxLdsBytes) return "LDS footprint exceeds 160 KiB";
  return "";
}

// MatmulParams::getKernelName (src/main.cc:119-145)
std::string kernel_name(const MatmulConfig& c) {
  std::ostringstream ss;
  ss << "GEMM_";
  ss << "MNK" << c.M << "x" << c.N << "x" << c.K << "_";
  ss << "DTabc" << dtype_name(c.dtA) << "x" << dtype_name(c.dtB) << "x" << dtype_name(c.dtC) << "_";
  ss << "AT" << c.ATRANS << "_";
  ss << "TTmn" << c.TM << "x" << c.TN << "_";
  ss << "BTmnk" << c.BM << "x" << c.BN << "x" << c.BK << "_";
  ss << "BLmn" << c.BLM << "x" << c.BLN << "_";
  ss << "WLmn" << c.WLM << "x" << c.WLN << "_";
  ss << "GLWab" << c.GLW_A << "x" << c.GLW_B << "_";
  ss << "GSW" << c.GSW << "_";
  ss << "WSWab" << c.WSW_A << "x" << c.WSW_B << "_";
  ss << "TSWab" << c.TSW_A << "x" << c.TSW_B << "_";
  ss << "LSU" << c.LSU << "_";
  ss << "BM" << c.BLOCK_MAPPING << "_";
  ss << "UNROLL" << c.UNROLL << "_";
  ss << "REGP" << c.REGP << "_";
  ss << "SHMP" << c.SHMP << "_";
  ss << "LC" << c.LC << "_";
  ss << "RC" << c.RC << "_";
  return ss.str();
}

// UserInputs.sharedMem (CompiledKernelFactory.py:30-44)
int reference_lds_bytes(const MatmulConfig& c) {
  int sizeA = c.BM * c.BK * dtype_size(c.dtA);
  int sizeB = c.BN * c.BK * dtype_size(c.dtB);
  int sizeAB = sizeA + sizeB;
  if (c.SHMP > 0) sizeAB *= 2;
  int sizeC = -1;
  if (c.LSU > 1) sizeC = c.BM * c.BN * c.LSU * dtype_size(c.dtA);
  return sizeAB > sizeC ? sizeAB : sizeC;
}

// (That kernel keeps 2..4 stages of (BM+BN)*BK*2 bytes in static LDS: as many as fit in 160 KiB.)
// Must state the same rule as DirectPlan<C>::ELIGIBLE in kcg_device_direct.h (a static_assert there
// compares the two): 16-bit inputs or fp32 throughout, at least one full K tile, both prefetch flags, LOAD_CONTINUOUS, 128-bit load
// widths, tiles (powers of two or multiples of 16 chunks) that split evenly into 1 KiB wave fetches, at least two rows of
// matrix-core tiles per wave, two LDS stages within 160 KiB; any M, N and K >= BK.
bool mfma_direct(const MatmulConfig& c) {
  MfmaPlan p = plan_mfma(c);
  const int es = dtype_size(c.dtA);
  if (!p.ok || !(es == 2 || (es == 4 && c.dtC == KCG_DT_FLOAT32))) return false;
  const int g = 16 / es;                                  // elements per 16-byte chunk
  if (!c.SHMP || !c.REGP || !c.LC || c.LSU != 1 || c.GLW_A != g || c.GLW_B != g) return false;
  // this path picks its own matrix-core tile: for 16-bit inputs 16x16x32 whenever the K tile is a
  // multiple of 32; for fp32 the larger tile where the wave tile holds two rows of them
  const bool fits32 = p.WM % 32 == 0 && p.WN % 32 == 0 && p.WM / 32 >= 2;   // two rows of tiles per wave
  const int mf = es == 2 ? ((c.BK % 32 == 0 || !fits32) ? 16 : 32) : (fits32 ? 32 : 16);
  const int ks = g * (64 / mf);
  if (c.BK % ks) return false;
  // edge tiles in M and N are handled; K needs one full tile
  if (c.K < c.BK) return false;
  if (p.WM / mf < 2) return false;                       // the K loop streams A fragments row by row
  const int nw = c.BLM * c.BLN;
  // tile extents: a power of two or a multiple of 16 chunks (the bank swizzle works on aligned groups of 16 chunks)
  auto tile_ok = [g](int x) { return is_pow2(x) || (x > 0 && x % (16 * g) == 0); };
  if (!tile_ok(c.BM) || !tile_ok(c.BN) || !is_pow2(c.BK) || c.BM < 32 || c.BN < 32) return false;
  if ((c.BM * c.BK / g) % (64 * nw) || (c.BN * c.BK / g) % (64 * nw)) return false;
  // (any K >= BK and any M and N that give A and B rows of at least one chunk: the 16-byte fetches take source
  // addresses of any alignment)
  if (c.N < g || (c.ATRANS ? c.M : c.K) < g) return false;
  const long lim = 1L << 31;                              // 32-bit byte offsets per lane inside a tile panel
  if ((long)c.BM * c.K * es >= lim || (long)c.BK * c.M * es >= lim || (long)c.BK * c.N * es >= lim) return false;
  return 2 * (c.BM + c.BN) * c.BK * es <= kMaxLdsBytes;
}

int lds_bytes(const MatmulConfig& c, int kind, bool allow_direct) {
  if (allow_direct && kind == KCG_KIND_MFMA && mfma_direct(c)) return 0;   // that path declares its stages statically
  const int stages = c.SHMP ? 2 : 1;
  const int szA = dtype_size(c.dtA), szB = dtype_size(c.dtB);
  const int accsz = (c.dtC == KCG_DT_FLOAT64) ? 8 : 4;
  int ab;
  if (kind == KCG_KIND_MFMA) {
    ab = stages * (c.BM + c.BN) * c.BK * szA;
  } else {
    const int lda = c.BM + simt_pad_a(c), ldb = c.BN;
    const int offB = (stages * c.BK * lda * szA + 15) & ~15;
    ab = offB + stages * c.BK * ldb * szB;
  }
  int cbytes = (c.LSU > 1) ? c.LSU * c.BM * c.BN * accsz : 0;
  int r = ab > cbytes ? ab : cbytes;
  return (r + 15) & ~15;
}

static int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  if (!v || !*v) return dflt;
  const int x = atoi(v);
  return x > 0 ? x : dflt;
}
// An MI355X in its default (single-partition) mode: 256 compute units in 8 XCDs.  Another partition mode
// (or another part) is described with $KCG_NUM_CUS / $KCG_NUM_XCDS; both are baked into the instantiation.
int num_cus() { return env_int("KCG_NUM_CUS", 256); }
int num_xcds() { return env_int("KCG_NUM_XCDS", 8); }

// Rewriter::BlockMapping with isCol=true (Rewriter.cc:726-761; Rewriter.h:112)
void block_mapping(const MatmulConfig& c, int bid, bool xcd_remap, int* by, int* bx) {
  const int gy = c.grid_y(), gx = c.grid_x();
  const int nb = gy * gx;
  const int nx = num_xcds();
  if (xcd_remap && nx > 1 && nb % nx == 0) bid = (bid % nx) * (nb / nx) + bid / nx;
  const int g = c.BLOCK_MAPPING;
  if (g > 0 && gy % g == 0) {
    const int gn = g * gx;
    *by = (bid / gn) * g + bid % g;
    *bx = (bid % gn) / g;
  } else {
    *by = bid / gx;
    *bx = bid % gx;
  }
}

std::string kernel_name_ex(const MatmulConfig& c, int epilogue) {
  return kernel_name(c) + (epilogue ? "EXab_" : "EX_");
}

std::string instantiation_source(const MatmulConfig& c, int kind, bool xcd_remap, bool allow_direct, int ex) {
  std::ostringstream s;
  const char* acc = (c.dtC == KCG_DT_FLOAT64) ? "double" : "float";
  s << "// generated by libkcg_gemm: instantiation of the " << (kind == KCG_KIND_MFMA ? "gemm_mfma" : "gemm_simt")
    << " template\n";
  s << "#include \"kcg_gemm_device.h\"\n";
  s << "namespace {\nstruct Cfg {\n";
  s << "  typedef " << dtype_ctype(c.dtA) << " TA;\n";
  s << "  typedef " << dtype_ctype(c.dtB) << " TB;\n";
  s << "  typedef " << dtype_ctype(c.dtC) << " TC;\n";
  s << "  typedef " << acc << " ACC;\n";
  auto I = [&](const char* n, int v) { s << "  static constexpr int " << n << " = " << v << ";\n"; };
  auto Bv = [&](const char* n, bool v) { s << "  static constexpr bool " << n << " = " << (v ? "true" : "false") << ";\n"; };
  I("M", c.M); I("N", c.N); I("K", c.K);
  I("BM", c.BM); I("BN", c.BN); I("BK", c.BK); I("TM", c.TM); I("TN", c.TN);
  I("WARP_SIZE", c.WARP_SIZE); I("BLM", c.BLM); I("BLN", c.BLN); I("WLM", c.WLM); I("WLN", c.WLN);
  I("GLW_A", c.GLW_A); I("GLW_B", c.GLW_B); I("WSW_A", c.WSW_A); I("WSW_B", c.WSW_B);
  I("TSW_A", c.TSW_A); I("TSW_B", c.TSW_B); I("LSU", c.LSU); I("BLOCK_MAPPING", c.BLOCK_MAPPING);
  I("GSW", c.GSW); I("UNROLL", c.UNROLL);
  Bv("REGP", c.REGP != 0); Bv("SHMP", c.SHMP != 0);
  I("LC", c.LC != 0); I("RC", c.RC != 0);
  Bv("ATRANS", c.ATRANS != 0);
  Bv("EDGE", c.edge());
  Bv("XCD_REMAP", xcd_remap);
  I("NUM_CU", num_cus()); I("NUM_XCD", num_xcds());
  Bv("EPI", ex > 0);
  Bv("DIRECT_ELIGIBLE", kind == KCG_KIND_MFMA && mfma_direct(c));   // the rule; the device header re-derives and compares it
  Bv("DIRECT", allow_direct && kind == KCG_KIND_MFMA && mfma_direct(c));
  I("SIMT_PAD_A", simt_pad_a(c)); I("SIMT_PAD_B", 0);
  s << "};\n}  // namespace\n\n";
  const char* fn = kind == KCG_KIND_MFMA ? "gemm_mfma" : "gemm_simt";
  if (ex < 0) {
    s << "extern \"C\" __global__ __launch_bounds__(" << c.thread_num() << ") void " << kernel_name(c)
      << "(const Cfg::TA* __restrict__ A, const Cfg::TB* __restrict__ B, Cfg::TC* __restrict__ C) {\n";
    s << "  extern __shared__ __attribute__((aligned(16))) char kcg_shm0[];\n";
    s << "  kcg::" << fn << "<Cfg>(A, B, C, kcg_shm0);\n";
    s << "}\n";
  } else {
    // batched / strided form: problem blockIdx.y of the batch lives stride_* elements further in each
    // buffer; alpha and beta are used only by an instantiation with the alpha/beta epilogue
    s << "extern \"C\" __global__ __launch_bounds__(" << c.thread_num() << ") void " << kernel_name_ex(c, ex)
      << "(const Cfg::TA* A, const Cfg::TB* B, Cfg::TC* C, long stride_a, long stride_b, long stride_c, float alpha, float beta) {\n";
    s << "  extern __shared__ __attribute__((aligned(16))) char kcg_shm0[];\n";
    s << "  const long z = blockIdx.y;\n";
    s << "  kcg::" << fn << "<Cfg>(A + z * stride_a, B + z * stride_b, C + z * stride_c, kcg_shm0, kcg::EpiArgs{alpha, beta});\n";
    s << "}\n";
  }
  return s.str();
}

}  // namespace kcg
