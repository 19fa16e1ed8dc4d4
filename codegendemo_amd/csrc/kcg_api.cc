// kcg_api.cc — the C ABI of libkcg_gemm.so (declared in include/kcg_gemm.h).
//
//   compile : config -> instantiation stub -> hiprtc (gfx950) -> code object file, with an on-disk
//             cache keyed by a hash of everything that determines the binary
//   load    : code object file -> hipModule / hipFunction
//   launch  : hipModuleLaunchKernel with three device pointers and dynamic LDS
//   bench   : HIP-event timing loop in C
//
// There is no CPU execution path here: without a HIP device, load/launch/benchmark fail with
// KCG_ERR_HIP.  Compilation alone needs no device.
#ifndef _GNU_SOURCE
#define _GNU_SOURCE   /* dlmopen */
#endif
#include <dlfcn.h>
#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <sys/types.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <cerrno>
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "kcg_config.h"

#define KCG_VERSION "kcg-gemm-gfx950 0.3"

// The device template headers, embedded at build time (directory given by -DKCG_DEVICE_HEADER_DIR):
// kcg_gemm_device.h is what the instantiation stub includes; it includes the others.
#define KCG_EMBED(sym, file)                         \
  __asm__(".section .rodata\n"                       \
          ".global " #sym "\n" #sym ":\n"            \
          ".incbin \"" KCG_DEVICE_HEADER_DIR "/" file "\"\n" \
          ".byte 0\n"                                \
          ".previous\n");                            \
  extern "C" const char sym[];
KCG_EMBED(kcg_device_src, "kcg_gemm_device.h")
KCG_EMBED(kcg_device_src_common, "kcg_device_common.h")
KCG_EMBED(kcg_device_src_simt, "kcg_device_simt.h")
KCG_EMBED(kcg_device_src_mfma_ops, "kcg_device_mfma_ops.h")
KCG_EMBED(kcg_device_src_direct, "kcg_device_direct.h")
KCG_EMBED(kcg_device_src_mfma, "kcg_device_mfma.h")
static const char* const kDeviceHeaderNames[] = {"kcg_gemm_device.h",     "kcg_device_common.h", "kcg_device_simt.h",
                                                 "kcg_device_mfma_ops.h", "kcg_device_direct.h", "kcg_device_mfma.h"};
static const char* const kDeviceHeaderSrcs[] = {kcg_device_src,          kcg_device_src_common, kcg_device_src_simt,
                                                kcg_device_src_mfma_ops, kcg_device_src_direct, kcg_device_src_mfma};
static const int kNumDeviceHeaders = 6;

namespace {

thread_local std::string g_err;

// Functions handed out by kcg_load: which argument list their kernel takes (3: the reference's three pointers,
// 8: the batched-strided form) and which module owns them.  kcg_launch / kcg_launch_batched refuse a known
// function of the other form instead of starting a kernel on a parameter block it would misread; a handle
// that did not come from kcg_load is launched as the caller says.
struct LoadedFunction {
  int n_args;
  uint64_t module;
  int es_a, es_b, es_c;   // element sizes of A, B, C from the DTabc part of the kernel name; 0: not known
};
std::mutex g_loaded_mu;
std::unordered_map<uint64_t, LoadedFunction> g_loaded;

LoadedFunction loaded_function(uint64_t function) {
  std::lock_guard<std::mutex> lock(g_loaded_mu);
  auto it = g_loaded.find(function);
  return it == g_loaded.end() ? LoadedFunction{0, 0, 0, 0, 0} : it->second;
}
int loaded_args(uint64_t function) { return loaded_function(function).n_args; }

// "..._DTabcfloat16xfloat16xfloat32_..." -> 2, 2, 4 (0 where the name does not say)
void element_sizes_from_name(const std::string& name, int es[3]) {
  es[0] = es[1] = es[2] = 0;
  size_t p = name.find("DTabc");
  if (p == std::string::npos) return;
  p += 5;
  for (int i = 0; i < 3; ++i) {
    static const struct { const char* text; int size; } types[] = {
        {"float16", 2}, {"bfloat16", 2}, {"float32", 4}, {"float64", 8}};
    for (const auto& t : types) {
      const size_t n = strlen(t.text);
      if (name.compare(p, n, t.text) == 0) {
        es[i] = t.size;
        p += n;
        break;
      }
    }
    if (!es[i]) return;
    if (i < 2) {
      if (p >= name.size() || name[p] != 'x') return;
      ++p;
    }
  }
}

int fail(int code, const std::string& msg) {
  g_err = msg;
  return code;
}

// ---------------------------------------------------------------------------------------------
// HIP runtime / hiprtc binding.  The library is NOT linked against libamdhip64 / libhiprtc: a
// process must talk to exactly one HIP runtime, and a host program may already carry its own (the
// PyTorch wheel bundles one next to libtorch_hip.so).  So the entry points are looked up at first
// use: an already-loaded libamdhip64.so.7 / libhiprtc.so.7 wins (RTLD_NOLOAD finds it whatever scope
// it was loaded in); otherwise the system one is opened through this library's RUNPATH.
// ---------------------------------------------------------------------------------------------
#define KCG_STR2(x) #x
#define KCG_STR(x) KCG_STR2(x)

#define KCG_HIP_FUNCS(X)      \
  X(hipSetDevice)             \
  X(hipModuleLoadData)        \
  X(hipModuleGetFunction)     \
  X(hipModuleUnload)          \
  X(hipFuncGetAttribute)      \
  X(hipModuleLaunchKernel)    \
  X(hipEventCreate)           \
  X(hipEventRecord)           \
  X(hipEventSynchronize)      \
  X(hipEventElapsedTime)      \
  X(hipEventDestroy)          \
  X(hipStreamSynchronize)     \
  X(hipGetDeviceProperties)   \
  X(hipGetErrorString)

#define KCG_RTC_FUNCS(X)      \
  X(hiprtcCreateProgram)      \
  X(hiprtcCompileProgram)     \
  X(hiprtcGetProgramLogSize)  \
  X(hiprtcGetProgramLog)      \
  X(hiprtcGetCodeSize)        \
  X(hiprtcGetCode)            \
  X(hiprtcDestroyProgram)     \
  X(hiprtcGetErrorString)     \
  X(hiprtcVersion)

struct HipApi {
#define X(name) decltype(&::name) p_##name = nullptr;
  KCG_HIP_FUNCS(X)
#undef X
  // hipFunction_t overload of hipFuncSetAttribute lives behind the plain C symbol
  hipError_t (*p_hipFuncSetAttribute)(const void*, hipFuncAttribute, int) = nullptr;
  std::string error;
  bool ok = false;
};
struct RtcApi {
#define X(name) decltype(&::name) p_##name = nullptr;
  KCG_RTC_FUNCS(X)
#undef X
  std::string error;
  bool ok = false;
};

void* open_shared(const char* soname, std::string* err) {
  void* h = dlopen(soname, RTLD_NOW | RTLD_NOLOAD);
  if (!h) h = dlopen(soname, RTLD_NOW | RTLD_LOCAL);
  if (!h && err) {
    const char* why = dlerror();   // one call: it clears the message it returns
    *err = std::string("cannot load ") + soname + ": " + (why ? why : "?");
  }
  return h;
}

const HipApi& hip_api() {
  static const HipApi api = [] {
    HipApi a;
    void* h = open_shared("libamdhip64.so.7", &a.error);
    if (!h) return a;
    bool all = true;
#define X(name)                                                              \
  a.p_##name = reinterpret_cast<decltype(&::name)>(dlsym(h, KCG_STR(name))); \
  if (!a.p_##name) { all = false; a.error += std::string(" missing symbol ") + KCG_STR(name); }
    KCG_HIP_FUNCS(X)
#undef X
    a.p_hipFuncSetAttribute =
        reinterpret_cast<hipError_t (*)(const void*, hipFuncAttribute, int)>(dlsym(h, "hipFuncSetAttribute"));
    a.ok = all;
    return a;
  }();
  return api;
}

// Which hiprtc compiles.  Default: the one the process already carries, else the system's (open_shared).
// $KCG_HIPRTC_LIB = path of another libhiprtc: that library is opened in a link namespace of its own
// (dlmopen), so that the compiler library it loads by name (libamd_comgr.so.3) is the one that lies beside
// it and not a copy of the same name the process has already loaded.  This is how one process (a Python
// process with PyTorch's bundled ROCm, say) builds kernels with the system's compiler as well, e.g. to put
// both builds through the same correctness gate.  Read at every compile.
// `identity` goes into the cache key: hiprtcVersion() alone does not tell two ROCm releases apart.
struct RtcLib {
  RtcApi api;
  std::string identity;
};

std::string library_identity(void* symbol) {
  Dl_info info;
  if (!symbol || !dladdr(symbol, &info) || !info.dli_fname) return "hiprtc:?";
  char real[PATH_MAX];
  std::string path = realpath(info.dli_fname, real) ? real : info.dli_fname;
  struct stat st;
  long size = stat(path.c_str(), &st) == 0 ? (long)st.st_size : -1;
  return "hiprtc:" + path + ":" + std::to_string(size);
}

const RtcLib& rtc_lib() {
  static std::mutex mu;
  static std::map<std::string, std::unique_ptr<RtcLib>> libs;
  const char* v = getenv("KCG_HIPRTC_LIB");
  const std::string which = (v && *v) ? v : "";
  std::lock_guard<std::mutex> lock(mu);
  auto it = libs.find(which);
  if (it != libs.end()) return *it->second;
  std::unique_ptr<RtcLib> lib(new RtcLib);
  RtcApi& a = lib->api;
  void* h = nullptr;
  if (which.empty()) {
    h = open_shared("libhiprtc.so.7", &a.error);
  } else {
    h = dlmopen(LM_ID_NEWLM, which.c_str(), RTLD_NOW | RTLD_LOCAL);
    if (!h) {
      const char* why = dlerror();
      a.error = " cannot load $KCG_HIPRTC_LIB=" + which + ": " + (why ? why : "?");
    }
  }
  if (h) {
    bool all = true;
#define X(name)                                                              \
  a.p_##name = reinterpret_cast<decltype(&::name)>(dlsym(h, KCG_STR(name))); \
  if (!a.p_##name) { all = false; a.error += std::string(" missing symbol ") + KCG_STR(name); }
    KCG_RTC_FUNCS(X)
#undef X
    a.ok = all;
    lib->identity = library_identity(reinterpret_cast<void*>(a.p_hiprtcVersion));
  }
  return *(libs[which] = std::move(lib));
}

#define HIPF(name) (hip_api().p_##name)

// Same text shape as the reference loader's errors (loaderCCode/hip.c:8-21).
int hip_fail(hipError_t e, const char* what) {
  char buf[1024];
  const char* txt = hip_api().ok ? HIPF(hipGetErrorString)(e) : "?";
  snprintf(buf, sizeof(buf), "KCG Error[HIP]:  Code: %d, Messsage: %s (%s)", (int)e, txt, what);
  g_err = buf;
  return KCG_ERR_HIP;
}

#define HIP_READY()                                                                         \
  do {                                                                                      \
    if (!hip_api().ok) return fail(KCG_ERR_HIP, "KCG Error[HIP]: runtime unavailable:" + hip_api().error); \
  } while (0)

#define HIP_TRY(expr)                                   \
  do {                                                  \
    hipError_t _e = (expr);                             \
    if (_e != hipSuccess) return hip_fail(_e, #expr);   \
  } while (0)

uint64_t fnv1a(const std::string& s, uint64_t h = 1469598103934665603ull) {
  for (unsigned char ch : s) {
    h ^= ch;
    h *= 1099511628211ull;
  }
  return h;
}

bool env_flag(const char* name, bool dflt) {
  const char* v = getenv(name);
  if (!v || !*v) return dflt;
  return !(v[0] == '0' || v[0] == 'n' || v[0] == 'N' || v[0] == 'f' || v[0] == 'F');
}

std::string library_dir() {
  Dl_info info;
  if (dladdr((void*)&kcg_device_src, &info) && info.dli_fname) {
    std::string p = info.dli_fname;
    size_t k = p.find_last_of('/');
    if (k != std::string::npos) return p.substr(0, k);
  }
  return ".";
}

std::string cache_dir() {
  const char* v = getenv("KCG_CACHE_DIR");
  if (v && *v) return v;
  return library_dir() + "/_kcg_cache";
}

bool make_dirs(const std::string& path) {
  std::string cur;
  for (size_t i = 0; i <= path.size(); ++i) {
    if (i == path.size() || path[i] == '/') {
      if (!cur.empty()) {
        if (mkdir(cur.c_str(), 0777) != 0 && errno != EEXIST) return false;
      }
    }
    if (i < path.size()) cur.push_back(path[i]);
  }
  return true;
}

bool file_exists(const std::string& p) {
  struct stat st;
  return stat(p.c_str(), &st) == 0 && S_ISREG(st.st_mode) && st.st_size > 0;
}

bool read_file(const std::string& p, std::vector<char>* out) {
  FILE* f = fopen(p.c_str(), "rb");
  if (!f) return false;
  fseek(f, 0, SEEK_END);
  long n = ftell(f);
  rewind(f);
  out->resize(n > 0 ? n : 0);
  size_t got = n > 0 ? fread(out->data(), 1, n, f) : 0;
  fclose(f);
  return (long)got == n;
}

// Write-then-rename so that concurrent compile processes never expose a partial code object.
bool write_file_atomic(const std::string& p, const char* data, size_t n) {
  static std::atomic<unsigned> counter{0};
  char suffix[64];
  snprintf(suffix, sizeof(suffix), ".tmp.%d.%u", (int)getpid(), counter.fetch_add(1));
  std::string tmp = p + suffix;
  FILE* f = fopen(tmp.c_str(), "wb");
  if (!f) return false;
  size_t w = fwrite(data, 1, n, f);
  if (fclose(f) != 0 || w != n) {
    unlink(tmp.c_str());
    return false;
  }
  if (rename(tmp.c_str(), p.c_str()) != 0) {
    unlink(tmp.c_str());
    return false;
  }
  return true;
}

const std::vector<std::string>& compile_flags() {
  // -amdgpu-spill-vgpr-to-agpr=0: under register pressure the compiler parks vector registers in unused
  // accumulation registers before it resorts to scratch memory.  Scalar-kernel configs with large thread
  // tiles and edge predicates built that way have returned wrong values (one staging or fragment register
  // holding another's contents) and are right with the option, at any load width and with or without
  // branches around the edge loads; kernels that do not spill are unaffected by it.  It also makes every
  // spill visible as scratch memory, which is what the direct-staging kernel's spill check looks at.
  static const std::vector<std::string> flags = {
      "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
      "-mllvm", "-amdgpu-spill-vgpr-to-agpr=0",
  };
  return flags;
}

// Extra hiprtc options from $KCG_EXTRA_FLAGS (space separated), e.g. "-DNAME=1" or "-save-temps";
// part of the cache key.  The reference had a comparable hook for injecting an LLVM pass plugin
// (AMDGCN_INSTRUMENTATION_LIB, LLVMIRTranslation.cc:98-108).
std::vector<std::string> extra_flags() {
  std::vector<std::string> out;
  const char* v = getenv("KCG_EXTRA_FLAGS");
  if (!v) return out;
  std::string cur;
  for (const char* p = v;; ++p) {
    if (*p == ' ' || *p == 0) {
      if (!cur.empty()) out.push_back(cur);
      cur.clear();
      if (*p == 0) break;
    } else {
      cur.push_back(*p);
    }
  }
  return out;
}

int resolve_kind(const kcg::MatmulConfig& c, int kind, std::string* why) {
  if (kind == KCG_KIND_SIMT) {
    *why = kcg::check_simt(c);
    return why->empty() ? (int)KCG_KIND_SIMT : (int)KCG_ERR_INVALID_CONFIG;
  }
  if (kind == KCG_KIND_MFMA) {
    *why = kcg::check_mfma(c);
    return why->empty() ? (int)KCG_KIND_MFMA : (int)KCG_ERR_INVALID_CONFIG;
  }
  if (kind != KCG_KIND_AUTO) {
    *why = "unknown kernel kind";
    return KCG_ERR_ARGUMENT;
  }
  std::string wm = kcg::check_mfma(c);
  if (wm.empty()) return KCG_KIND_MFMA;
  std::string ws = kcg::check_simt(c);
  if (ws.empty()) return KCG_KIND_SIMT;
  *why = "matrix-core kernel: " + wm + "; SIMT kernel: " + ws;
  return KCG_ERR_INVALID_CONFIG;
}

int copy_out(const std::string& s, char* out, int out_len) {
  if (out && out_len > 0) {
    size_t n = std::min((size_t)out_len - 1, s.size());
    memcpy(out, s.data(), n);
    out[n] = 0;
  }
  return (int)s.size();
}

}  // namespace

extern "C" {

const char* kcg_last_error(void) { return g_err.c_str(); }
const char* kcg_version(void) { return KCG_VERSION; }

const char* kcg_cfg_keyword(int index) {
  static const char* const kw[KCG_CFG_LEN] = {
      "BLOCK_SIZE_M", "BLOCK_SIZE_N", "BLOCK_SIZE_K", "THREAD_SIZE_M", "THREAD_SIZE_N", "WARP_SIZE",
      "BLOCK_LAYOUT_M", "BLOCK_LAYOUT_N", "WARP_LAYOUT_M", "WARP_LAYOUT_N",
      "GLOB_LOAD_WIDTH_A", "GLOB_LOAD_WIDTH_B", "WARP_SCATTER_WIDTH_A", "WARP_SCATTER_WIDTH_B",
      "THREAD_SCATTER_WIDTH_A", "THREAD_SCATTER_WIDTH_B", "LOCAL_SPLIT_U", "BLOCK_MAPPING", "GLOB_STORE_WIDTH",
      "UNROLL_NUM", "REG_PREFETCH", "SHARED_PREFETCH", "LOAD_CONTINUOUS", "REDUCE_C_CONTINUOUS",
      "DATATYPE_A", "DATATYPE_B", "DATATYPE_C", "M_SIZE", "N_SIZE", "K_SIZE", "IS_ATRANS"};
  if (index < 0 || index >= KCG_CFG_LEN) return nullptr;
  return kw[index];
}

int kcg_dtype_size(int dtype) { return kcg::dtype_size(dtype); }

int kcg_check_config(const kcg_matmul_cfg* cfg, int kind) {
  if (!cfg) return fail(KCG_ERR_ARGUMENT, "cfg is null");
  std::string why;
  int k = resolve_kind(kcg::MatmulConfig::from(*cfg), kind, &why);
  if (k < 0) return fail(k, "invalid config: " + why);
  g_err.clear();
  return KCG_OK;
}

int kcg_select_kind(const kcg_matmul_cfg* cfg) {
  if (!cfg) return fail(KCG_ERR_ARGUMENT, "cfg is null");
  std::string why;
  int k = resolve_kind(kcg::MatmulConfig::from(*cfg), KCG_KIND_AUTO, &why);
  if (k < 0) return fail(k, "invalid config: " + why);
  return k;
}

int kcg_kernel_name(const kcg_matmul_cfg* cfg, char* out, int out_len) {
  if (!cfg) return fail(KCG_ERR_ARGUMENT, "cfg is null");
  return copy_out(kcg::kernel_name(kcg::MatmulConfig::from(*cfg)), out, out_len);
}

int kcg_launch_dims(const kcg_matmul_cfg* cfg, int32_t grid[3], int32_t block[3]) {
  if (!cfg || !grid || !block) return fail(KCG_ERR_ARGUMENT, "null argument");
  kcg::MatmulConfig c = kcg::MatmulConfig::from(*cfg);
  if (c.BM <= 0 || c.BN <= 0 || c.TM <= 0 || c.TN <= 0) return fail(KCG_ERR_INVALID_CONFIG, "invalid config: tile sizes must be positive");
  grid[0] = c.grid_y() * c.grid_x();
  grid[1] = grid[2] = 1;
  block[0] = c.thread_num();
  block[1] = block[2] = 1;
  return KCG_OK;
}

int kcg_reference_lds_bytes(const kcg_matmul_cfg* cfg) {
  if (!cfg) return fail(KCG_ERR_ARGUMENT, "cfg is null");
  return kcg::reference_lds_bytes(kcg::MatmulConfig::from(*cfg));
}

int kcg_block_mapping(const kcg_matmul_cfg* cfg, int bid, int xcd_remap, int32_t* by, int32_t* bx) {
  if (!cfg || !by || !bx) return fail(KCG_ERR_ARGUMENT, "null argument");
  kcg::MatmulConfig c = kcg::MatmulConfig::from(*cfg);
  if (c.BM <= 0 || c.BN <= 0) return fail(KCG_ERR_INVALID_CONFIG, "invalid config: tile sizes must be positive");
  if (bid < 0 || bid >= c.grid_x() * c.grid_y()) return fail(KCG_ERR_ARGUMENT, "block id out of range");
  int y, x;
  kcg::block_mapping(c, bid, xcd_remap != 0, &y, &x);
  *by = y;
  *bx = x;
  return KCG_OK;
}

int kcg_instantiation_source(const kcg_matmul_cfg* cfg, int kind, char* out, int out_len) {
  if (!cfg) return fail(KCG_ERR_ARGUMENT, "cfg is null");
  kcg::MatmulConfig c = kcg::MatmulConfig::from(*cfg);
  std::string why;
  int k = resolve_kind(c, kind, &why);
  if (k < 0) return fail(k, "invalid config: " + why);
  return copy_out(kcg::instantiation_source(c, k, env_flag("KCG_XCD_REMAP", true)), out, out_len);
}

// What the metadata note of a code object says about its (one) kernel: the msgpack key is followed by its
// unsigned value.  -1 where the key is not there (the caller then does not know).
static long code_object_meta(const std::vector<char>& code, const char* key) {
  const size_t klen = strlen(key);
  for (size_t i = 0; i + klen + 1 <= code.size(); ++i) {
    if (memcmp(code.data() + i, key, klen) != 0) continue;
    const unsigned char* p = reinterpret_cast<const unsigned char*>(code.data()) + i + klen;
    const size_t left = code.size() - (i + klen);
    if (left >= 1 && p[0] <= 0x7f) return p[0];
    if (left >= 2 && p[0] == 0xcc) return p[1];
    if (left >= 3 && p[0] == 0xcd) return (p[1] << 8) | p[2];
    if (left >= 5 && p[0] == 0xce) return ((long)p[1] << 24) | (p[2] << 16) | (p[3] << 8) | p[4];
    if (left >= 9 && p[0] == 0xcf) {
      long v = 0;
      for (int b = 1; b <= 8; ++b) v = (v << 8) | p[b];
      return v;
    }
  }
  return -1;
}

struct CodeMeta {
  long scratch, vgprs, vgpr_spills, sgpr_spills;
  static CodeMeta of(const std::vector<char>& code) {
    return CodeMeta{code_object_meta(code, ".private_segment_fixed_size"), code_object_meta(code, ".vgpr_count"),
                    code_object_meta(code, ".vgpr_spill_count"), code_object_meta(code, ".sgpr_spill_count")};
  }
  bool known() const { return scratch >= 0 && vgprs >= 0; }
  // the register allocator ran out of vector registers: scratch memory in use, vector registers spilled, or the
  // whole file of 512 taken.  (Scalar registers spilled into lanes of a vector register alone do not count: that
  // is what the compiler does in every large kernel, 110 of 1900 cached instantiations, none of them ever wrong.)
  bool under_pressure() const { return !known() || scratch != 0 || vgpr_spills > 0 || vgprs >= 512; }
};

// Outcome of build_variant besides the kcg_status values: the direct-staging build would spill.
static const int kBuildSpills = 1;

// -DKCG_DIAG_...: builds of the direct-staging kernel that leave work out on purpose (their C is wrong)
static bool has_diagnostic_flag(const std::vector<std::string>& flags) {
  for (const auto& f : flags)
    if (f.find("KCG_DIAG_") != std::string::npos) return true;
  return false;
}

// "<name>.<hash>.buildinfo" beside a cached code object: what kcg_kernel_info reports about the build
static void write_build_info(const std::string& path, const kcg_kernel_info& k) {
  char text[200];
  const int n = snprintf(text, sizeof(text), "build_flags=%d scratch_bytes=%d vgprs=%d sgpr_spills=%d lds_bytes=%d kind=%d\n",
                         k.build_flags, k.scratch_bytes, k.vgprs, k.sgpr_spills, k.lds_bytes, k.kind);
  write_file_atomic(path, text, (size_t)n);
}
static bool read_build_info(const std::string& path, kcg_kernel_info* k) {
  std::vector<char> raw;
  if (!read_file(path, &raw)) return false;
  raw.push_back(0);
  int f = 0, sc = 0, vg = 0, sg = 0, lds = 0, kind = 0;
  if (sscanf(raw.data(), "build_flags=%d scratch_bytes=%d vgprs=%d sgpr_spills=%d lds_bytes=%d kind=%d", &f, &sc, &vg, &sg, &lds,
             &kind) != 6)
    return false;
  k->build_flags = f; k->scratch_bytes = sc; k->vgprs = vg; k->sgpr_spills = sg; k->lds_bytes = lds; k->kind = kind;
  return true;
}

// Builds (or finds in the cache) the code object of config c as kernel family k; `allow_direct` lets a
// matrix-core config that is eligible for direct global->LDS staging use that kernel.
// ex < 0: the reference's three-pointer kernel; 0 / 1: the batched-strided form without / with alpha-beta.
static int build_variant(const kcg::MatmulConfig& c, int k, bool allow_direct, const std::string& arch, int ex, kcg_kernel_info* out) {
  const bool xcd = env_flag("KCG_XCD_REMAP", true);
  const bool direct = allow_direct && k == KCG_KIND_MFMA && kcg::mfma_direct(c);
  const bool declined = !allow_direct && k == KCG_KIND_MFMA && kcg::mfma_direct(c);
  const std::string name = ex < 0 ? kcg::kernel_name(c) : kcg::kernel_name_ex(c, ex);
  const std::string stub = kcg::instantiation_source(c, k, xcd, allow_direct, ex);
  const std::vector<std::string> extra = extra_flags();
  const bool diagnostic = has_diagnostic_flag(extra);

  memset(out, 0, sizeof(*out));
  if (name.size() >= sizeof(out->kernel_name)) return fail(KCG_ERR_ARGUMENT, "kernel name too long");
  memcpy(out->kernel_name, name.c_str(), name.size() + 1);
  out->grid[0] = c.grid_y() * c.grid_x();
  out->grid[1] = out->grid[2] = 1;
  out->block[0] = c.thread_num();
  out->block[1] = out->block[2] = 1;
  out->lds_bytes = kcg::lds_bytes(c, k, allow_direct);
  out->kind = k;
  out->scratch_bytes = out->vgprs = out->sgpr_spills = -1;

  // A build that computes a wrong C on purpose must be asked for twice: by its flag and by $KCG_ALLOW_DIAG=1
  // (the reference's comparable hook, an LLVM pass plugin named in the environment, is opt-in as well:
  // LLVMIRTranslation.cc:98-108).  Such a kernel keeps the reference name; kcg_kernel_info says what it is.
  if (diagnostic && !env_flag("KCG_ALLOW_DIAG", false))
    return fail(KCG_ERR_ARGUMENT, "$KCG_EXTRA_FLAGS asks for a diagnostic build (-DKCG_DIAG_...: the kernel leaves work out and its "
                                  "result is wrong on purpose); set KCG_ALLOW_DIAG=1 to build it");

  const RtcLib& rtc = rtc_lib();           // one compiler for the whole call, whatever happens to the environment
  if (!rtc.api.ok) return fail(KCG_ERR_COMPILE, "hiprtc unavailable:" + rtc.api.error);
#define RTC(name) (rtc.api.p_##name)
  std::string flags_text;
  for (const auto& f : compile_flags()) flags_text += f + " ";
  {
    int major = 0, minor = 0;
    RTC(hiprtcVersion)(&major, &minor);
    flags_text += "hiprtc" + std::to_string(major) + "." + std::to_string(minor) + " " + rtc.identity + " ";
  }
  for (const auto& f : extra) flags_text += f + " ";
  if (!env_flag("KCG_SPILL_REBUILD", true)) flags_text += "first-build-kept ";
  uint64_t h = fnv1a(KCG_VERSION);
  h = fnv1a(arch, h);
  h = fnv1a(flags_text, h);
  h = fnv1a(stub, h);
  for (int i = 0; i < kNumDeviceHeaders; ++i) h = fnv1a(kDeviceHeaderSrcs[i], h);
  char hex[32];
  snprintf(hex, sizeof(hex), "%016llx", (unsigned long long)h);

  const std::string dir = cache_dir();
  if (!make_dirs(dir)) return fail(KCG_ERR_IO, "cannot create cache directory " + dir);
  const std::string stem = dir + "/" + name + "." + hex;
  const std::string path = stem + ".hsaco";
  if (path.size() >= sizeof(out->code_path)) return fail(KCG_ERR_IO, "code object path too long");
  memcpy(out->code_path, path.c_str(), path.size() + 1);
  // remembers that this very build (same sources, flags, compiler) spilled: no need to compile it again
  const std::string spill_marker = stem + ".spills";
  const std::string info_path = stem + ".buildinfo";

  if (!env_flag("KCG_CACHE_BYPASS", false)) {
    if (file_exists(path) && read_build_info(info_path, out)) {
      out->cache_hit = 1;
      g_err.clear();
      return KCG_OK;
    }
    if (direct && file_exists(spill_marker)) return kBuildSpills;
  }

  // one hiprtc build of the stub with the engine's flags, $KCG_EXTRA_FLAGS and `more` behind them
  auto compile = [&](const std::vector<std::string>& more, std::vector<char>* code) -> int {
    hiprtcProgram prog;
    hiprtcResult r = RTC(hiprtcCreateProgram)(&prog, stub.c_str(), "kcg_instance.hip", kNumDeviceHeaders,
                                              const_cast<const char**>(kDeviceHeaderSrcs),
                                              const_cast<const char**>(kDeviceHeaderNames));
    if (r != HIPRTC_SUCCESS) return fail(KCG_ERR_COMPILE, std::string("hiprtcCreateProgram: ") + RTC(hiprtcGetErrorString)(r));
    std::vector<std::string> opts = compile_flags();
    opts.push_back("--offload-arch=" + arch);
    for (const auto& f : extra) opts.push_back(f);
    for (const auto& f : more) opts.push_back(f);
    std::vector<const char*> optv;
    for (const auto& o : opts) optv.push_back(o.c_str());
    r = RTC(hiprtcCompileProgram)(prog, (int)optv.size(), optv.data());
    if (r != HIPRTC_SUCCESS) {
      size_t n = 0;
      RTC(hiprtcGetProgramLogSize)(prog, &n);
      std::string log(n, 0);
      if (n) RTC(hiprtcGetProgramLog)(prog, &log[0]);
      RTC(hiprtcDestroyProgram)(&prog);
      return fail(KCG_ERR_COMPILE, std::string("hiprtc: ") + RTC(hiprtcGetErrorString)(r) + " for " + name + "\n" + log);
    }
    size_t n = 0;
    r = RTC(hiprtcGetCodeSize)(prog, &n);
    code->assign(n, 0);
    if (r == HIPRTC_SUCCESS) r = RTC(hiprtcGetCode)(prog, code->data());
    RTC(hiprtcDestroyProgram)(&prog);
    if (r != HIPRTC_SUCCESS || n == 0) return fail(KCG_ERR_COMPILE, "hiprtc returned no code object");
    return KCG_OK;
  };
#undef RTC
  std::vector<char> code;
  if (int rc = compile({}, &code)) return rc;
  CodeMeta meta = CodeMeta::of(code);
  std::string note;
  // The direct-staging kernel reads LDS with instructions the compiler does not know to be
  // asynchronous: a fragment register spilled to scratch memory would be stored before its data has
  // arrived.  Such a build is never used (nor cached): the caller falls back to register staging.
  // (a code object whose metadata does not say counts as spilling: the kernel is not used unverified)
  if (direct && (!meta.known() || meta.scratch != 0 || meta.vgpr_spills > 0)) {
    const char text[] = "direct-staging build needs scratch memory (register spills); register staging is used instead\n";
    write_file_atomic(spill_marker, text, sizeof(text) - 1);
    return kBuildSpills;
  }
  // OPEN DEFECT, worked around: a register-staged or scalar kernel that the register allocator could not fit
  // (CodeMeta::under_pressure) is built once more at -O1, and that build is the one kept.  One such kernel
  // (fp64, one wave on a 64x64x64 tile with both prefetch flags, M=8 N=208 K=592: 512 registers, 1 KiB of
  // scratch per lane) returns wrong sums at -O2 and -O3 and the right ones at -O1; the cause inside the compiler
  // is not known.  All spilling kernels of a 1000-config random sample (184 of them) are right at -O1 and run
  // 9 % slower at the median.  Such configs never win a tuning run; they must still be right.
  // kcg_kernel_info.build_flags says which build a caller got.  $KCG_SPILL_REBUILD=0 keeps the first build.
  if (!direct && meta.under_pressure() && env_flag("KCG_SPILL_REBUILD", true)) {
    std::vector<char> calm;
    if (int rc = compile({"-O1"}, &calm)) return rc;
    code.swap(calm);
    out->build_flags |= KCG_BUILD_LOW_OPT;
    if (!meta.known()) {
      out->build_flags |= KCG_BUILD_META_UNKNOWN;
      note = "note: the code object's metadata does not state its register use; the kernel was rebuilt at -O1 as if it spilled";
    }
    meta = CodeMeta::of(code);
  }
  if (diagnostic) {
    out->build_flags |= KCG_BUILD_DIAGNOSTIC;
    std::string given;
    for (const auto& f : extra) given += (given.empty() ? "" : " ") + f;
    note = "note: diagnostic build (" + given + "): the result of this kernel is wrong on purpose";
  }
  if (declined) out->build_flags |= KCG_BUILD_DIRECT_DECLINED;
  out->scratch_bytes = (int32_t)meta.scratch;
  out->vgprs = (int32_t)meta.vgprs;
  out->sgpr_spills = (int32_t)meta.sgpr_spills;
  if (!write_file_atomic(path, code.data(), code.size())) return fail(KCG_ERR_IO, "cannot write " + path);
  write_build_info(info_path, *out);
  if (env_flag("KCG_KEEP_SOURCE", false)) {
    std::string sp = stem + ".hip";
    write_file_atomic(sp, stub.data(), stub.size());
  }
  g_err = note;
  return KCG_OK;
}

static int compile_entry(const kcg_matmul_cfg* cfg, const char* arch_in, int kind, int ex, kcg_kernel_info* out) {
  if (!cfg || !out) return fail(KCG_ERR_ARGUMENT, "null argument");
  kcg::MatmulConfig c = kcg::MatmulConfig::from(*cfg);
  std::string why;
  int k = resolve_kind(c, kind, &why);
  if (k < 0) return fail(k, "invalid config: " + why);
  const std::string arch = (arch_in && *arch_in) ? arch_in : "gfx950";
  int r = build_variant(c, k, /*allow_direct=*/true, arch, ex, out);
  if (r == kBuildSpills) r = build_variant(c, k, /*allow_direct=*/false, arch, ex, out);
  return r;
}

int kcg_compile_matmul(const kcg_matmul_cfg* cfg, const char* arch_in, int kind, kcg_kernel_info* out) {
  return compile_entry(cfg, arch_in, kind, -1, out);
}

int kcg_compile_matmul_ex(const kcg_matmul_cfg* cfg, const char* arch_in, int kind, int epilogue, kcg_kernel_info* out) {
  if (epilogue != KCG_EPILOGUE_NONE && epilogue != KCG_EPILOGUE_ALPHA_BETA) return fail(KCG_ERR_ARGUMENT, "unknown epilogue");
  return compile_entry(cfg, arch_in, kind, epilogue, out);
}

int kcg_code_object_info(const char* code_path, kcg_kernel_info* out) {
  if (!code_path || !out) return fail(KCG_ERR_ARGUMENT, "null argument");
  std::string p = code_path;
  const std::string ext = ".hsaco";
  if (p.size() <= ext.size() || p.compare(p.size() - ext.size(), ext.size(), ext) != 0)
    return fail(KCG_ERR_ARGUMENT, "not a code object of this library (no .hsaco suffix): " + p);
  memset(out, 0, sizeof(*out));
  if (p.size() >= sizeof(out->code_path)) return fail(KCG_ERR_IO, "code object path too long");
  memcpy(out->code_path, p.c_str(), p.size() + 1);
  if (!read_build_info(p.substr(0, p.size() - ext.size()) + ".buildinfo", out))
    return fail(KCG_ERR_IO, "no build record beside " + p + " (the code object was not written by kcg_compile_matmul)");
  g_err.clear();
  return KCG_OK;
}

int kcg_compiler_identity(char* out, int out_len) {
  const RtcLib& rtc = rtc_lib();
  if (!rtc.api.ok) return fail(KCG_ERR_COMPILE, "hiprtc unavailable:" + rtc.api.error);
  return copy_out(rtc.identity, out, out_len);
}

int kcg_load(const char* code_path, const char* kernel_name, int lds_bytes, int device, uint64_t* module,
             uint64_t* function, int32_t* n_regs, int32_t* n_spills) {
  if (!code_path || !kernel_name || !module || !function) return fail(KCG_ERR_ARGUMENT, "null argument");
  std::vector<char> code;
  if (!read_file(code_path, &code) || code.empty()) return fail(KCG_ERR_IO, std::string("cannot read code object ") + code_path);
  HIP_READY();
  HIP_TRY(HIPF(hipSetDevice)(device));
  hipModule_t mod;
  hipFunction_t fn;
  HIP_TRY(HIPF(hipModuleLoadData)(&mod, code.data()));
  hipError_t e = HIPF(hipModuleGetFunction)(&fn, mod, kernel_name);
  if (e != hipSuccess) {
    (void)HIPF(hipModuleUnload)(mod);
    return hip_fail(e, "hipModuleGetFunction");
  }
  if (lds_bytes > 64 * 1024) {
    e = hip_api().p_hipFuncSetAttribute
            ? hip_api().p_hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes)
            : hipErrorNotSupported;
    if (e != hipSuccess) {
      (void)HIPF(hipModuleUnload)(mod);
      return hip_fail(e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
    }
  }
  int regs = 0, local = 0;
  (void)HIPF(hipFuncGetAttribute)(&regs, HIP_FUNC_ATTRIBUTE_NUM_REGS, fn);
  (void)HIPF(hipFuncGetAttribute)(&local, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, fn);
  if (n_regs) *n_regs = regs;
  if (n_spills) *n_spills = local / 4;   // scratch dwords per lane; 0 means no spilling
  *module = (uint64_t)(uintptr_t)mod;
  *function = (uint64_t)(uintptr_t)fn;
  {
    const std::string name(kernel_name);
    auto ends = [&](const char* suffix) {
      const size_t n = strlen(suffix);
      return name.size() >= n && name.compare(name.size() - n, n, suffix) == 0;
    };
    int es[3];
    element_sizes_from_name(name, es);
    std::lock_guard<std::mutex> lock(g_loaded_mu);
    g_loaded[*function] = LoadedFunction{(ends("EX_") || ends("EXab_")) ? 8 : 3, *module, es[0], es[1], es[2]};
  }
  g_err.clear();
  return KCG_OK;
}

int kcg_launch(uint64_t function, const int32_t grid[3], const int32_t block[3], int lds_bytes, uint64_t stream,
               uint64_t a, uint64_t b, uint64_t c) {
  if (!function || !grid || !block) return fail(KCG_ERR_ARGUMENT, "null function / dims");
  if ((int64_t)grid[0] * grid[1] * grid[2] <= 0) return KCG_OK;  // empty grid: nothing to do
  if (!a || !b || !c) return fail(KCG_ERR_ARGUMENT, "null device pointer");
  if ((a | b | c) & 15) return fail(KCG_ERR_ARGUMENT, "a, b and c must be 16-byte aligned");
  if (loaded_args(function) == 8) return fail(KCG_ERR_ARGUMENT, "this kernel has the batched-strided form: use kcg_launch_batched");
  void* pa = (void*)(uintptr_t)a;
  void* pb = (void*)(uintptr_t)b;
  void* pc = (void*)(uintptr_t)c;
  void* params[3] = {&pa, &pb, &pc};
  HIP_READY();
  HIP_TRY(HIPF(hipModuleLaunchKernel)((hipFunction_t)(uintptr_t)function, grid[0], grid[1], grid[2], block[0], block[1],
                                block[2], lds_bytes, (hipStream_t)(uintptr_t)stream, params, nullptr));
  return KCG_OK;
}

int kcg_launch_batched(uint64_t function, const int32_t grid[3], const int32_t block[3], int lds_bytes, uint64_t stream,
                       uint64_t a, uint64_t b, uint64_t c, int32_t batch, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                       float alpha, float beta) {
  if (!function || !grid || !block) return fail(KCG_ERR_ARGUMENT, "null function / dims");
  if (batch < 0 || batch > 65535) return fail(KCG_ERR_ARGUMENT, "batch must be in [0, 65535]");
  if (stride_a < 0 || stride_b < 0 || stride_c < 0) return fail(KCG_ERR_ARGUMENT, "strides must not be negative");
  if (batch > 1 && stride_c == 0) return fail(KCG_ERR_ARGUMENT, "stride_c = 0 would make the problems of a batch write the same C");
  if ((int64_t)grid[0] * grid[1] * grid[2] <= 0 || batch == 0) return KCG_OK;  // nothing to do
  if (grid[1] != 1 || grid[2] != 1) return fail(KCG_ERR_ARGUMENT, "the batch goes on grid[1]: grid must be {n, 1, 1}");
  if (!a || !b || !c) return fail(KCG_ERR_ARGUMENT, "null device pointer");
  if ((a | b | c) & 15) return fail(KCG_ERR_ARGUMENT, "a, b and c must be 16-byte aligned");
  const LoadedFunction lf = loaded_function(function);
  if (lf.n_args == 3) return fail(KCG_ERR_ARGUMENT, "this kernel has the three-pointer form: use kcg_launch");
  // problem z starts stride * z elements into each buffer and must be as aligned as problem 0: the kernels move
  // 16-byte vectors relative to the start of a matrix
  if (batch > 1 && ((stride_a * lf.es_a) % 16 || (stride_b * lf.es_b) % 16 || (stride_c * lf.es_c) % 16))
    return fail(KCG_ERR_ARGUMENT, "stride_a, stride_b and stride_c must be multiples of 16 bytes (every problem of a batch "
                                  "must start 16-byte aligned)");
  void* pa = (void*)(uintptr_t)a;
  void* pb = (void*)(uintptr_t)b;
  void* pc = (void*)(uintptr_t)c;
  long sa = (long)stride_a, sb = (long)stride_b, sc = (long)stride_c;
  void* params[8] = {&pa, &pb, &pc, &sa, &sb, &sc, &alpha, &beta};
  HIP_READY();
  HIP_TRY(HIPF(hipModuleLaunchKernel)((hipFunction_t)(uintptr_t)function, grid[0], batch, 1, block[0], block[1], block[2],
                                lds_bytes, (hipStream_t)(uintptr_t)stream, params, nullptr));
  return KCG_OK;
}

// The timing loop shared by kcg_benchmark and kcg_benchmark_batched: `launch` starts the kernel once on `stream`.
extern "C++" {
template <class Launch>
static int timing_loop(uint64_t stream, int warmup, int iters, int reps, float* median_ms, float* min_ms, Launch launch) {
  if (iters <= 0) return fail(KCG_ERR_ARGUMENT, "iters must be positive");
  hipStream_t st = (hipStream_t)(uintptr_t)stream;
  hipEvent_t e0, e1;
  HIP_READY();
  HIP_TRY(HIPF(hipEventCreate)(&e0));
  {
    hipError_t e = HIPF(hipEventCreate)(&e1);
    if (e != hipSuccess) {
      (void)HIPF(hipEventDestroy)(e0);
      return hip_fail(e, "hipEventCreate");
    }
  }
  int rc = KCG_OK;
  std::vector<float> samples;
  auto timed = [&](int n, float* ms) -> int {
    hipError_t e = HIPF(hipEventRecord)(e0, st);
    if (e != hipSuccess) return hip_fail(e, "hipEventRecord");
    for (int i = 0; i < n; ++i) {
      int r = launch();
      if (r != KCG_OK) return r;
    }
    e = HIPF(hipEventRecord)(e1, st);
    if (e != hipSuccess) return hip_fail(e, "hipEventRecord");
    e = HIPF(hipEventSynchronize)(e1);
    if (e != hipSuccess) return hip_fail(e, "hipEventSynchronize");
    e = HIPF(hipEventElapsedTime)(ms, e0, e1);
    if (e != hipSuccess) return hip_fail(e, "hipEventElapsedTime");
    return KCG_OK;
  };
  for (int i = 0; i < warmup && rc == KCG_OK; ++i) rc = launch();
  if (rc == KCG_OK) {
    hipError_t e = HIPF(hipStreamSynchronize)(st);
    if (e != hipSuccess) rc = hip_fail(e, "hipStreamSynchronize");
  }
  if (rc == KCG_OK && reps <= 0) {
    float probe = 0.f;
    rc = timed(1, &probe);
    if (rc == KCG_OK) {
      reps = probe > 0.f ? (int)(1.0f / probe) + 1 : 1;
      if (reps > 1000) reps = 1000;
    }
  }
  for (int i = 0; i < iters && rc == KCG_OK; ++i) {
    float ms = 0.f;
    rc = timed(reps, &ms);
    if (rc == KCG_OK) samples.push_back(ms / (float)reps);
  }
  (void)HIPF(hipEventDestroy)(e0);
  (void)HIPF(hipEventDestroy)(e1);
  if (rc != KCG_OK) return rc;
  std::sort(samples.begin(), samples.end());
  const size_t n = samples.size();
  if (median_ms) *median_ms = (n % 2) ? samples[n / 2] : 0.5f * (samples[n / 2 - 1] + samples[n / 2]);
  if (min_ms) *min_ms = samples[0];
  return KCG_OK;
}
}  // extern "C++"

int kcg_benchmark(uint64_t function, const int32_t grid[3], const int32_t block[3], int lds_bytes, uint64_t stream,
                  uint64_t a, uint64_t b, uint64_t c, int warmup, int iters, int reps, float* median_ms,
                  float* min_ms) {
  return timing_loop(stream, warmup, iters, reps, median_ms, min_ms,
                     [&]() { return kcg_launch(function, grid, block, lds_bytes, stream, a, b, c); });
}

int kcg_benchmark_batched(uint64_t function, const int32_t grid[3], const int32_t block[3], int lds_bytes, uint64_t stream,
                          uint64_t a, uint64_t b, uint64_t c, int32_t batch, int64_t stride_a, int64_t stride_b,
                          int64_t stride_c, float alpha, float beta, int warmup, int iters, int reps, float* median_ms,
                          float* min_ms) {
  return timing_loop(stream, warmup, iters, reps, median_ms, min_ms, [&]() {
    return kcg_launch_batched(function, grid, block, lds_bytes, stream, a, b, c, batch, stride_a, stride_b, stride_c, alpha, beta);
  });
}

int kcg_unload(uint64_t module) {
  if (!module) return fail(KCG_ERR_ARGUMENT, "null module");
  HIP_READY();
  {
    std::lock_guard<std::mutex> lock(g_loaded_mu);
    for (auto it = g_loaded.begin(); it != g_loaded.end();) it = it->second.module == module ? g_loaded.erase(it) : std::next(it);
  }
  HIP_TRY(HIPF(hipModuleUnload)((hipModule_t)(uintptr_t)module));
  return KCG_OK;
}

int kcg_device_info(int device, int32_t* cu_count, int32_t* clock_khz, int32_t* lds_per_block, char* arch_name,
                    int arch_len) {
  hipDeviceProp_t p;
  HIP_READY();
  HIP_TRY(HIPF(hipGetDeviceProperties)(&p, device));
  if (cu_count) *cu_count = p.multiProcessorCount;
  if (clock_khz) *clock_khz = p.clockRate;
  if (lds_per_block) *lds_per_block = (int32_t)p.sharedMemPerBlock;
  copy_out(p.gcnArchName, arch_name, arch_len);
  return KCG_OK;
}

}  // extern "C"
