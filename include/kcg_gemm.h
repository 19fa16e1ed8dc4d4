/*
 * kcg_gemm.h — C ABI of libkcg_gemm.so, the MI355X (gfx950) GEMM engine that sits behind the
 * KCG operator API: a 31-integer tuning config goes in, a gfx950 code object containing one
 * kernel `GEMM_MNK…` (three device-pointer arguments, dynamic LDS) comes out, is loaded, launched on
 * caller-owned device buffers and timed.
 *
 * Every entry point is plain C (pointers, sizes, integers); nothing here depends on Python or torch.
 * Functions return 0 on success and a negative kcg_status on failure; the failure text is kept in a
 * thread-local buffer readable with kcg_last_error().  Nothing throws across this boundary.
 *
 * Each declaration names the reference interface it stands in for (paths relative to the KCG tree).
 */
#ifndef KCG_GEMM_H
#define KCG_GEMM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes -------------------------------------------------------------------------- */
enum kcg_status {
  KCG_OK = 0,
  KCG_ERR_INVALID_CONFIG = -1, /* config fails a validity predicate (see kcg_check_config)     */
  KCG_ERR_COMPILE = -2,        /* hiprtc rejected the instantiation; log in kcg_last_error()    */
  KCG_ERR_IO = -3,             /* cache directory / code-object file problem                    */
  KCG_ERR_HIP = -4,            /* a HIP runtime call failed: "KCG Error[HIP]: Code: N, …"       */
  KCG_ERR_ARGUMENT = -5        /* null pointer, bad size, bad handle                            */
};

/* ---- dtype codes: KcgDtype, include/Common/Utils.h:110-120 == EnumKernelDType, Utils.py:198-209.
 * bfloat16 is an addition of this engine (the reference has no bf16 code); 3 keeps `code % 30`
 * from colliding and is NOT the byte size — use kcg_dtype_size(). */
enum kcg_dtype {
  KCG_DT_FLOAT16 = 2,
  KCG_DT_BFLOAT16 = 3,
  KCG_DT_FLOAT32 = 4,
  KCG_DT_FLOAT64 = 8
};

/* ---- the tuning config: 31 int32 in the argument order of compile_kernel_matmul,
 * src/main.cc:64-96 (Python caller Runtime/python/kcg/KCGCompiler.py:14-45). */
enum kcg_cfg_index {
  KCG_BLOCK_SIZE_M = 0, KCG_BLOCK_SIZE_N, KCG_BLOCK_SIZE_K,
  KCG_THREAD_SIZE_M, KCG_THREAD_SIZE_N, KCG_WARP_SIZE,
  KCG_BLOCK_LAYOUT_M, KCG_BLOCK_LAYOUT_N, KCG_WARP_LAYOUT_M, KCG_WARP_LAYOUT_N,
  KCG_GLOB_LOAD_WIDTH_A, KCG_GLOB_LOAD_WIDTH_B,
  KCG_WARP_SCATTER_WIDTH_A, KCG_WARP_SCATTER_WIDTH_B,
  KCG_THREAD_SCATTER_WIDTH_A, KCG_THREAD_SCATTER_WIDTH_B,
  KCG_LOCAL_SPLIT_U, KCG_BLOCK_MAPPING, KCG_GLOB_STORE_WIDTH,
  KCG_UNROLL_NUM, KCG_REG_PREFETCH, KCG_SHARED_PREFETCH, KCG_LOAD_CONTINUOUS, KCG_REDUCE_C_CONTINUOUS,
  KCG_DTYPE_A, KCG_DTYPE_B, KCG_DTYPE_C,
  KCG_M, KCG_N, KCG_K,
  KCG_IS_ATRANS,
  KCG_CFG_LEN /* == 31 */
};

typedef struct kcg_matmul_cfg {
  int32_t v[31];
} kcg_matmul_cfg;

/* Which kernel family an instantiation uses. */
enum kcg_kernel_kind {
  KCG_KIND_AUTO = 0, /* MFMA when the wave tile can be covered by MFMA tiles, else SIMT          */
  KCG_KIND_SIMT = 1, /* scalar-FMA register-tiled kernel that follows the config literally        */
  KCG_KIND_MFMA = 2  /* wave-tiled matrix-core kernel                                            */
};

/* Result of a compile: KernelInfo (include/Common/Utils.h:131-136) + the dynamic-LDS byte count the
 * reference recomputes in UserInputs.sharedMem() (Runtime/python/kcg/CompiledKernelFactory.py:30-44). */
typedef struct kcg_kernel_info {
  char code_path[1024];  /* gfx950 code object on disk (the reference's hsacoPath)                */
  char kernel_name[512]; /* symbol inside it == reference kernel name (src/main.cc:119-145)       */
  int32_t grid[3];
  int32_t block[3];
  int32_t lds_bytes;     /* dynamic LDS to pass at launch                                          */
  int32_t kind;          /* kcg_kernel_kind actually chosen                                        */
  int32_t cache_hit;     /* 1 if the code object came from the on-disk cache                       */
  int32_t build_flags;   /* kcg_build_flag bits: how this code object was built                    */
  int32_t scratch_bytes; /* scratch memory per lane (register spills), -1: the code object does not say */
  int32_t vgprs;         /* vector + accumulation registers per lane (of 512), -1: unknown          */
  int32_t sgpr_spills;   /* scalar registers spilled into vector-register lanes, -1: unknown        */
} kcg_kernel_info;

/* How a code object was built (kcg_kernel_info.build_flags). */
enum kcg_build_flag {
  KCG_BUILD_LOW_OPT = 1,         /* built at -O1: the -O3 build ran out of vector registers (scratch memory, vector
                                  * spills or all 512 registers taken); one such -O3 build is known to compute wrong
                                  * sums, cause unknown, so none is handed out.  Typically ~10 % slower.           */
  KCG_BUILD_DIAGNOSTIC = 2,      /* $KCG_EXTRA_FLAGS held a -DKCG_DIAG_ flag (needs KCG_ALLOW_DIAG=1): this kernel
                                  * leaves work out and its result is WRONG on purpose                            */
  KCG_BUILD_DIRECT_DECLINED = 4, /* the config selects the direct-staging kernel, but that build would spill: this is
                                  * the register-staged kernel                                                    */
  KCG_BUILD_META_UNKNOWN = 8     /* the code object's metadata did not state its register use (treated as spilling) */
};

/* ---- config semantics (host only, no GPU needed) ------------------------------------------- */

/* Keyword string of config slot i ("BLOCK_SIZE_M", …): include/Common/Utils.h:186-217 ==
 * ConfigKeywords, Runtime/python/kcg/Utils.py:359-390.  NULL if i is out of range. */
const char* kcg_cfg_keyword(int index);

/* Bytes per element of a kcg_dtype, 0 if unknown (reference: sizeof(), Utils.py:219-221). */
int kcg_dtype_size(int dtype);

/* Validity of a config for this engine.  Folds KernelArgMatmul.check() (Operators/matmul.py:180-194),
 * TuningSpaceChecker_Matmul.check_warp/check_size (matmul.py:267-313) and the divisibility rules the
 * reference schedule assumes silently (Optimizer.cc:10-36,310-329; Rewriter.cc:427-441,603-610) into
 * one predicate; problem sizes need NOT be multiples of the block tile (edge tiles are predicated).
 * `kind` is a kcg_kernel_kind; with KCG_KIND_AUTO the config is valid if either family accepts it.
 * Returns KCG_OK or KCG_ERR_INVALID_CONFIG with the reason in kcg_last_error(). */
int kcg_check_config(const kcg_matmul_cfg* cfg, int kind);

/* Kernel family KCG_KIND_AUTO resolves to for this config (KCG_KIND_SIMT / KCG_KIND_MFMA),
 * or KCG_ERR_INVALID_CONFIG. */
int kcg_select_kind(const kcg_matmul_cfg* cfg);

/* Kernel name, byte-for-byte the string MatmulParams::getKernelName() builds (src/main.cc:119-145).
 * Returns the length written (excluding NUL) or a negative status. */
int kcg_kernel_name(const kcg_matmul_cfg* cfg, char* out, int out_len);

/* Launch geometry: grid = ceil(M/BM)*ceil(N/BN) x1x1, block = (BM/TM)*(BN/TN)*LOCAL_SPLIT_U x1x1
 * (Optimizer.cc:302-303,314,336; LoweringPasses.cc:303-313), padded to 3 dims like main.cc:335-342. */
int kcg_launch_dims(const kcg_matmul_cfg* cfg, int32_t grid[3], int32_t block[3]);

/* Dynamic LDS bytes by the reference's own formula (CompiledKernelFactory.py:30-44). */
int kcg_reference_lds_bytes(const kcg_matmul_cfg* cfg);

/* Block swizzle of Rewriter::BlockMapping (Rewriter.cc:726-761): linear block id -> (by, bx).
 * With xcd_remap != 0 the id is first passed through the engine's XCD remap (hardware block ids are
 * dealt round-robin to the XCDs — 8 on an MI355X, or $KCG_NUM_XCDS — and the remap gives each XCD one
 * contiguous part of the swizzled order so neighbouring tiles share that XCD's L2); applied only when the
 * block count is a multiple of the XCD count.  The kernels are built with the remap unless KCG_XCD_REMAP=0. */
int kcg_block_mapping(const kcg_matmul_cfg* cfg, int bid, int xcd_remap, int32_t* by, int32_t* bx);

/* ---- compile: replaces compile_kernel_matmul (src/main.cc:315-357) -------------------------- */

/* Instantiates the hand-written gfx950 kernel template for `cfg`, builds it with hiprtc for `arch`
 * ("gfx950"; NULL means "gfx950") and writes the code object into the cache directory
 * ($KCG_CACHE_DIR, default "<dir of this library>/_kcg_cache").  A second call with the same config,
 * kind, arch and kernel source is a cache hit and does not compile.  `kind` is a kcg_kernel_kind.
 * Thread-safe and re-entrant; needs no GPU.
 * KCG_ERR_INVALID_CONFIG: the config breaks a rule (text says which), nothing was compiled.
 * KCG_ERR_COMPILE: hiprtc failed.
 * A config that selects the direct-staging kernel but whose build would spill registers to scratch memory
 * (that kernel cannot tolerate spills) gets the register-staged kernel instead (out->build_flags says so); a
 * "<name>.<hash>.spills" marker in the cache directory remembers the decision.
 * KCG_ERR_ARGUMENT: $KCG_EXTRA_FLAGS names a -DKCG_DIAG_ switch (a build that is wrong on purpose) without
 * KCG_ALLOW_DIAG=1.  On KCG_OK kcg_last_error() is "" or a line that starts with "note:". */
int kcg_compile_matmul(const kcg_matmul_cfg* cfg, const char* arch, int kind, kcg_kernel_info* out);

/* What kcg_compile_matmul recorded about a code object it wrote (the "<name>.<hash>.buildinfo" file beside it):
 * fills lds_bytes, kind, build_flags, scratch_bytes, vgprs and sgpr_spills of *out (code_path is copied, the other
 * fields are zero).  Lets a caller that holds only (path, kernel name, config) — the reference's UserInputs,
 * Runtime/python/kcg/CompiledKernelFactory.py:19-28, which recomputes the LDS size from the config — launch the
 * kernel with the size that belongs to this very code object.  KCG_ERR_IO when there is no such record. */
int kcg_code_object_info(const char* code_path, kcg_kernel_info* out);

/* Which compiler kcg_compile_matmul uses right now: "hiprtc:<path of the library>:<its size>" (part of the cache
 * key: hiprtcVersion() does not tell ROCm releases apart).  Default: the hiprtc the process already carries, else
 * the system's.  $KCG_HIPRTC_LIB=<path of a libhiprtc.so> selects another one, loaded in a link namespace of
 * its own so that it brings its own compiler library along; read at every compile.  The reference's counterpart
 * is the fixed LLVM it links (src/lib/Target/HSACOTranslation.cc:153-257).  Returns the length or a negative status. */
int kcg_compiler_identity(char* out, int out_len);

/* ---- batched / strided GEMM with an alpha-beta epilogue ---------------------------------------------
 * The reference has neither: it lists batched GEMM as the next step of its roadmap (结果汇总.md:21-22) and
 * profiles its kernels against the vendor sgemm, whose call carries alpha, beta and leading dimensions
 * (runRoc.cpp:27-28,53-66).  These two entry points give the engine that call shape. */
enum kcg_epilogue {
  KCG_EPILOGUE_NONE = 0,       /* C = A B                                   (alpha, beta ignored)   */
  KCG_EPILOGUE_ALPHA_BETA = 1  /* C = alpha * (A B) + beta * C; beta == 0: C is not read (as in BLAS) */
};

/* Like kcg_compile_matmul, but the kernel takes (A, B, C, stride_a, stride_b, stride_c, alpha, beta) and
 * computes problem z of a batch on grid row z from the buffers z * stride_* elements further on.  Same
 * template, same tuning config, same cache; the kernel symbol is the reference name followed by "EX_"
 * (no epilogue) or "EXab_" (alpha-beta epilogue).  Launch it with kcg_launch_batched only. */
int kcg_compile_matmul_ex(const kcg_matmul_cfg* cfg, const char* arch, int kind, int epilogue, kcg_kernel_info* out);

/* Launches `batch` problems of a kernel built by kcg_compile_matmul_ex: grid = {info.grid[0], batch, 1}.
 * stride_* are in elements of the respective buffer; stride_a or stride_b may be 0 (one operand shared by
 * the whole batch), stride_c may not (unless batch == 1).  batch <= 65535; batch == 0 launches nothing.
 * For batch > 1 every stride must be a multiple of 16 bytes (stride * element size): each problem has to start as
 * aligned as the first one (checked for functions that kcg_load handed out; KCG_ERR_ARGUMENT otherwise).
 * alpha and beta are read only by a kernel with KCG_EPILOGUE_ALPHA_BETA.  Asynchronous on `stream`. */
int kcg_launch_batched(uint64_t function, const int32_t grid[3], const int32_t block[3], int lds_bytes,
                       uint64_t stream, uint64_t a, uint64_t b, uint64_t c, int32_t batch,
                       int64_t stride_a, int64_t stride_b, int64_t stride_c, float alpha, float beta);

/* kcg_benchmark for a kernel of the batched-strided form: the same timing loop around kcg_launch_batched (one
 * launch = the whole batch).  With beta != 0 every launch reads what the previous one wrote to C. */
int kcg_benchmark_batched(uint64_t function, const int32_t grid[3], const int32_t block[3], int lds_bytes,
                          uint64_t stream, uint64_t a, uint64_t b, uint64_t c, int32_t batch,
                          int64_t stride_a, int64_t stride_b, int64_t stride_c, float alpha, float beta,
                          int warmup, int iters, int reps, float* median_ms, float* min_ms);

/* The HIP source text that kcg_compile_matmul would hand to hiprtc for this config (the generated
 * instantiation stub; the template header is embedded in the library).  Returns bytes needed. */
int kcg_instantiation_source(const kcg_matmul_cfg* cfg, int kind, char* out, int out_len);

/* ---- load / launch: replace load_binary (loaderCCode/hip.c:60-133) and the generated
 * launch() stub (HIPLauncher.py:107-141,189-238) ------------------------------------------------ */

/* Reads the code object file, hipModuleLoadData + hipModuleGetFunction on `device`; raises the
 * function's dynamic-LDS limit when lds_bytes > 64 KiB.  n_regs / n_spills as hip.c:115-121. */
int kcg_load(const char* code_path, const char* kernel_name, int lds_bytes, int device,
             uint64_t* module, uint64_t* function, int32_t* n_regs, int32_t* n_spills);

/* hipModuleLaunchKernel(function, grid, block, lds_bytes, stream, {&a,&b,&c}); asynchronous on the
 * caller's stream (0 = null stream).  Skips the launch when the grid is empty (HIPLauncher.py:138).
 * a/b/c are device addresses owned by the caller, 16-byte aligned (what hipMalloc and torch hand out: the kernels
 * move 16-byte vectors; rows inside the matrices may start anywhere).  A function that kcg_load handed out for a kernel of
 * the batched-strided form (kcg_compile_matmul_ex) is refused with KCG_ERR_ARGUMENT: its parameter block
 * has eight entries (and kcg_launch_batched refuses a three-pointer kernel likewise). */
int kcg_launch(uint64_t function, const int32_t grid[3], const int32_t block[3], int lds_bytes,
               uint64_t stream, uint64_t a, uint64_t b, uint64_t c);

/* (For kernels built by kcg_compile_matmul only: it launches with the three-pointer argument list.)
 * The timing loop of PerfTester._test_perf (KCGTask.py:162-181) done in C with HIP events on
 * `stream`: `warmup` untimed launches, then `iters` samples; each sample brackets `reps` back-to-back
 * launches (reps <= 0: chosen so one sample lasts >= 1 ms) and is divided by reps.
 * Outputs per-launch median and minimum in milliseconds. */
int kcg_benchmark(uint64_t function, const int32_t grid[3], const int32_t block[3], int lds_bytes,
                  uint64_t stream, uint64_t a, uint64_t b, uint64_t c,
                  int warmup, int iters, int reps, float* median_ms, float* min_ms);

int kcg_unload(uint64_t module);

/* Device facts the roofline report needs: CU count, max engine clock (kHz), LDS per workgroup. */
int kcg_device_info(int device, int32_t* cu_count, int32_t* clock_khz, int32_t* lds_per_block,
                    char* arch_name, int arch_len);

/* Thread-local text of the last failure in this thread ("" if none). */
const char* kcg_last_error(void);

/* Library version string. */
const char* kcg_version(void);

#ifdef __cplusplus
}
#endif
#endif /* KCG_GEMM_H */
