// kcg_runner — stand-alone (no Python) runner for the engine's GEMM kernels on one GPU.
//
// It plays the role of the reference's C++ check programs: runkernel.cpp (load a code object given on
// the command line, launch it several times, compare against a naive GPU kernel with an absolute
// tolerance of 0.01, runkernel.cpp:49-112) and the main() of matmul.cpp (HIP-event timing, TFLOPS
// print, naive `gemm_kernel` + `verify_kernel`, matmul.cpp:2327-2348,2386-2553).
//
//   kcg_runner --config <file.json> [--index i] [--kind auto|simt|mfma] [--iters n] [--tol t]
//              [--dist uniform|normal] [--timeline 1|2] [--dump-c file] [--diag "-DKCG_DIAG_..."]
//       compiles entry i of a {"cfgs": [...]} file (or a single flat config object) through
//       libkcg_gemm.so, loads it, verifies it against the naive kernel and times it
//       (--compile-only 1 stops after the compile: fills the code-object cache on a host without a GPU).
//       --dist: operands uniform on [-1,1) (default) or normal(0, 0.5), the distribution the 16-bit
//       benchmark uses (on a power-limited part the speed of a matrix-core kernel depends on the data).
//       --dump-c: writes the kernel's C (raw fp32, row-major) so that it can be checked outside this program; the
//       inputs are a pure function of the shape: a 64-bit LCG (seed 0x4B4347) fills A[M,K] then B[K,N] in row-major order.
//       --timeline: builds the direct-staging kernel with its in-kernel time stamps (-DKCG_TIMELINE=level
//       added to $KCG_EXTRA_FLAGS), runs it back to back and prints where the time of one launch goes:
//       block start, first K tile landed, K loop done, C stores issued / acknowledged, per XCD and over
//       all waves, the shader clock during the K loop, and the gap to the next launch.
//       --diag: adds the given switches to $KCG_EXTRA_FLAGS and sets KCG_ALLOW_DIAG=1: a build of the direct-staging
//       kernel that leaves part of its work out, to time what is left.  Its result is wrong on purpose; the
//       verification is still printed, but does not decide the exit status.
//   kcg_runner M N K gridX blockX <code-object> <kernel-name> [ldsBytes] [dtypeCode] [isATrans]
//       the reference runner's argument list (runkernel.cpp:63-66): launches an existing code object
//
// Two micro-benchmarks of the GPU itself live in kcg_probes.hip and are only dispatched from here:
//   kcg_runner --mfma-peak [dtype: f16|bf16]
//       what the matrix pipeline of this GPU sustains with nothing else going on: a loop of independent
//       matrix-core instructions on register operands, timed over ~0.3 s per case, for both 16-bit
//       instruction shapes and for operands of all zeros and of normal(0, 0.5) values.  On a
//       power-limited part the second figure is the ceiling of any GEMM on such data.  Also prints how long
//       the blocks of each of the eight XCDs took in the last launch (the XCDs do not run at one clock).
//
//   kcg_runner --launch-cost
//       the fixed costs a short GEMM pays per launch on this GPU: the period of back-to-back launches of
//       an empty kernel (1 block; 256 blocks; 256 blocks with 64 KiB of LDS each) and of a kernel that
//       only writes 64 MiB (the fp32 result of a 4096 x 4096 product); and, on a line of its own before that,
//       when a global->LDS fetch issued behind 32 stores of the same wave lands and when the wave's counter says so
//
// Build: make -C codegendemo_amd/csrc runner      (hipcc --offload-arch=gfx950)
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

#include "../../include/kcg_gemm.h"
#include "kcg_probes.h"

#define HIP_OK(x)                                                                      \
  do {                                                                                 \
    hipError_t e_ = (x);                                                               \
    if (e_ != hipSuccess) {                                                            \
      fprintf(stderr, "HIP error %d (%s) at %s:%d\n", (int)e_, hipGetErrorString(e_), __FILE__, __LINE__); \
      exit(3);                                                                         \
    }                                                                                  \
  } while (0)

// ---- naive reference kernel: one thread per C element, fp32 accumulation in ascending k -------------
// (gemm_kernel, matmul.cpp:2327-2337, for both A layouts and any input type)
template <class T>
__global__ void gemm_naive(const T* __restrict__ A, const T* __restrict__ B, float* __restrict__ D, int M, int N, int K,
                           int a_trans) {
  const int col = blockIdx.x * blockDim.x + threadIdx.x;
  const int row = blockIdx.y * blockDim.y + threadIdx.y;
  if (row >= M || col >= N) return;
  float acc = 0.f;
  for (int k = 0; k < K; ++k) {
    const float a = a_trans ? (float)A[(size_t)k * M + row] : (float)A[(size_t)row * K + k];
    acc += a * (float)B[(size_t)k * N + col];
  }
  D[(size_t)row * N + col] = acc;
}

// ---- compare kernel: counts |C - D| >= tol (NaN counts), keeps the largest error and the first offender
// (verify_kernel, matmul.cpp:2339-2348 printed offenders from the device; here they are counted)
template <class TC>
__global__ void verify(const TC* __restrict__ C, const float* __restrict__ D, size_t n, float tol,
                       unsigned long long* bad, unsigned int* max_err_bits, unsigned long long* first_bad) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float err = fabsf((float)C[i] - D[i]);
  if (!(err < tol)) {
    atomicAdd(bad, 1ull);
    atomicMin(first_bad, (unsigned long long)i);
  }
  if (err == err) atomicMax(max_err_bits, __float_as_uint(err));
}


static float lcg_uniform(uint64_t& s) {   // [-1, 1)
  s = s * 6364136223846793005ull + 1442695040888963407ull;
  return (float)((int32_t)(s >> 40) - (1 << 23)) / (float)(1 << 23);
}

static float lcg_normal(uint64_t& st, float std) {   // Box-Muller on two uniforms
  st = st * 6364136223846793005ull + 1442695040888963407ull;
  const float u1 = ((float)(st >> 40) + 1.0f) / 16777217.0f;
  st = st * 6364136223846793005ull + 1442695040888963407ull;
  const float u2 = (float)(st >> 40) / 16777216.0f;
  return sqrtf(-2.0f * logf(u1)) * cosf(6.2831853f * u2) * std;
}

template <class T>
static void* upload(const std::vector<float>& h) {
  std::vector<T> t(h.size());
  for (size_t i = 0; i < h.size(); ++i) t[i] = (T)h[i];
  void* d;
  HIP_OK(hipMalloc(&d, t.size() * sizeof(T)));
  HIP_OK(hipMemcpy(d, t.data(), t.size() * sizeof(T), hipMemcpyHostToDevice));
  return d;
}

// ---- where the time of one launch goes: reads the records a -DKCG_TIMELINE kernel writes (layout: see
// kcg_device_direct.h) for the last of `launches` back-to-back launches -----------------------------
static int timeline_report(uint64_t module, uint64_t function, const kcg_kernel_info& info, int waves_per_block,
                           uint64_t dA, uint64_t dB, uint64_t dC, double flops, int level) {
  const int TLW = 8;
  const size_t nrec = (size_t)info.grid[0] * waves_per_block;
  unsigned long long* d_rec;
  HIP_OK(hipMalloc(&d_rec, nrec * TLW * sizeof(unsigned long long)));
  HIP_OK(hipMemset(d_rec, 0, nrec * TLW * sizeof(unsigned long long)));
  hipDeviceptr_t sym;
  size_t sym_bytes = 0;
  if (hipModuleGetGlobal(&sym, &sym_bytes, (hipModule_t)(uintptr_t)module, "kcg_timeline_ptr") != hipSuccess || sym_bytes != sizeof(void*)) {
    fprintf(stderr, "this kernel carries no time stamps (only the direct-staging kernel does)\n");
    HIP_OK(hipFree(d_rec));
    return 2;
  }
  HIP_OK(hipMemcpy((void*)sym, &d_rec, sizeof(void*), hipMemcpyHostToDevice));
  const int warm = 300, launches = 100;
  for (int i = 0; i < warm; ++i) kcg_launch(function, info.grid, info.block, info.lds_bytes, 0, dA, dB, dC);
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0)); HIP_OK(hipEventCreate(&e1));
  HIP_OK(hipEventRecord(e0, 0));
  for (int i = 0; i < launches; ++i) kcg_launch(function, info.grid, info.block, info.lds_bytes, 0, dA, dB, dC);
  HIP_OK(hipEventRecord(e1, 0));
  HIP_OK(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  const double period_us = ms * 1e3 / launches;
  std::vector<unsigned long long> h(nrec * TLW);
  HIP_OK(hipMemcpy(h.data(), d_rec, h.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost));
  // the module must not keep the address of a freed buffer: a later launch would write its stamps there
  unsigned long long* const none = nullptr;
  HIP_OK(hipMemcpy((void*)sym, &none, sizeof(void*), hipMemcpyHostToDevice));
  HIP_OK(hipFree(d_rec));

  unsigned long long t0 = ~0ull;
  for (size_t r = 0; r < nrec; ++r) if (h[r * TLW] && h[r * TLW] < t0) t0 = h[r * TLW];
  struct Stat { double mn = 1e30, mx = -1e30, sum = 0; long n = 0; void add(double v) { mn = v < mn ? v : mn; mx = v > mx ? v : mx; sum += v; ++n; } double mean() const { return n ? sum / n : 0; } };
  const char* names[5] = {"block_start", "first_tile_landed", "k_loop_done", "stores_issued", "stores_acknowledged"};
  Stat all[5], xcd_loop[8], xcd_tail[8], xcd_end[8], clk, barrier;
  for (size_t r = 0; r < nrec; ++r) {
    const unsigned long long* w = &h[r * TLW];
    if (!w[0]) continue;
    for (int p = 0; p < 5; ++p) all[p].add((double)(w[p] - t0) * 0.01);            // 100 MHz -> us
    const int xcd = (int)((w[6] >> 32) & 0xF) % 8;
    const double loop_us = (double)(w[2] - w[1]) * 0.01;
    xcd_loop[xcd].add(loop_us);
    xcd_tail[xcd].add((double)(w[4] - w[2]) * 0.01);
    xcd_end[xcd].add((double)(w[4] - t0) * 0.01);
    if (loop_us > 0) clk.add((double)w[5] / loop_us);                               // cycles per us = MHz
    if (level >= 2 && w[5]) barrier.add(100.0 * (double)w[7] / (double)w[5]);
  }
  printf("{\"timeline\": {\"kernel\": \"%s\", \"level\": %d, \"launch_period_us\": %.2f, \"tflops\": %.1f, \"waves\": %ld,\n", info.kernel_name, level,
         period_us, flops / (period_us * 1e-6) / 1e12, all[0].n);
  printf("  \"us_after_first_block_start\": {");
  for (int p = 0; p < 5; ++p) printf("%s\"%s\": {\"first\": %.2f, \"mean\": %.2f, \"last\": %.2f}", p ? ", " : "", names[p], all[p].mn, all[p].mean(), all[p].mx);
  printf("},\n  \"gap_to_next_launch_us\": %.2f,\n", period_us - all[4].mx);
  printf("  \"k_loop_shader_clock_mhz\": {\"min\": %.0f, \"mean\": %.0f, \"max\": %.0f},\n", clk.mn, clk.mean(), clk.mx);
  if (level >= 2) printf("  \"barrier_wait_pct_of_k_loop_cycles\": {\"min\": %.2f, \"mean\": %.2f, \"max\": %.2f},\n", barrier.mn, barrier.mean(), barrier.mx);
  printf("  \"by_xcd\": [");
  for (int x = 0; x < 8; ++x)
    printf("%s{\"xcd\": %d, \"waves\": %ld, \"k_loop_us_mean\": %.2f, \"k_loop_us_max\": %.2f, \"k_loop_end_to_store_ack_us_mean\": %.2f, \"last_ack_us\": %.2f}",
           x ? ",\n             " : "", x, xcd_loop[x].n, xcd_loop[x].mean(), xcd_loop[x].mx, xcd_tail[x].mean(), xcd_end[x].mx);
  printf("]}}\n");
  return 0;
}

// minimal reader for the flat {"KEY": int, ...} objects of the tuning files
static bool read_config(const std::string& path, int index, kcg_matmul_cfg* cfg) {
  std::ifstream f(path);
  if (!f) return false;
  std::stringstream ss;
  ss << f.rdbuf();
  std::string text = ss.str();
  size_t start = 0;
  size_t arr = text.find("\"cfgs\"");
  if (arr != std::string::npos) {
    start = text.find('[', arr);
    for (int i = 0; i <= index; ++i) {
      start = text.find('{', start + (i ? 1 : 0));
      if (start == std::string::npos) return false;
      if (i < index) start = text.find('}', start);
    }
  }
  size_t end = text.find('}', start);
  std::string obj = text.substr(start, end - start);
  for (int i = 0; i < KCG_CFG_LEN; ++i) {
    std::string key = std::string("\"") + kcg_cfg_keyword(i) + "\"";
    size_t p = obj.find(key);
    if (p == std::string::npos) {
      fprintf(stderr, "config is missing %s\n", key.c_str());
      return false;
    }
    p = obj.find(':', p);
    cfg->v[i] = (int32_t)strtol(obj.c_str() + p + 1, nullptr, 10);
  }
  return true;
}

int main(int argc, char** argv) {
  kcg_matmul_cfg cfg;
  memset(&cfg, 0, sizeof(cfg));
  kcg_kernel_info info;
  memset(&info, 0, sizeof(info));
  int iters = 20, kind = KCG_KIND_AUTO, index = 0, compile_only = 0, timeline = 0;
  bool normal_dist = false;
  const char* dump_c = nullptr;
  const char* diag = nullptr;
  float tol = 0.01f;   // the reference runner's tolerance (runkernel.cpp:34)
  int M = 0, N = 0, K = 0, dt = KCG_DT_FLOAT32, dtc = KCG_DT_FLOAT32, atrans = 1;

  if (argc >= 2 && !strcmp(argv[1], "--mfma-peak")) {
    return kcg_probe_mfma_peak(argc >= 3 ? argv[2] : "f16");
  }
  if (argc >= 2 && !strcmp(argv[1], "--launch-cost")) return kcg_probe_launch_cost();
  if (argc >= 3 && !strcmp(argv[1], "--config")) {
    std::string path = argv[2];
    for (int i = 3; i + 1 < argc; i += 2) {
      if (!strcmp(argv[i], "--index")) index = atoi(argv[i + 1]);
      else if (!strcmp(argv[i], "--iters")) iters = atoi(argv[i + 1]);
      else if (!strcmp(argv[i], "--tol")) tol = (float)atof(argv[i + 1]);
      else if (!strcmp(argv[i], "--compile-only")) compile_only = atoi(argv[i + 1]);
      else if (!strcmp(argv[i], "--timeline")) timeline = atoi(argv[i + 1]);
      else if (!strcmp(argv[i], "--dist")) normal_dist = !strcmp(argv[i + 1], "normal");
      else if (!strcmp(argv[i], "--dump-c")) dump_c = argv[i + 1];
      else if (!strcmp(argv[i], "--diag")) diag = argv[i + 1];
      else if (!strcmp(argv[i], "--kind"))
        kind = !strcmp(argv[i + 1], "simt") ? KCG_KIND_SIMT : !strcmp(argv[i + 1], "mfma") ? KCG_KIND_MFMA : KCG_KIND_AUTO;
    }
    if (!read_config(path, index, &cfg)) {
      fprintf(stderr, "cannot read config %d of %s\n", index, path.c_str());
      return 2;
    }
    if (diag) {
      const char* old = getenv("KCG_EXTRA_FLAGS");
      std::string flags = std::string(old ? old : "") + " " + diag;
      setenv("KCG_EXTRA_FLAGS", flags.c_str(), 1);
      setenv("KCG_ALLOW_DIAG", "1", 1);
    }
    if (timeline > 0) {
      const char* old = getenv("KCG_EXTRA_FLAGS");
      std::string flags = std::string(old ? old : "") + " -DKCG_TIMELINE=" + std::to_string(timeline);
      setenv("KCG_EXTRA_FLAGS", flags.c_str(), 1);
    }
    if (kcg_compile_matmul(&cfg, "gfx950", kind, &info) != KCG_OK) {
      fprintf(stderr, "compile failed: %s\n", kcg_last_error());
      return 2;
    }
    M = cfg.v[KCG_M]; N = cfg.v[KCG_N]; K = cfg.v[KCG_K];
    dt = cfg.v[KCG_DTYPE_A]; dtc = cfg.v[KCG_DTYPE_C]; atrans = cfg.v[KCG_IS_ATRANS];
    printf("compiled %s (%s kernel, cache %s%s%s%s)\n", info.kernel_name, info.kind == KCG_KIND_MFMA ? "matrix-core" : "SIMT",
           info.cache_hit ? "hit" : "miss", (info.build_flags & KCG_BUILD_LOW_OPT) ? ", -O1 rebuild" : "",
           (info.build_flags & KCG_BUILD_DIRECT_DECLINED) ? ", register staging instead of direct staging" : "",
           (info.build_flags & KCG_BUILD_DIAGNOSTIC) ? ", DIAGNOSTIC BUILD: result wrong on purpose" : "");
    {
      char id[1024];
      if (kcg_compiler_identity(id, sizeof(id)) > 0) printf("compiler %s\n", id);
    }
    if (compile_only) return 0;
  } else if (argc >= 8) {
    M = atoi(argv[1]); N = atoi(argv[2]); K = atoi(argv[3]);
    info.grid[0] = atoi(argv[4]); info.grid[1] = info.grid[2] = 1;
    info.block[0] = atoi(argv[5]); info.block[1] = info.block[2] = 1;
    snprintf(info.code_path, sizeof(info.code_path), "%s", argv[6]);
    snprintf(info.kernel_name, sizeof(info.kernel_name), "%s", argv[7]);
    info.lds_bytes = argc > 8 ? atoi(argv[8]) : 2048;   // runkernel.cpp launched with 2048 B of dynamic LDS
    if (argc > 9) dt = atoi(argv[9]);
    dtc = (dt == KCG_DT_FLOAT64) ? dt : KCG_DT_FLOAT32;
    if (argc > 10) atrans = atoi(argv[10]);
    iters = 7;                                           // runkernel.cpp:104-108
  } else {
    fprintf(stderr, "usage: %s --mfma-peak [f16|bf16]\n       %s --config file.json [--index i] [--kind auto|simt|mfma] [--iters n] [--tol t] [--compile-only 1]\n"
                    "       %s M N K gridX blockX code-object kernel-name [ldsBytes] [dtypeCode] [isATrans]\n", argv[0], argv[0], argv[0]);
    return 2;
  }
  if (dt == KCG_DT_FLOAT64 || (dtc != KCG_DT_FLOAT32)) {
    fprintf(stderr, "runner verifies float32-output kernels with float32/float16/bfloat16 inputs\n");
    return 2;
  }

  // inputs: logical A[M,K], laid out as the kernel expects
  uint64_t seed = 0x4B4347;
  std::vector<float> a((size_t)M * K), b((size_t)K * N), abuf((size_t)M * K);
  for (auto& x : a) x = normal_dist ? lcg_normal(seed, 0.5f) : lcg_uniform(seed);
  for (auto& x : b) x = normal_dist ? lcg_normal(seed, 0.5f) : lcg_uniform(seed);
  if (atrans) {
    for (int i = 0; i < M; ++i)
      for (int k = 0; k < K; ++k) abuf[(size_t)k * M + i] = a[(size_t)i * K + k];
  } else {
    abuf = a;
  }
  void *dA, *dB;
  float *dC, *dD;
  if (dt == KCG_DT_FLOAT32) { dA = upload<float>(abuf); dB = upload<float>(b); }
  else if (dt == KCG_DT_FLOAT16) { dA = upload<_Float16>(abuf); dB = upload<_Float16>(b); }
  else { dA = upload<__bf16>(abuf); dB = upload<__bf16>(b); }
  HIP_OK(hipMalloc(&dC, (size_t)M * N * sizeof(float)));
  HIP_OK(hipMalloc(&dD, (size_t)M * N * sizeof(float)));
  HIP_OK(hipMemset(dC, 0xFF, (size_t)M * N * sizeof(float)));   // NaN pattern: unwritten elements fail the check

  uint64_t module = 0, function = 0;
  int32_t regs = 0, spills = 0;
  if (kcg_load(info.code_path, info.kernel_name, info.lds_bytes, 0, &module, &function, &regs, &spills) != KCG_OK) {
    fprintf(stderr, "load failed: %s\n", kcg_last_error());
    return 3;
  }
  printf("M=%d N=%d K=%d grid=%d block=%d lds=%d B regs=%d scratch=%d dwords\n", M, N, K, info.grid[0], info.block[0],
         info.lds_bytes, regs, spills);

  if (kcg_launch(function, info.grid, info.block, info.lds_bytes, 0, (uint64_t)dA, (uint64_t)dB, (uint64_t)dC) != KCG_OK) {
    fprintf(stderr, "launch failed: %s\n", kcg_last_error());
    return 3;
  }
  dim3 nb(16, 16), ng((N + 15) / 16, (M + 15) / 16);
  if (dt == KCG_DT_FLOAT32) hipLaunchKernelGGL(gemm_naive<float>, ng, nb, 0, 0, (const float*)dA, (const float*)dB, dD, M, N, K, atrans);
  else if (dt == KCG_DT_FLOAT16) hipLaunchKernelGGL(gemm_naive<_Float16>, ng, nb, 0, 0, (const _Float16*)dA, (const _Float16*)dB, dD, M, N, K, atrans);
  else hipLaunchKernelGGL(gemm_naive<__bf16>, ng, nb, 0, 0, (const __bf16*)dA, (const __bf16*)dB, dD, M, N, K, atrans);
  unsigned long long *dBad, *dFirst;
  unsigned int* dMax;
  HIP_OK(hipMalloc(&dBad, 8)); HIP_OK(hipMalloc(&dFirst, 8)); HIP_OK(hipMalloc(&dMax, 4));
  HIP_OK(hipMemset(dBad, 0, 8)); HIP_OK(hipMemset(dFirst, 0xFF, 8)); HIP_OK(hipMemset(dMax, 0, 4));
  const size_t n = (size_t)M * N;
  hipLaunchKernelGGL(verify<float>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, 0, dC, dD, n, tol, dBad, dMax, dFirst);
  HIP_OK(hipDeviceSynchronize());
  unsigned long long bad = 0, first = 0;
  unsigned int maxbits = 0;
  HIP_OK(hipMemcpy(&bad, dBad, 8, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(&first, dFirst, 8, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(&maxbits, dMax, 4, hipMemcpyDeviceToHost));
  float maxerr;
  memcpy(&maxerr, &maxbits, 4);
  if (bad) printf("have %llu error! first at (y=%llu, x=%llu), max |err| %.3e (tol %.3g)\n", bad, first / N, first % N, maxerr, tol);
  else printf("no error! max |err| %.3e (tol %.3g)\n", maxerr, tol);

  if (dump_c) {   // the kernel's result as raw fp32, row-major [M, N]: lets a caller check it against its own reference
    std::vector<float> hc((size_t)M * N);
    HIP_OK(hipMemcpy(hc.data(), dC, hc.size() * sizeof(float), hipMemcpyDeviceToHost));
    FILE* f = fopen(dump_c, "wb");
    if (!f || fwrite(hc.data(), sizeof(float), hc.size(), f) != hc.size()) {
      fprintf(stderr, "cannot write %s\n", dump_c);
      return 3;
    }
    fclose(f);
  }

  float med = 0.f, mn = 0.f;
  if (kcg_benchmark(function, info.grid, info.block, info.lds_bytes, 0, (uint64_t)dA, (uint64_t)dB, (uint64_t)dC, 20, iters, 0,
                    &med, &mn) != KCG_OK) {
    fprintf(stderr, "benchmark failed: %s\n", kcg_last_error());
    return 3;
  }
  printf("time cost: %.4f ms (median of %d), min %.4f ms;  tflops = %.2f\n", med, iters, mn,
         2.0 * M * N * K / (med * 1e-3) / 1e12);
  if (timeline > 0) {
    const int rc = timeline_report(module, function, info, info.block[0] / 64, (uint64_t)dA, (uint64_t)dB, (uint64_t)dC,
                                   2.0 * M * N * K, timeline);
    if (rc) return rc;
  }
  kcg_unload(module);
  return (bad && !(info.build_flags & KCG_BUILD_DIAGNOSTIC)) ? 1 : 0;
}
