// kcg_runner — stand-alone (no Python) runner for the engine's GEMM kernels on one GPU.
//
// It plays the role of the reference's C++ check programs: runkernel.cpp (load a code object given on
// the command line, launch it several times, compare against a naive GPU kernel with an absolute
// tolerance of 0.01, runkernel.cpp:49-112) and the main() of matmul.cpp (HIP-event timing, TFLOPS
// print, naive `gemm_kernel` + `verify_kernel`, matmul.cpp:2327-2348,2386-2553).
//
//   kcg_runner --config <file.json> [--index i] [--kind auto|simt|mfma] [--iters n] [--tol t]
//              [--dist uniform|normal] [--timeline 1|2] [--dump-c file]
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
//   kcg_runner M N K gridX blockX <code-object> <kernel-name> [ldsBytes] [dtypeCode] [isATrans]
//       the reference runner's argument list (runkernel.cpp:63-66): launches an existing code object
//
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

// ---- sustained matrix-core rate: 64 independent accumulator tiles worth of work per iteration ----------
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef __bf16 b8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));
template <class V> struct PeakOp;
template <> struct PeakOp<h8_t> {
  __device__ static f4_t small(h8_t a, h8_t b, f4_t c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
  __device__ static f16_t big(h8_t a, h8_t b, f16_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct PeakOp<b8_t> {
  __device__ static f4_t small(b8_t a, b8_t b, f4_t c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
  __device__ static f16_t big(b8_t a, b8_t b, f16_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
// opnd: 32 fragments of 8 values per lane (65536 lanes).  SMALL: 8x8 tiles of 16x16x32 over two k-steps;
// otherwise 4x4 tiles of 32x32x16 over four k-steps: 2^22 flop per lane-iteration either way.
template <class V, bool SMALL>
__global__ __launch_bounds__(256) void mfma_peak(const V* __restrict__ opnd, float* sink, int iters, long long* ticks) {
  const long long t_begin = __builtin_amdgcn_s_memrealtime();   // 100 MHz
  const int tid = blockIdx.x * 256 + threadIdx.x;
  V frag[32];
#pragma unroll
  for (int f = 0; f < 32; ++f) frag[f] = opnd[(size_t)f * 65536 + tid];
  float s = 0.f;
  if constexpr (SMALL) {
    f4_t acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = f4_t{0, 0, 0, 0};
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int k = 0; k < 2; ++k)
#pragma unroll
        for (int q = 0; q < 64; ++q) {
          acc[q / 8][q % 8] = PeakOp<V>::small(frag[k * 16 + 8 + q % 8], frag[k * 16 + q / 8], acc[q / 8][q % 8]);
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) s += acc[i][j][0] + acc[i][j][3];
  } else {
    f16_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int q = 0; q < 16; ++q) {
          acc[q / 4][q % 4] = PeakOp<V>::big(frag[k * 8 + 4 + q % 4], frag[k * 8 + q / 4], acc[q / 4][q % 4]);
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) s += acc[i][j][0] + acc[i][j][15];
  }
  if (s == 1234.5f) sink[tid] = s;   // keeps the loop alive; practically never true
  if (ticks && threadIdx.x == 0) ticks[blockIdx.x] = __builtin_amdgcn_s_memrealtime() - t_begin;
}

// xcd_ns (optional, 8 values): mean block duration of the last launch per XCD (blocks are dealt to the
// eight XCDs round-robin), in nanoseconds
template <class V, bool SMALL>
static double run_mfma_peak(const V* d_opnd, float* d_sink, double* xcd_ns = nullptr) {
  const int iters = 3000, launches = 50;           // 64 (or 4x16) instructions of 2^22/64 flop per lane-iteration
  long long* d_ticks;
  HIP_OK(hipMalloc(&d_ticks, 256 * sizeof(long long)));
  for (int i = 0; i < launches; ++i) hipLaunchKernelGGL((mfma_peak<V, SMALL>), dim3(256), dim3(256), 0, 0, d_opnd, d_sink, iters, d_ticks);
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0)); HIP_OK(hipEventCreate(&e1));
  HIP_OK(hipEventRecord(e0, 0));
  for (int i = 0; i < launches; ++i) hipLaunchKernelGGL((mfma_peak<V, SMALL>), dim3(256), dim3(256), 0, 0, d_opnd, d_sink, iters, d_ticks);
  HIP_OK(hipEventRecord(e1, 0));
  HIP_OK(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  if (xcd_ns) {
    long long h[256];
    HIP_OK(hipMemcpy(h, d_ticks, sizeof(h), hipMemcpyDeviceToHost));
    for (int x = 0; x < 8; ++x) {
      double sum = 0;
      for (int b = x; b < 256; b += 8) sum += (double)h[b] * 10.0;
      xcd_ns[x] = sum / 32;
    }
  }
  HIP_OK(hipFree(d_ticks));
  const double flops = (double)launches * iters * 128.0 * 16 * 16 * 32 * 2 * 4 * 256;   // per block: 4 waves
  return flops / (ms * 1e-3) / 1e12;
}

template <class V, class E>
static int mfma_peak_main(const char* tname) {
  const size_t n = (size_t)32 * 65536;
  std::vector<V> h(n);
  V* d;
  float* sink;
  HIP_OK(hipMalloc(&d, n * sizeof(V)));
  HIP_OK(hipMalloc(&sink, 65536 * sizeof(float)));
  uint64_t st = 0x4B4347;
  printf("{\"mfma_peak\": {\"dtype\": \"%s\"", tname);
  for (int pass = 0; pass < 2; ++pass) {
    for (size_t i = 0; i < n; ++i)
      for (int e = 0; e < 8; ++e) {
        float g = 0.f;
        if (pass == 1) {   // normal(0, 0.5): Box-Muller on two uniforms
          st = st * 6364136223846793005ull + 1442695040888963407ull;
          const float u1 = ((float)(st >> 40) + 1.0f) / 16777217.0f;
          st = st * 6364136223846793005ull + 1442695040888963407ull;
          const float u2 = (float)(st >> 40) / 16777216.0f;
          g = sqrtf(-2.0f * logf(u1)) * cosf(6.2831853f * u2) * 0.5f;
        }
        h[i][e] = (E)g;
      }
    HIP_OK(hipMemcpy(d, h.data(), n * sizeof(V), hipMemcpyHostToDevice));
    double xcd[8];
    const double small = run_mfma_peak<V, true>(d, sink, xcd), big = run_mfma_peak<V, false>(d, sink);
    printf(", \"%s\": {\"16x16x32\": %.1f, \"32x32x16\": %.1f, \"16x16x32_block_us_by_xcd\": [", pass == 0 ? "zeros" : "normal(0,0.5)", small, big);
    for (int x = 0; x < 8; ++x) printf("%s%.1f", x ? ", " : "", xcd[x] * 1e-3);
    printf("]}");
  }
  printf(", \"unit\": \"TFLOP/s\"}}\n");
  HIP_OK(hipFree(d));
  HIP_OK(hipFree(sink));
  return 0;
}

// ---- fixed costs of a launch: what a GEMM of a few hundred microseconds pays besides its K loop ------
__global__ void empty_kernel(float* sink) {
  if (sink == nullptr && threadIdx.x == 12345) *sink = 0.f;   // never true
}
template <int LDS_BYTES>
__global__ __launch_bounds__(256) void empty_kernel_lds(float* sink) {
  __shared__ char big[LDS_BYTES];
  if (sink == nullptr) { big[threadIdx.x] = 1; *sink = big[255 - threadIdx.x]; }   // never true; keeps the array
}
// every block writes its own contiguous piece of `out` with 16-byte stores, nothing else
__global__ __launch_bounds__(256) void write_only(float4* __restrict__ out, size_t per_block) {
  float4* p = out + (size_t)blockIdx.x * per_block;
  const float4 v = {1.f, 2.f, 3.f, 4.f};
  for (size_t i = threadIdx.x; i < per_block; i += 256) p[i] = v;
}

// the C stores of a 256 x 256 x (4 waves of 128 x 128) GEMM epilogue and nothing else: block b owns tile
// (b / 16, b % 16) of a 4096 x 4096 fp32 matrix.  LINE = 64: every store instruction of a wave writes 16 rows x
// 64 contiguous bytes (what 16x16 accumulator tiles give); LINE = 128: 8 rows x 128 bytes (whole cache
// lines per row).  NT: non-temporal stores.
template <int LINE, bool NT>
__global__ __launch_bounds__(256) void write_tiles(float* __restrict__ out) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int row0 = (blockIdx.x / 16) * 256 + (wave / 2) * 128, col0 = (blockIdx.x % 16) * 256 + (wave % 2) * 128;
  constexpr int LPR = LINE / 16, RPI = 64 / LPR;       // lanes per row, rows per instruction
  typedef float v4 __attribute__((ext_vector_type(4)));
  const v4 v = {1.f, 2.f, 3.f, 4.f};
  for (int r = 0; r < 128; r += RPI)
    for (int c = 0; c < 128; c += LINE / 4) {
      v4* p = (v4*)(out + (size_t)(row0 + r + lane / LPR) * 4096 + col0 + c + (lane % LPR) * 4);
      if constexpr (NT) __builtin_nontemporal_store(v, p);
      else *p = v;
    }
}

// What a wave can know about a global->LDS fetch it issued behind its own stores.  Every wave (one per block, one
// block per compute unit) optionally issues NSTORES 16-byte-per-lane stores to cold lines, then one 16-byte-per-lane
// fetch of cache-resident data into LDS that it had filled with a marker, and measures (shader-clock cycles)
//   [0] until the fetched data is visible in LDS (polling the last lane's slot),
//   [1] until s_waitcnt vmcnt(0) returns (the wave's only counter for fetches and stores alike).
template <int NSTORES>
__global__ __launch_bounds__(64) void fetch_behind_stores(const float4* __restrict__ src, float4* __restrict__ sink,
                                                            unsigned long long* __restrict__ out) {
  __shared__ __attribute__((aligned(1024))) float4 lds[64];
  const int lane = threadIdx.x;
  lds[lane] = float4{-1.f, -1.f, -1.f, -1.f};
  __syncthreads();
  // every store instruction writes 16 rows x 64 bytes, rows 1 KiB apart (the shape of the GEMM epilogue's stores)
  float4* mine = sink + ((size_t)blockIdx.x * 512 + lane % 16) * 64 + lane / 16;
  const float4 v = {1.f, 2.f, 3.f, 4.f};
  const unsigned lds_probe = (unsigned)(unsigned long)lds + 63 * 16;
  const unsigned long long t0 = __builtin_amdgcn_s_memtime();
#pragma unroll
  for (int i = 0; i < NSTORES; ++i) mine[(size_t)i * 16 * 64] = v;
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + lane),
                                   (__attribute__((address_space(3))) void*)lds, 16, 0, 0);
  unsigned long long t_seen = 0;
  for (int spin = 0; spin < 200000; ++spin) {                        // bounded: every wave leaves the loop
    // (read with an instruction the compiler does not connect with the fetch: it would wait for vmcnt(0) first)
    unsigned probe;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(probe) : "v"(lds_probe) : "memory");
    if (__builtin_amdgcn_readfirstlane((int)probe) != __float_as_int(-1.f)) {
      t_seen = __builtin_amdgcn_s_memtime();
      break;
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);                                // vmcnt(0), nothing else
  const unsigned long long t_cnt = __builtin_amdgcn_s_memtime();
  if (lane == 0) {
    out[blockIdx.x * 2] = t_seen ? t_seen - t0 : 0;
    out[blockIdx.x * 2 + 1] = t_cnt - t0;
  }
}

template <int NSTORES>
static void run_fetch_behind_stores(double* seen_cycles, double* counted_cycles) {
  float4 *src, *sink;
  unsigned long long* out;
  HIP_OK(hipMalloc(&src, 64 * sizeof(float4)));
  HIP_OK(hipMalloc(&sink, (size_t)256 * 512 * 64 * sizeof(float4)));   // 128 MiB
  HIP_OK(hipMalloc(&out, 512 * sizeof(unsigned long long)));
  HIP_OK(hipMemset(src, 0, 64 * sizeof(float4)));                    // zeros differ from the marker
  for (int i = 0; i < 20; ++i) hipLaunchKernelGGL((fetch_behind_stores<NSTORES>), dim3(256), dim3(64), 0, 0, src, sink, out);
  HIP_OK(hipDeviceSynchronize());
  unsigned long long h[512];
  HIP_OK(hipMemcpy(h, out, sizeof(h), hipMemcpyDeviceToHost));
  double a = 0, b = 0;
  for (int i = 0; i < 256; ++i) { a += (double)h[2 * i]; b += (double)h[2 * i + 1]; }
  *seen_cycles = a / 256;
  *counted_cycles = b / 256;
  HIP_OK(hipFree(src)); HIP_OK(hipFree(sink)); HIP_OK(hipFree(out));
}

template <class F>
static double launch_period_us(F launch, int n) {
  for (int i = 0; i < 200; ++i) launch();
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0)); HIP_OK(hipEventCreate(&e1));
  HIP_OK(hipEventRecord(e0, 0));
  for (int i = 0; i < n; ++i) launch();
  HIP_OK(hipEventRecord(e1, 0));
  HIP_OK(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  HIP_OK(hipEventDestroy(e0)); HIP_OK(hipEventDestroy(e1));
  return ms * 1e3 / n;
}

static int launch_cost_main() {
  float* sink;
  const size_t bytes = (size_t)64 << 20;   // the C matrix of a 4096 x 4096 fp32 result
  HIP_OK(hipMalloc(&sink, bytes));
  const int n = 2000;
  const double e1 = launch_period_us([&] { hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, 0, sink); }, n);
  const double e256 = launch_period_us([&] { hipLaunchKernelGGL(empty_kernel, dim3(256), dim3(256), 0, 0, sink); }, n);
  const double elds = launch_period_us([&] { hipLaunchKernelGGL((empty_kernel_lds<65536>), dim3(256), dim3(256), 0, 0, sink); }, n);
  const double w = launch_period_us([&] { hipLaunchKernelGGL(write_only, dim3(256), dim3(256), 0, 0, (float4*)sink, bytes / 16 / 256); }, 500);
  const double t64 = launch_period_us([&] { hipLaunchKernelGGL((write_tiles<64, false>), dim3(256), dim3(256), 0, 0, sink); }, 500);
  const double t128 = launch_period_us([&] { hipLaunchKernelGGL((write_tiles<128, false>), dim3(256), dim3(256), 0, 0, sink); }, 500);
  const double t64nt = launch_period_us([&] { hipLaunchKernelGGL((write_tiles<64, true>), dim3(256), dim3(256), 0, 0, sink); }, 500);
  const double t128nt = launch_period_us([&] { hipLaunchKernelGGL((write_tiles<128, true>), dim3(256), dim3(256), 0, 0, sink); }, 500);
  double seen0, cnt0, seen32, cnt32;
  run_fetch_behind_stores<0>(&seen0, &cnt0);
  run_fetch_behind_stores<32>(&seen32, &cnt32);
  printf("{\"fetch_behind_stores\": {\"unit\": \"shader-clock cycles, mean over 256 waves\", "
         "\"alone\": {\"data_visible_in_lds\": %.0f, \"vmcnt_0\": %.0f}, "
         "\"behind_32_stores\": {\"data_visible_in_lds\": %.0f, \"vmcnt_0\": %.0f}}}\n", seen0, cnt0, seen32, cnt32);
  printf("{\"launch_cost\": {\"period_us\": {\"empty_1_block\": %.2f, \"empty_256_blocks\": %.2f, \"empty_256_blocks_64KiB_lds\": %.2f, "
         "\"write_64MiB\": %.2f, \"write_64MiB_as_gemm_tiles_64B_per_row\": %.2f, \"write_64MiB_as_gemm_tiles_128B_per_row\": %.2f, "
         "\"same_64B_nontemporal\": %.2f, \"same_128B_nontemporal\": %.2f}, \"write_GBps\": %.0f, "
         "\"note\": \"back-to-back launches on one stream, HIP events around the whole run\"}}\n",
         e1, e256, elds, w, t64, t128, t64nt, t128nt, bytes / (w - e256) * 1e-3);
  HIP_OK(hipFree(sink));
  return 0;
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
  float tol = 0.01f;   // the reference runner's tolerance (runkernel.cpp:34)
  int M = 0, N = 0, K = 0, dt = KCG_DT_FLOAT32, dtc = KCG_DT_FLOAT32, atrans = 1;

  if (argc >= 2 && !strcmp(argv[1], "--mfma-peak")) {
    if (argc >= 3 && !strcmp(argv[2], "bf16")) return mfma_peak_main<b8_t, __bf16>("bf16");
    return mfma_peak_main<h8_t, _Float16>("f16");
  }
  if (argc >= 2 && !strcmp(argv[1], "--launch-cost")) return launch_cost_main();
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
      else if (!strcmp(argv[i], "--kind"))
        kind = !strcmp(argv[i + 1], "simt") ? KCG_KIND_SIMT : !strcmp(argv[i + 1], "mfma") ? KCG_KIND_MFMA : KCG_KIND_AUTO;
    }
    if (!read_config(path, index, &cfg)) {
      fprintf(stderr, "cannot read config %d of %s\n", index, path.c_str());
      return 2;
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
    printf("compiled %s (%s kernel, cache %s)\n", info.kernel_name, info.kind == KCG_KIND_MFMA ? "matrix-core" : "SIMT",
           info.cache_hit ? "hit" : "miss");
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
  return bad ? 1 : 0;
}
