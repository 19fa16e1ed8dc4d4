// kcg_probes.hip — micro-benchmarks of the GPU itself, linked into kcg_runner (second translation unit):
//   kcg_probe_mfma_peak   : what the matrix pipeline sustains with nothing else going on
//   kcg_probe_launch_cost : the fixed costs a short GEMM pays per launch
// They launch no kernel of the engine; kcg_runner.hip (the twin of the reference's runkernel.cpp) only
// dispatches "--mfma-peak" / "--launch-cost" to them.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "kcg_probes.h"

#define HIP_OK(x)                                                                      \
  do {                                                                                 \
    hipError_t e_ = (x);                                                               \
    if (e_ != hipSuccess) {                                                            \
      fprintf(stderr, "HIP error %d (%s) at %s:%d\n", (int)e_, hipGetErrorString(e_), __FILE__, __LINE__); \
      exit(3);                                                                         \
    }                                                                                  \
  } while (0)

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

int kcg_probe_mfma_peak(const char* dtype) {
  if (dtype && !strcmp(dtype, "bf16")) return mfma_peak_main<b8_t, __bf16>("bf16");
  return mfma_peak_main<h8_t, _Float16>("f16");
}

int kcg_probe_launch_cost() { return launch_cost_main(); }
