/*
 * host_matmul.c — CPU oracle for the KCG GEMM hot path.  TEST INFRASTRUCTURE ONLY: it is linked and
 * called by the test-suite, by the smoke check and by the benchmark's cpu_baseline leg, as the checker
 * or as the reported CPU baseline — never by the product library or the product Python package.
 *
 * What it restates (paths relative to the KCG reference tree):
 *   - hostMatmul, matmul.cpp:2350-2360: the reference's CPU matmul, a plain i-j-k triple loop that
 *     accumulates C[i*N+j] += A[k*M+i] * B[k*N+j] in fp32 with A stored [K,M]; C is zeroed by the
 *     caller first (matmul.cpp:2425-2428).
 *   - Matmul::buildNaiveExpress, src/lib/Operators/Matmul.cc:41-65: the definition the generated
 *     kernel implements: acc = 0; for k ascending: acc = acc + A(i,k)*B(k,j)   (mulf then addf).
 *
 * Pinning (see tests/test_oracle.py): every function below is checked against closed forms
 * (identity, all-ones, one-hot probes, small-integer matrices that are exact in fp32), against a
 * brute-force pure-Python triple loop on tiny shapes and against numpy float64 matmul.  The reference
 * ships no golden vectors for this path.  Where the reference tree is present, oracle/Makefile also builds
 * the reference's own hostMatmul (oracle/_ref/libhostmatmul_ref.so) and the tests require bit equality
 * with oracle_host_matmul_f32_ijk.
 *
 * Built with -ffp-contract=off so that a*b+c is never fused: each C element is the fp32 sum, in
 * ascending k, of individually rounded fp32 products, exactly what the reference loop computes when
 * it is built without contraction.
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define CLONES __attribute__((target_clones("avx2", "default")))

/* The reference loop, verbatim in structure: i-j-k order, single thread, accumulates INTO c
 * (caller zeroes c).  a_trans != 0: A is [K,M] (A(i,k) = a[k*M+i], hostMatmul's layout);
 * a_trans == 0: A is [M,K] (A(i,k) = a[i*K+k]).  Only rows [row_begin,row_end) of C are produced. */
void oracle_host_matmul_f32_ijk(const float* a, const float* b, float* c, int M, int N, int K, int a_trans,
                                int row_begin, int row_end) {
  for (int i = row_begin; i < row_end; i++) {
    for (int j = 0; j < N; j++) {
      for (int k = 0; k < K; k++) {
        float av = a_trans ? a[(size_t)k * M + i] : a[(size_t)i * K + k];
        c[(size_t)i * N + j] += av * b[(size_t)k * N + j];
      }
    }
  }
}

/* Same arithmetic, loop order i-k-j so the inner loop streams rows of B and C: every C element
 * still receives its products one at a time in ascending k, so the result is bit-identical to the
 * i-j-k loop.  Rows are spread over `nthreads` OpenMP threads (<=0: all).  Overwrites c rows. */
CLONES static void row_ikj_f32(const float* a, const float* b, float* crow, int i, int M, int N, int K, int a_trans) {
  for (int j = 0; j < N; j++) crow[j] = 0.0f;
  for (int k = 0; k < K; k++) {
    const float av = a_trans ? a[(size_t)k * M + i] : a[(size_t)i * K + k];
    const float* brow = b + (size_t)k * N;
    for (int j = 0; j < N; j++) crow[j] = crow[j] + av * brow[j];
  }
}

void oracle_matmul_f32(const float* a, const float* b, float* c, int M, int N, int K, int a_trans, int nthreads,
                       int row_begin, int row_end) {
#ifdef _OPENMP
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#pragma omp parallel for schedule(dynamic, 4) num_threads(nthreads)
#endif
  for (int i = row_begin; i < row_end; i++) row_ikj_f32(a, b, c + (size_t)i * N, i, M, N, K, a_trans);
}

/* fp32 inputs, fp64 products and accumulation, fp64 result: the "exact" value used to bound the
 * error of both the fp32 oracle and the device kernels. */
CLONES static void row_ikj_f64acc(const float* a, const float* b, double* crow, int i, int M, int N, int K, int a_trans) {
  for (int j = 0; j < N; j++) crow[j] = 0.0;
  for (int k = 0; k < K; k++) {
    const double av = a_trans ? a[(size_t)k * M + i] : a[(size_t)i * K + k];
    const float* brow = b + (size_t)k * N;
    for (int j = 0; j < N; j++) crow[j] = crow[j] + av * (double)brow[j];
  }
}

void oracle_matmul_f32_f64acc(const float* a, const float* b, double* c, int M, int N, int K, int a_trans,
                              int nthreads, int row_begin, int row_end) {
#ifdef _OPENMP
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#pragma omp parallel for schedule(dynamic, 4) num_threads(nthreads)
#endif
  for (int i = row_begin; i < row_end; i++) row_ikj_f64acc(a, b, c + (size_t)i * N, i, M, N, K, a_trans);
}

/* fp64 GEMM for DATATYPE 8 configs (Matmul.cc accepts f64): sequential-k fp64. */
void oracle_matmul_f64(const double* a, const double* b, double* c, int M, int N, int K, int a_trans, int nthreads,
                       int row_begin, int row_end) {
#ifdef _OPENMP
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#pragma omp parallel for schedule(dynamic, 4) num_threads(nthreads)
#endif
  for (int i = row_begin; i < row_end; i++) {
    double* crow = c + (size_t)i * N;
    for (int j = 0; j < N; j++) crow[j] = 0.0;
    for (int k = 0; k < K; k++) {
      const double av = a_trans ? a[(size_t)k * M + i] : a[(size_t)i * K + k];
      const double* brow = b + (size_t)k * N;
      for (int j = 0; j < N; j++) crow[j] = crow[j] + av * brow[j];
    }
  }
}

/* Batched / strided GEMM with the alpha-beta epilogue of the vendor sgemm call the reference profiles against
 * (runRoc.cpp:27-28,53-66; batched GEMM is the next item of the reference's roadmap, 结果汇总.md:21-22):
 *   for z in [0, batch):  C_z = alpha * (A_z B_z) + beta * C_z
 * with X_z = x + z * stride_x (strides in elements; stride_a / stride_b may be 0).  The product is the same
 * sequential-k fp32 sum as above; then one multiplication by alpha, one by beta and one addition, each rounded
 * to fp32.  beta == 0: C is not read (BLAS rule), the result is alpha * (A B).  c is read and overwritten. */
void oracle_matmul_f32_batched_ab(const float* a, const float* b, float* c, int M, int N, int K, int a_trans, int batch,
                                  long stride_a, long stride_b, long stride_c, float alpha, float beta, int nthreads) {
#ifdef _OPENMP
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#endif
  for (int z = 0; z < batch; z++) {
    const float* az = a + (size_t)z * stride_a;
    const float* bz = b + (size_t)z * stride_b;
    float* cz = c + (size_t)z * stride_c;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 4) num_threads(nthreads)
#endif
    for (int i = 0; i < M; i++) {
      float* acc = (float*)malloc((size_t)N * sizeof(float));
      row_ikj_f32(az, bz, acc, i, M, N, K, a_trans);
      float* crow = cz + (size_t)i * N;
      for (int j = 0; j < N; j++) {
        const float scaled = alpha * acc[j];
        if (beta == 0.0f) {
          crow[j] = scaled;
        } else {
          const float old = beta * crow[j];
          crow[j] = scaled + old;
        }
      }
      free(acc);
    }
  }
}

int oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
