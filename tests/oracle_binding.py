"""ctypes binding of oracle/liboracle.so for the tests (the oracle is test infrastructure)."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB = os.path.join(ORACLE_DIR, "liboracle.so")


class Oracle:
    def __init__(self, lib):
        self.lib = lib
        fp = ctypes.POINTER(ctypes.c_float)
        dp = ctypes.POINTER(ctypes.c_double)
        i = ctypes.c_int
        lib.oracle_host_matmul_f32_ijk.argtypes = [fp, fp, fp, i, i, i, i, i, i]
        lib.oracle_matmul_f32.argtypes = [fp, fp, fp, i, i, i, i, i, i, i]
        lib.oracle_matmul_f32_f64acc.argtypes = [fp, fp, dp, i, i, i, i, i, i, i]
        lib.oracle_matmul_f64.argtypes = [dp, dp, dp, i, i, i, i, i, i, i]
        lib.oracle_max_threads.restype = i
        lg, f = ctypes.c_long, ctypes.c_float
        lib.oracle_matmul_f32_batched_ab.argtypes = [fp, fp, fp, i, i, i, i, i, lg, lg, lg, f, f, i]

    @staticmethod
    def _f(x):
        return x.ctypes.data_as(ctypes.POINTER(ctypes.c_float))

    @staticmethod
    def _d(x):
        return x.ctypes.data_as(ctypes.POINTER(ctypes.c_double))

    @staticmethod
    def _shape(a, b, a_trans):
        K, N = b.shape
        M = a.shape[1] if a_trans else a.shape[0]
        assert (a.shape[0] if a_trans else a.shape[1]) == K
        return M, N, K

    def ijk(self, a, b, a_trans, rows=None):
        """The reference loop (i-j-k, single thread).  a: [K,M] if a_trans else [M,K]."""
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32)
        M, N, K = self._shape(a, b, a_trans)
        r0, r1 = rows or (0, M)
        c = np.zeros((M, N), np.float32)
        self.lib.oracle_host_matmul_f32_ijk(self._f(a), self._f(b), self._f(c), M, N, K, int(a_trans), r0, r1)
        return c[r0:r1]

    def matmul(self, a, b, a_trans, rows=None, nthreads=0):
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32)
        M, N, K = self._shape(a, b, a_trans)
        r0, r1 = rows or (0, M)
        c = np.zeros((M, N), np.float32) if rows is None else np.zeros((M, N), np.float32)
        self.lib.oracle_matmul_f32(self._f(a), self._f(b), self._f(c), M, N, K, int(a_trans), nthreads, r0, r1)
        return c[r0:r1]

    def matmul_f64acc(self, a, b, a_trans, rows=None, nthreads=0):
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32)
        M, N, K = self._shape(a, b, a_trans)
        r0, r1 = rows or (0, M)
        c = np.zeros((M, N), np.float64)
        self.lib.oracle_matmul_f32_f64acc(self._f(a), self._f(b), self._d(c), M, N, K, int(a_trans), nthreads, r0, r1)
        return c[r0:r1]

    def matmul_f64(self, a, b, a_trans, rows=None, nthreads=0):
        a = np.ascontiguousarray(a, np.float64)
        b = np.ascontiguousarray(b, np.float64)
        M, N, K = self._shape(a, b, a_trans)
        r0, r1 = rows or (0, M)
        c = np.zeros((M, N), np.float64)
        self.lib.oracle_matmul_f64(self._d(a), self._d(b), self._d(c), M, N, K, int(a_trans), nthreads, r0, r1)
        return c[r0:r1]

    def batched_ab(self, a, b, c0, M, N, K, a_trans, batch, strides, alpha, beta, nthreads=0):
        """C_z = alpha * A_z B_z + beta * C_z over flat fp32 buffers (strides in elements); returns the new c."""
        a = np.ascontiguousarray(a, np.float32).ravel()
        b = np.ascontiguousarray(b, np.float32).ravel()
        c = np.array(c0, np.float32).ravel().copy()
        sa, sb, sc = strides
        assert a.size >= (batch - 1) * sa + M * K and b.size >= (batch - 1) * sb + K * N and c.size >= (batch - 1) * sc + M * N
        self.lib.oracle_matmul_f32_batched_ab(self._f(a), self._f(b), self._f(c), M, N, K, int(a_trans), batch,
                                              sa, sb, sc, alpha, beta, nthreads)
        return c

    def max_threads(self):
        return self.lib.oracle_max_threads()


REF_LIB = os.path.join(ORACLE_DIR, "_ref", "libhostmatmul_ref.so")


def load_reference_build():
    """The reference's own hostMatmul (matmul.cpp:2349-2360) compiled by oracle/Makefile; None where that
    build does not exist (no reference tree at build time)."""
    if not os.path.exists(REF_LIB):
        return None
    lib = ctypes.CDLL(REF_LIB)
    fp = ctypes.POINTER(ctypes.c_float)
    lib.ref_host_matmul_f32.argtypes = [fp, fp, fp, ctypes.c_int, ctypes.c_int, ctypes.c_int]

    def host_matmul(a_km, b_kn):
        """a_km: A stored [K, M] (hostMatmul's layout); accumulates into a zeroed C (matmul.cpp:2425-2428)."""
        a_km = np.ascontiguousarray(a_km, np.float32)
        b_kn = np.ascontiguousarray(b_kn, np.float32)
        K, M = a_km.shape
        N = b_kn.shape[1]
        c = np.zeros((M, N), np.float32)
        lib.ref_host_matmul_f32(a_km.ctypes.data_as(fp), b_kn.ctypes.data_as(fp), c.ctypes.data_as(fp), M, N, K)
        return c
    return host_matmul


def build():
    out = subprocess.run(["make", "-B", "-C", ORACLE_DIR], capture_output=True, text=True)
    if out.returncode != 0:
        raise RuntimeError("building the oracle failed:\n" + out.stdout + out.stderr)


def load():
    if not os.path.exists(LIB):
        build()
    return Oracle(ctypes.CDLL(LIB))
