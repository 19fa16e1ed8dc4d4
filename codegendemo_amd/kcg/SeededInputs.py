"""Deterministic synthetic GEMM inputs.

The reference's harness draws unseeded torch.randn matrices (KCGTask.py:85-87); benchmarks and parity
tests of this engine need the same matrices in every process and on every machine, so inputs come from
a counter-based generator: element i of stream s is a pure function of (seed, s, i).

  uniform(shape, stream)      i.i.d. uniform on [-1, 1), exact in fp32 (24-bit integers / 2^23 - 1)
  normal(shape, stream, std)  i.i.d. N(0, std^2) by Box-Muller on two 24-bit uniforms, fp64 -> fp32
  small_ints(shape, stream)   integers in [-lim, lim]: products and sums stay exact in fp32 and in
                              fp16-input/fp32-accumulate arithmetic, so any correct GEMM must match
                              bit for bit whatever its summation order

A is always generated logically as [M, K]; `a_operand` lays it out the way a config's IS_ATRANS asks
(the reference harness does `a.T.contiguous()`, KCGTask.py:139,156-158).
"""
import numpy as np

SEED = 0x4B4347          # "KCG"
STREAM_A, STREAM_B = 1, 2

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def _mix64(x):
    """splitmix64 finalizer, vectorised over uint64 arrays (wraps modulo 2^64)."""
    x = x.copy()
    with np.errstate(over="ignore"):
        x ^= x >> np.uint64(30)
        x *= np.uint64(0xBF58476D1CE4E5B9)
        x ^= x >> np.uint64(27)
        x *= np.uint64(0x94D049BB133111EB)
        x ^= x >> np.uint64(31)
    return x


def raw_bits(n, stream, seed=SEED):
    """n 64-bit words of stream `stream`."""
    with np.errstate(over="ignore"):
        base = _mix64(np.array([np.uint64(seed) + np.uint64(stream) * _GOLDEN], dtype=np.uint64))[0]
        idx = np.arange(n, dtype=np.uint64)
        return _mix64(base + (idx + np.uint64(1)) * _GOLDEN)


def uniform(shape, stream, seed=SEED):
    n = int(np.prod(shape))
    bits = raw_bits(n, stream, seed)
    u24 = (bits >> np.uint64(40)).astype(np.int64)                  # 24 bits
    return ((u24 - (1 << 23)).astype(np.float32) / np.float32(1 << 23)).reshape(shape)


def normal(shape, stream, std=1.0, seed=SEED):
    n = int(np.prod(shape))
    bits = raw_bits(n, stream, seed)
    u1 = ((bits >> np.uint64(40)).astype(np.float64) + 1.0) / float(1 << 24)          # (0, 1]
    u2 = ((bits >> np.uint64(16)) & np.uint64(0xFFFFFF)).astype(np.float64) / float(1 << 24)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (z * std).astype(np.float32).reshape(shape)


def small_ints(shape, stream, lim=4, seed=SEED):
    n = int(np.prod(shape))
    bits = raw_bits(n, stream, seed)
    v = (bits >> np.uint64(33)).astype(np.int64) % (2 * lim + 1) - lim
    return v.astype(np.float32).reshape(shape)


def a_operand(a_mk, is_a_transposed):
    """[M,K] matrix -> the buffer a kernel built with IS_ATRANS expects."""
    return np.ascontiguousarray(a_mk.T) if is_a_transposed else np.ascontiguousarray(a_mk)


def checksum(x):
    """Order-dependent 64-bit checksum of an array's bytes (for input fixtures)."""
    b = np.ascontiguousarray(x).reshape(-1).view(np.uint8)
    pad = (-b.size) % 8
    if pad:
        b = np.concatenate([b, np.zeros(pad, np.uint8)])
    w = b.view(np.uint64)
    with np.errstate(over="ignore"):
        h = _mix64(w + np.arange(1, w.size + 1, dtype=np.uint64) * _GOLDEN)
        return int(np.bitwise_xor.reduce(h)) ^ (w.size * 0x9E3779B9)
