"""Two fixed pseudo-random samples of tuning configs (both kernel families, all input types, both A
layouts, prefetch flags, split-U, odd tile/wave shapes, 1..17 K tiles; the second with edge tiles in M,
N and K), each checked bit for bit on small-integer data: the first against the CPU oracle, the second
against the exact integer product.  The samples are deterministic, so the build step can precompile them.
Every sample runs twice: built by the hiprtc the process carries and by the system's (tests.gemm_helpers.hiprtc_params)."""
import random

import numpy as np
import pytest

from codegendemo_amd import _native
from codegendemo_amd.kcg import SeededInputs as SI
from codegendemo_amd.kcg.ConfigGenerator import make_config
from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig
from tests.gemm_helpers import hiprtc_params, run_gemm

pytestmark = pytest.mark.gpu


def random_configs(n_matrix=60, n_simt=30, seed=20240607):
    """-> [(config, kind)]: valid configs only, drawn with a fixed seed (no GPU needed)."""
    rng = random.Random(seed)
    out = []
    while sum(1 for _, k in out if k == _native.KIND_MFMA) < n_matrix:
        dtype = rng.choice([2, 3, 4, 4, 2, 8])
        BK = rng.choice([8, 16, 32, 64] if dtype in (4, 8) else [16, 32, 64])
        kw = dict(BM=rng.choice([64, 128, 256]), BN=rng.choice([64, 128, 256]), BK=BK, TM=rng.choice([4, 8, 16]),
                  TN=rng.choice([2, 4, 8, 16]), warp_layout=rng.choice([(8, 8), (4, 16), (16, 4)]), dtype=dtype,
                  is_atrans=rng.choice([0, 1]), block_mapping=rng.choice([0, 2, 8]))
        kw["shared_prefetch"], kw["reg_prefetch"] = rng.choice([(1, 1), (1, 1), (1, 1), (1, 0), (0, 1), (0, 0)])
        kw.update(M=kw["BM"] * rng.choice([1, 2]), N=kw["BN"] * rng.choice([1, 2, 3]),
                  K=BK * rng.choice([1, 2, 3, 4, 5, 7, 9, 12, 17]))
        if dtype in (2, 3):
            kw["dtype_c"] = 4
        if dtype == 8:
            kw["scatter"] = 2
        try:
            cfg = make_config(**kw)
            if _native.is_valid_config(kernelArgFromConfig(cfg).values(), _native.KIND_MFMA):
                out.append((cfg, _native.KIND_MFMA))
        except (ValueError, _native.KcgError):
            continue
    while sum(1 for _, k in out if k == _native.KIND_SIMT) < n_simt:
        dtype = rng.choice([2, 3, 4, 4, 8])
        BK = rng.choice([8, 16, 32])
        kw = dict(BM=rng.choice([32, 64, 128]), BN=rng.choice([32, 64, 128]), BK=BK, TM=rng.choice([2, 4, 8]),
                  TN=rng.choice([2, 4, 8]), warp_layout=rng.choice([(8, 8), (4, 16), (16, 4)]), dtype=dtype,
                  is_atrans=rng.choice([0, 1]), block_mapping=rng.choice([0, 2, 8]), lsu=rng.choice([1, 1, 2]),
                  scatter=rng.choice([1, 2]), load_continuous=rng.choice([0, 1]), reduce_c_continuous=rng.choice([0, 1]),
                  shared_prefetch=rng.choice([0, 1]), reg_prefetch=rng.choice([0, 1]))
        kw.update(M=kw["BM"] * rng.choice([1, 2]), N=kw["BN"] * rng.choice([1, 2, 3]), K=BK * rng.choice([1, 2, 3, 5, 8]))
        if dtype in (2, 3):
            kw["dtype_c"] = 4
        try:
            cfg = make_config(**kw)
            if _native.is_valid_config(kernelArgFromConfig(cfg).values(), _native.KIND_SIMT):
                out.append((cfg, _native.KIND_SIMT))
        except (ValueError, _native.KcgError):
            continue
    return out


def random_edge_configs(n_matrix=50, n_simt=30, n_direct=25, seed=20250311):
    """-> [(config, kind)]: a second fixed sample whose shapes are not multiples of the tiles: rows and
    columns beyond M and N, K remainders (whole k-steps and odd ones), 16-bit outputs, 2..16-wide thread
    tiles also for the scalar kernel, one-wave blocks, narrow load widths."""
    rng = random.Random(seed)
    out = []
    want = {_native.KIND_MFMA: n_matrix, _native.KIND_SIMT: n_simt}
    have = {_native.KIND_MFMA: 0, _native.KIND_SIMT: 0}
    while have != want:
        kind = rng.choice([_native.KIND_SIMT, _native.KIND_MFMA, _native.KIND_MFMA])
        if have[kind] == want[kind]:
            continue
        dtype = rng.choice([2, 3, 4, 4, 8])
        g = {2: 8, 3: 8, 4: 4, 8: 2}[dtype]
        BM, BN = rng.choice([32, 64, 128, 256]), rng.choice([32, 64, 128, 256])
        BK = rng.choice([8, 16, 32, 64] if dtype in (4, 8) else [16, 32, 64])
        kw = dict(BM=BM, BN=BN, BK=BK, TM=rng.choice([2, 4, 8, 16]), TN=rng.choice([2, 4, 8, 16]),
                  warp_layout=rng.choice([(8, 8), (8, 8), (4, 16), (16, 4)]), dtype=dtype, is_atrans=rng.choice([0, 1]),
                  block_mapping=rng.choice([0, 2, 8]), lsu=rng.choice([1, 1, 1, 2]),
                  load_continuous=rng.choice([0, 1, 1, 1]), reduce_c_continuous=rng.choice([0, 1]))
        kw["shared_prefetch"], kw["reg_prefetch"] = rng.choice([(1, 1), (1, 1), (1, 1), (1, 0), (0, 1), (0, 0)])
        out16 = dtype in (2, 3) and rng.random() < 0.3
        if dtype in (2, 3):
            kw["dtype_c"] = dtype if out16 else 4
        if rng.random() < 0.3:
            kw["scatter"] = rng.choice([1, 2])
        if rng.random() < 0.1:
            kw["glw"] = rng.choice([1, 2])
        kt = rng.choice([1, 2, 3] if out16 else [1, 2, 3, 4, 5, 7, 9, 12, 17])     # 16-bit sums must stay exact
        kw.update(M=BM * rng.choice([1, 2]) - rng.choice([0, 0, g, 3 * g, 1, 5, BM - g]),
                  N=BN * rng.choice([1, 2, 3]) - rng.choice([0, 0, g, 2 * g, 3, BN - g]),
                  K=BK * kt + rng.choice([0, 0, 8, 16, 32, 4, 24, 2, 1, 5]) % BK)
        if kw["M"] <= 0 or kw["N"] <= 0:
            continue
        try:
            cfg = make_config(**kw)
            if _native.is_valid_config(kernelArgFromConfig(cfg).values(), kind):
                out.append((cfg, kind))
                have[kind] += 1
        except (ValueError, _native.KcgError):
            continue
    # ... and configs that take the direct-staging kernel with such shapes (K remainders included)
    n = 0
    while n < n_direct:
        dtype = rng.choice([2, 3, 4, 4])
        g = 4 if dtype == 4 else 8
        BM, BN = rng.choice([64, 128, 256]), rng.choice([64, 128, 256])
        BK = rng.choice([8, 16, 32, 64] if dtype == 4 else [16, 32, 64])
        out16 = dtype != 4 and rng.random() < 0.3
        kt = rng.choice([1, 2, 3] if out16 else [1, 2, 3, 4, 5, 7, 9, 12, 17])
        kw = dict(BM=BM, BN=BN, BK=BK, TM=rng.choice([2, 4, 8, 16]), TN=rng.choice([2, 4, 8, 16]),
                  warp_layout=rng.choice([(8, 8), (8, 8), (4, 16), (16, 4)]), dtype=dtype, is_atrans=rng.choice([0, 1]),
                  block_mapping=rng.choice([0, 2, 4, 8]), shared_prefetch=1, reg_prefetch=1,
                  M=BM * rng.choice([1, 2]) - g * rng.choice([0, 1, 3, BM // g - 1, BM // (2 * g)]),
                  N=BN * rng.choice([1, 2, 3]) - g * rng.choice([0, 1, 2, BN // g - 1, BN // (2 * g)]),
                  K=BK * kt + rng.choice([0, 8, 16, 32, 48]) % BK)
        if dtype != 4:
            kw["dtype_c"] = dtype if out16 else 4
        if kw["M"] <= 0 or kw["N"] <= 0 or (kw["M"] % BM == 0 and kw["N"] % BN == 0 and kw["K"] % BK == 0):
            continue
        try:
            cfg = make_config(**kw)
            v = kernelArgFromConfig(cfg).values()
            if _native.is_valid_config(v, _native.KIND_MFMA) and \
                    "DIRECT = true" in _native.instantiation_source(v, _native.KIND_MFMA):
                out.append((cfg, _native.KIND_MFMA))
                n += 1
        except (ValueError, _native.KcgError):
            continue
    return out


def random_odd_direct_configs(n=30, seed=20251125):
    """-> [(config, kind)]: a third fixed sample: fp32 configs that take the direct-staging kernel although M, N
    or K is not a multiple of the 16-byte vector (rows of A and B then do not start on 16-byte boundaries and
    the kernel fetches element by element): odd extents in every dimension, K remainders of any length, both A
    layouts, all matrix-core tile shapes and block sizes."""
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        BM, BN = rng.choice([32, 64, 128, 256]), rng.choice([32, 64, 128, 256])
        BK = rng.choice([8, 16, 32, 64])
        kt = rng.choice([1, 2, 3, 4, 5, 7, 9, 12, 17])
        kw = dict(BM=BM, BN=BN, BK=BK, TM=rng.choice([2, 4, 8, 16]), TN=rng.choice([2, 4, 8, 16]),
                  warp_layout=rng.choice([(8, 8), (8, 8), (4, 16), (16, 4)]), dtype=4, is_atrans=rng.choice([0, 1]),
                  block_mapping=rng.choice([0, 2, 4, 8]), shared_prefetch=1, reg_prefetch=1,
                  M=BM * rng.choice([1, 2]) - rng.choice([0, 1, 2, 3, 5, 7, BM - 1, BM // 2 + 1]),
                  N=BN * rng.choice([1, 2, 3]) - rng.choice([0, 1, 2, 3, 6, 9, BN - 1, BN // 2 - 1]),
                  K=BK * kt + rng.choice([0, 1, 2, 3, 5, 6, 7, 9, 13, 31]) % BK)
        if kw["M"] <= 0 or kw["N"] <= 0 or (kw["M"] % 4 == 0 and kw["N"] % 4 == 0 and kw["K"] % 4 == 0):
            continue
        try:
            cfg = make_config(**kw)
            v = kernelArgFromConfig(cfg).values()
            if _native.is_valid_config(v, _native.KIND_MFMA) and \
                    "DIRECT = true" in _native.instantiation_source(v, _native.KIND_MFMA):
                out.append((cfg, _native.KIND_MFMA))
        except (ValueError, _native.KcgError):
            continue
    return out


def random_even_16bit_direct_configs(n=20, seed=20251126):
    """-> [(config, kind)]: fp16 / bf16 configs that take the direct-staging kernel although M, N or K is not a
    multiple of 8 (all three even: the kernel then fetches two elements per lane), K remainders of any even length,
    both A layouts, 16-bit and fp32 outputs."""
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        dtype = rng.choice([2, 3])
        BM, BN = rng.choice([32, 64, 128, 256]), rng.choice([32, 64, 128, 256])
        BK = rng.choice([16, 32, 64])
        out16 = rng.random() < 0.3
        kt = rng.choice([1, 2, 3] if out16 else [1, 2, 3, 4, 5, 7, 9, 12])
        kw = dict(BM=BM, BN=BN, BK=BK, TM=rng.choice([2, 4, 8, 16]), TN=rng.choice([2, 4, 8, 16]),
                  warp_layout=rng.choice([(8, 8), (8, 8), (4, 16), (16, 4)]), dtype=dtype, dtype_c=dtype if out16 else 4,
                  is_atrans=rng.choice([0, 1]), block_mapping=rng.choice([0, 2, 4, 8]), shared_prefetch=1, reg_prefetch=1,
                  M=BM * rng.choice([1, 2]) - rng.choice([0, 2, 4, 6, 10, BM - 2, BM // 2 + 2]),
                  N=BN * rng.choice([1, 2, 3]) - rng.choice([0, 2, 4, 6, 12, BN - 2, BN // 2 - 2]),
                  K=BK * kt + rng.choice([0, 2, 4, 6, 10, 14, 30]) % BK)
        if kw["M"] <= 0 or kw["N"] <= 0 or (kw["M"] % 8 == 0 and kw["N"] % 8 == 0 and kw["K"] % 8 == 0):
            continue
        try:
            cfg = make_config(**kw)
            v = kernelArgFromConfig(cfg).values()
            if _native.is_valid_config(v, _native.KIND_MFMA) and \
                    "DIRECT = true" in _native.instantiation_source(v, _native.KIND_MFMA):
                out.append((cfg, _native.KIND_MFMA))
        except (ValueError, _native.KcgError):
            continue
    return out


def odd16_class(cfg):
    """Which special case of 16-bit rows of odd length a config exercises: 'a-kcont' / 'a-rowcont' / 'b' — that operand
    has an even number of odd-length rows, so its last row starts 2 bytes off a 4-byte boundary (the chunk at its end is
    fetched from further down and shifted into place, like the last chunk of every matrix whose rows are not whole
    chunks); 'k-odd' — the last k value shares its 32-bit word with one that does not exist; 'plain' — odd rows, none
    of these."""
    M, N, K, at = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"], cfg["IS_ATRANS"]
    out = []
    if not at and K % 2 == 1 and M % 2 == 0:
        out.append("a-kcont")
    if at and M % 2 == 1 and K % 2 == 0:
        out.append("a-rowcont")
    if N % 2 == 1 and K % 2 == 0:
        out.append("b")
    if K % 2 == 1:
        out.append("k-odd")
    return out or ["plain"]


def random_odd_16bit_direct_configs(n=36, seed=20251127):
    """-> [(config, kind)]: fp16 / bf16 configs with an odd M, N or K that take the direct-staging kernel (rows that
    start 2 bytes off a 4-byte boundary), at least six of each class of odd16_class, K remainders of any length
    (also none: the last row of B then sits in a full tile), both A layouts, 16-bit and fp32 outputs."""
    rng = random.Random(seed)
    out, seen = [], {}
    while len(out) < n or min(seen.get(c, 0) for c in ("a-kcont", "a-rowcont", "b", "k-odd")) < 6:
        dtype = rng.choice([2, 3])
        BM, BN = rng.choice([32, 64, 128, 256]), rng.choice([32, 64, 128, 256])
        BK = rng.choice([16, 32, 64])
        out16 = rng.random() < 0.3
        kt = rng.choice([1, 2, 3] if out16 else [1, 2, 3, 4, 5, 7, 9, 12])
        kw = dict(BM=BM, BN=BN, BK=BK, TM=rng.choice([2, 4, 8, 16]), TN=rng.choice([2, 4, 8, 16]),
                  warp_layout=rng.choice([(8, 8), (8, 8), (4, 16), (16, 4)]), dtype=dtype, dtype_c=dtype if out16 else 4,
                  is_atrans=rng.choice([0, 1]), block_mapping=rng.choice([0, 2, 4, 8]), shared_prefetch=1, reg_prefetch=1,
                  M=BM * rng.choice([1, 2]) - rng.choice([0, 1, 2, 3, 5, 8, BM - 1, BM // 2 + 1]),
                  N=BN * rng.choice([1, 2, 3]) - rng.choice([0, 1, 2, 3, 7, 8, BN - 1, BN // 2 - 1]),
                  K=BK * kt + rng.choice([0, 0, 1, 2, 3, 5, 8, 13, 31]) % BK)
        if kw["M"] <= 0 or kw["N"] <= 0 or (kw["M"] % 2 == 0 and kw["N"] % 2 == 0 and kw["K"] % 2 == 0):
            continue
        try:
            cfg = make_config(**kw)
            v = kernelArgFromConfig(cfg).values()
            if _native.is_valid_config(v, _native.KIND_MFMA) and \
                    "DIRECT = true" in _native.instantiation_source(v, _native.KIND_MFMA):
                if len(out) >= n and all(seen.get(c, 0) >= 6 for c in odd16_class(cfg)):
                    continue
                out.append((cfg, _native.KIND_MFMA))
                for c in odd16_class(cfg):
                    seen[c] = seen.get(c, 0) + 1
        except (ValueError, _native.KcgError):
            continue
    return out


@pytest.mark.parametrize("hiprtc", hiprtc_params())
def test_random_odd_16bit_shapes_through_the_direct_kernel_are_bit_exact(hiprtc):
    """fp16 / bf16 with odd extents: every other row of an operand starts 2 bytes off a 4-byte boundary, the chunk
    at the end of a row brings the next row's first elements with it, and the chunk at the end of the matrix is fetched
    from further down and moved into place in LDS."""
    cases = random_odd_16bit_direct_configs()
    direct, classes = 0, {}
    for i, (cfg, kind) in enumerate(cases):
        M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
        lim = 2 if cfg["DATATYPE_C"] == 4 else 1       # 16-bit outputs: |sums| <= K <= 255 stay exact
        a = SI.small_ints((M, K), SI.STREAM_A, lim=lim)
        b = SI.small_ints((K, N), SI.STREAM_B, lim=lim)
        print(f"[case] random odd 16-bit direct {i} {odd16_class(cfg)} {kernelArgFromConfig(cfg).values()}", flush=True)
        got, info = run_gemm(cfg, a, b, kind, hiprtc=hiprtc)
        if info["lds_bytes"] == 0:
            direct += 1
            for c in odd16_class(cfg):
                classes[c] = classes.get(c, 0) + 1
        want = a.astype(np.float64) @ b.astype(np.float64)
        bad = int((got.astype(np.float64) != want).sum()) + int(np.isnan(got).sum())
        assert bad == 0, f"random odd 16-bit config {i} ({info['kernel_name']}): {bad} wrong elements"
    # (configs whose per-lane fetch offsets do not fit the register file are built with register staging instead)
    assert direct >= 28 and all(classes.get(c, 0) >= 4 for c in ("a-kcont", "a-rowcont", "b", "k-odd")), (direct, classes)


@pytest.mark.parametrize("hiprtc", hiprtc_params())
def test_random_odd_shapes_through_the_direct_kernel_are_bit_exact(hiprtc):
    cases = random_odd_direct_configs() + random_even_16bit_direct_configs()
    direct = 0
    for i, (cfg, kind) in enumerate(cases):
        M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
        lim = 2 if cfg["DATATYPE_C"] == 4 else 1       # 16-bit outputs: |sums| <= K <= 222 stay exact
        a = SI.small_ints((M, K), SI.STREAM_A, lim=lim)
        b = SI.small_ints((K, N), SI.STREAM_B, lim=lim)
        print(f"[case] random odd direct {i} {kernelArgFromConfig(cfg).values()}", flush=True)
        got, info = run_gemm(cfg, a, b, kind, hiprtc=hiprtc)
        direct += int(info["lds_bytes"] == 0)
        want = a.astype(np.float64) @ b.astype(np.float64)
        bad = int((got.astype(np.float64) != want).sum()) + int(np.isnan(got).sum())
        assert bad == 0, f"random odd config {i} ({info['kernel_name']}): {bad} wrong elements"
    # (a few of the sample need more registers for their per-lane fetch offsets than they have and are built with
    # register staging instead: the library's rule for direct-staging builds that would spill)
    assert direct >= 35


@pytest.mark.parametrize("hiprtc", hiprtc_params())
def test_random_edge_config_sample_is_bit_exact(hiprtc):
    """Entries in {-1, 0, 1}: every sum is an integer of magnitude <= K, exact in fp32 and, for the 16-bit
    outputs (K <= 255 there), in fp16 and bf16 as well."""
    cases = random_edge_configs()
    direct = 0
    for i, (cfg, kind) in enumerate(cases):
        M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
        a = SI.small_ints((M, K), SI.STREAM_A, lim=1)
        b = SI.small_ints((K, N), SI.STREAM_B, lim=1)
        print(f"[case] random edge {i} kind={kind} {kernelArgFromConfig(cfg).values()}", flush=True)
        got, info = run_gemm(cfg, a, b, kind, hiprtc=hiprtc)
        direct += int(kind == _native.KIND_MFMA and info["lds_bytes"] == 0)
        want = a.astype(np.float64) @ b.astype(np.float64)
        bad = int((got.astype(np.float64) != want).sum()) + int(np.isnan(got).sum())
        assert bad == 0, f"random edge config {i} ({info['kernel_name']}): {bad} wrong elements"
    assert direct >= 20


@pytest.mark.parametrize("hiprtc", hiprtc_params())
def test_random_config_sample_is_bit_exact(oracle, hiprtc):
    cases = random_configs()
    direct = 0
    for i, (cfg, kind) in enumerate(cases):
        M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
        a = SI.small_ints((M, K), SI.STREAM_A, lim=2)
        b = SI.small_ints((K, N), SI.STREAM_B, lim=2)
        print(f"[case] random {i} kind={kind} {kernelArgFromConfig(cfg).values()}", flush=True)
        got, info = run_gemm(cfg, a, b, kind, hiprtc=hiprtc)
        direct += int(kind == _native.KIND_MFMA and info["lds_bytes"] == 0)
        want = oracle.matmul(a, b, a_trans=False)
        bad = int((got != want).sum()) + int(np.isnan(got).sum())
        assert bad == 0, f"random config {i} ({info['kernel_name']}): {bad} wrong elements"
    assert direct >= 10          # the sample reaches the direct-staging kernel often enough to mean something
