"""A fixed pseudo-random sample of tuning configs (both kernel families, all input types, both A layouts,
prefetch flags, split-U, odd tile/wave shapes, 1..17 K tiles), each checked bit for bit against the CPU
oracle on small-integer data.  The sample is deterministic, so the build step can precompile it."""
import random

import numpy as np
import pytest

from codegendemo_amd import _native
from codegendemo_amd.kcg import SeededInputs as SI
from codegendemo_amd.kcg.ConfigGenerator import make_config
from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig
from tests.gemm_helpers import run_gemm

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


def test_random_config_sample_is_bit_exact(oracle):
    cases = random_configs()
    direct = 0
    for i, (cfg, kind) in enumerate(cases):
        M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
        a = SI.small_ints((M, K), SI.STREAM_A, lim=2)
        b = SI.small_ints((K, N), SI.STREAM_B, lim=2)
        print(f"[case] random {i} kind={kind} {kernelArgFromConfig(cfg).values()}", flush=True)
        got, info = run_gemm(cfg, a, b, kind)
        direct += int(kind == _native.KIND_MFMA and info["lds_bytes"] == 0)
        want = oracle.matmul(a, b, a_trans=False)
        bad = int((got != want).sum()) + int(np.isnan(got).sum())
        assert bad == 0, f"random config {i} ({info['kernel_name']}): {bad} wrong elements"
    assert direct >= 10          # the sample reaches the direct-staging kernel often enough to mean something
