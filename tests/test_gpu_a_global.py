"""A straight from global memory (the build switch -DKCG_A_GLOBAL=1 of the direct-staging kernel): a k-contiguous A
has the fragment layout of the matrix-core instructions in memory, so its fragments can be loaded with one
global_load_dwordx4 per lane instead of going through LDS; the kernel then counts those loads and its global->LDS
fetches of B on one in-order counter (VmSchedule).  The switch is off in the product (measured: slower, see the
profile of the fp16 kernel); these cases keep it correct: bit-exact on integers for every tile shape class, edge tiles
in M and N, 1..17 K tiles (shorter than, equal to and longer than the stage ring), and block rows of which whole wave
rows lie beyond M - such a wave once computed negative row offsets, which a 32-bit unsigned lane offset turns into
addresses 4 GiB further on."""
import numpy as np
import pytest

from codegendemo_amd import _native
from codegendemo_amd.kcg import SeededInputs as SI
from codegendemo_amd.kcg.ConfigGenerator import make_config
from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig
from tests.gemm_helpers import run_gemm

FLAGS = "-DKCG_A_GLOBAL=1"
DIRECT = dict(shared_prefetch=1, reg_prefetch=1, is_atrans=0)
CASES = [
    ("f16-128x128x64-full", dict(M=256, N=384, K=64 * 9, dtype=2, dtype_c=4, BM=128, BN=128, BK=64, TM=8, TN=8)),
    ("f16-256x256x64-wave-rows-beyond-M", dict(M=383, N=250, K=64 * 5, dtype=2, dtype_c=4, BM=256, BN=256, BK=64, TM=16, TN=16)),
    ("bf16-128x128x32-one-step-tiles", dict(M=257, N=190, K=32 * 7, dtype=3, dtype_c=4, BM=128, BN=128, BK=32, TM=8, TN=8)),
    ("f16-64x64x32-M-1", dict(M=1, N=64, K=32 * 3, dtype=2, dtype_c=4, BM=64, BN=64, BK=32, TM=4, TN=4)),
    ("f32-256x256x32-17-tiles", dict(M=512, N=256, K=32 * 17, BM=256, BN=256, BK=32, TM=16, TN=8)),
    ("f32-128x128x16-edge", dict(M=127 + 128, N=129, K=16 * 4, BM=128, BN=128, BK=16, TM=8, TN=8)),
    ("f32-64x128x8-one-tile", dict(M=319, N=128, K=8, BM=128, BN=128, BK=8, TM=8, TN=8)),
    ("f16-out16-128x128x32", dict(M=250, N=256, K=32 * 2, dtype=2, dtype_c=2, BM=128, BN=128, BK=32, TM=8, TN=8)),
]


def configs_to_build():
    """(config, kind, epilogue, hiprtc, flags) for the build step."""
    return [(make_config(**kw, **DIRECT), _native.KIND_MFMA, None, None, FLAGS) for _tag, kw in CASES]


@pytest.mark.gpu
@pytest.mark.parametrize("tag,kw", CASES, ids=[c[0] for c in CASES])
def test_a_from_global_memory_is_bit_exact(oracle, tag, kw):
    cfg = make_config(**kw, **DIRECT)
    M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
    with _native.use_flags(FLAGS):
        assert "DIRECT = true" in _native.instantiation_source(kernelArgFromConfig(cfg).values(), _native.KIND_MFMA)
    lim = 2 if cfg["DATATYPE_C"] == 4 else 1
    a = SI.small_ints((M, K), SI.STREAM_A, lim=lim)
    b = SI.small_ints((K, N), SI.STREAM_B, lim=lim)
    print(f"[case] A from global memory {tag} {kernelArgFromConfig(cfg).values()}", flush=True)
    got, info = run_gemm(cfg, a, b, _native.KIND_MFMA, flags=FLAGS)
    assert info["lds_bytes"] == 0 and not info["direct_declined"]            # the direct-staging kernel
    want = oracle.matmul(a, b, a_trans=False)
    bad = int((got != want).sum()) + int(np.isnan(got).sum())
    assert bad == 0, f"{tag}: {bad} wrong elements"
