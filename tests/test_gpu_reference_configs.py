"""The reference's own known-answer set for this path, on the GPU against the CPU oracle.

The reference ships no golden output vectors; what it does ship is (1) TuningCombs/best_combs_1024.json, the 270
configs its tuner kept for fp32 1024^3 — every one of them ran correctly on the authors' hardware (the tuner only
ranks kernels that pass its check against torch.matmul, Runtime/python/kcg/KCGTask.py:177) — and (2) the tuning
spaces its tuner enumerates (Runtime/python/kcg/TuningConfigs/GEMM_configs_1024.json, _2048.json, _4096.json).
"The existing config JSONs drive it unchanged" is checked here: all 270 kept configs, and a seeded sample of 64
points of each space drawn through ConfigGenerator with the reference's own pruning rules, run through the kcg API
on integer data and must equal the oracle (the exact integer product, which test_oracle ties to the oracle) bit for
bit.  Points of a space that the rules reject come back as KCG_ERR_INVALID_CONFIG, never as a kernel (CPU test).
The data files are the reference's, re-encoded by tests/golden/make_fixtures.py."""
import numpy as np
import pytest

from codegendemo_amd import _native
from codegendemo_amd.kcg import ConfigGenerator
from codegendemo_amd.kcg import SeededInputs as SI
from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig
from tests import fixtures
from tests.gemm_helpers import run_gemm

SPACES = ("GEMM_configs_1024.json", "GEMM_configs_2048.json", "GEMM_configs_4096.json")
SAMPLE, SEED = 64, 20261125


def space_sample(name):
    """-> (valid, rejected) of the reference's tuning space `name` (deterministic: the build step precompiles `valid`)."""
    return ConfigGenerator.sample_cfgs(fixtures.tuning_spaces()[name], SAMPLE, SEED)


def configs_to_build():
    out = [(cfg, _native.KIND_AUTO) for cfg in fixtures.best_combs_1024()]
    for name in SPACES:
        out += [(cfg, _native.KIND_AUTO) for cfg in space_sample(name)[0]]
    return out


class Problem:
    """Integer operands of one shape and their exact product (shared by all configs of that shape)."""
    _cache = {}

    @classmethod
    def get(cls, M, N, K, oracle):
        key = (M, N, K)
        if key not in cls._cache:
            a = SI.small_ints((M, K), SI.STREAM_A, lim=2)
            b = SI.small_ints((K, N), SI.STREAM_B, lim=2)
            want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)     # |sums| <= 4 K: exact
            rows = (M // 2, M // 2 + 16)                                                 # ... and equal to the oracle's
            assert np.array_equal(want[rows[0]:rows[1]], oracle.matmul(a, b, a_trans=False, rows=rows))
            cls._cache = {key: (a, b, want)}                                             # one shape at a time in memory
        return cls._cache[key]


def check_configs(configs, label, oracle):
    kinds = {1: 0, 2: 0}
    for i, cfg in enumerate(configs):
        M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
        a, b, want = Problem.get(M, N, K, oracle)
        print(f"[case] {label} {i} {kernelArgFromConfig(cfg).values()}", flush=True)
        got, info = run_gemm(cfg, a, b, _native.KIND_AUTO, poison=(i % 8 == 0))
        kinds[info["kind"]] += 1
        bad = int((got != want).sum()) + int(np.isnan(got).sum())
        assert bad == 0, f"{label} config {i} ({info['kernel_name']}): {bad} wrong elements"
    return kinds


@pytest.mark.gpu
def test_all_270_configs_the_reference_tuner_kept_are_bit_exact(oracle):
    configs = fixtures.best_combs_1024()
    assert len(configs) == 270 and all(c["IS_ATRANS"] == 1 and c["M_SIZE"] == 1024 for c in configs)
    kinds = check_configs(configs, "best_combs_1024", oracle)
    assert kinds[1] > 0 and kinds[2] > 0          # both kernel families serve the reference's file


@pytest.mark.gpu
@pytest.mark.parametrize("name", SPACES)
def test_sample_of_a_reference_tuning_space_is_bit_exact(oracle, name):
    valid, _ = space_sample(name)
    assert len(valid) == SAMPLE
    check_configs(valid, name, oracle)


@pytest.mark.parametrize("name", SPACES)
def test_rejected_points_of_a_reference_tuning_space_are_reported_not_built(name, tmp_path, monkeypatch):
    monkeypatch.setenv("KCG_CACHE_DIR", str(tmp_path))
    valid, rejected = space_sample(name)
    assert len(valid) == SAMPLE and len(rejected) == SAMPLE
    for cfg in rejected:
        values = [int(cfg[k]) for k in _native.keywords()]
        c = _native.make_cfg(values)
        info = _native.KernelInfo()
        import ctypes
        assert _native.lib().kcg_compile_matmul(ctypes.byref(c), b"gfx950", _native.KIND_AUTO, ctypes.byref(info)) == _native.ERR_INVALID_CONFIG
        assert _native.last_error().startswith("invalid config:")
    assert not any(f.endswith(".hsaco") for f in __import__("os").listdir(tmp_path))
    for cfg in valid[:3]:                                  # ... and the valid ones are accepted
        _native.check_config(kernelArgFromConfig(cfg).values())
