"""BASELINE config 2 on the GPU: the fp32 2048^3 sweep over BM/BN in {32,64,128}, BK in {8,16,32},
TM/TN in {4,8}, LDS prefetch on/off (and, beyond the BASELINE grid, register prefetch on/off, which
together with LDS prefetch routes eligible tiles to the direct-staging kernel).  Every feasible grid point must compile, launch, return a timing
and match the CPU oracle within 1e-4*K*max|a|*max|b|; infeasible points (no block/warp layout exists)
are reported as skipped, not failed."""
import os

import numpy as np
import pytest

from codegendemo_amd import _native
from codegendemo_amd.kcg import SeededInputs as SI
from codegendemo_amd.kcg.ConfigGenerator import read_params, sweep_grid_points
from tests.gemm_helpers import build_kernel, fp32_tolerance, to_device

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SPACE = os.path.join(ROOT, "codegendemo_amd", "TuningConfigs", "GEMM_configs_2048_sweep.json")


def sweep_configs():
    return sweep_grid_points(read_params(SPACE))


def test_fp32_2048_sweep_every_config_is_correct_and_timed(oracle):
    import torch
    cfgs, skipped = sweep_configs()
    assert len(cfgs) + len(skipped) == 3 * 3 * 3 * 2 * 2 * 2 * 2
    assert len(cfgs) >= 360
    M = N = K = 2048
    a = SI.uniform((M, K), SI.STREAM_A)
    b = SI.uniform((K, N), SI.STREAM_B)
    want = torch.from_numpy(oracle.matmul(a, b, a_trans=False)).to("cuda:0")
    tol = fp32_tolerance(K, a, b)
    a_dev = to_device(a, torch.float32)
    b_dev = to_device(b, torch.float32)
    results = []
    kinds = {1: 0, 2: 0}
    direct = 0
    poison_a = torch.full_like(a_dev, float("nan"))
    poison_b = torch.full_like(b_dev, float("nan"))
    for i, cfg in enumerate(cfgs):
        tag = "BM{BLOCK_SIZE_M} BN{BLOCK_SIZE_N} BK{BLOCK_SIZE_K} TM{THREAD_SIZE_M} TN{THREAD_SIZE_N} SHMP{SHARED_PREFETCH} REGP{REG_PREFETCH}".format(**cfg)
        print(f"[case] sweep {i} {tag}", flush=True)
        kpm, ui, kernel, info = build_kernel(cfg)
        kinds[info["kind"]] += 1
        direct += int(info["kind"] == 2 and info["lds_bytes"] == 0)
        c_dev = torch.empty((M, N), dtype=torch.float32, device="cuda:0")
        kernel.run(poison_a, poison_b, c_dev)     # leaves NaN in LDS: a read ahead of its fetch would show
        c_dev.fill_(float("nan"))
        kernel.run(a_dev, b_dev, c_dev)
        torch.cuda.synchronize()
        err = float((c_dev - want).abs().max().item())
        assert err <= tol, f"{tag}: max|err| {err} > {tol}"       # NaN (unwritten C) fails too
        med, mn = kernel.benchmark(a_dev, b_dev, c_dev, warmup=1, iters=3, reps=0)
        assert med > 0
        results.append((2.0 * M * N * K / med / 1e9, tag, info["kind"]))
        kernel.unload()
    results.sort(reverse=True)
    print(f"sweep: {len(cfgs)} configs ok ({kinds[2]} matrix-core, {direct} of them direct-staging, {kinds[1]} SIMT), "
          f"{len(skipped)} grid points skipped")
    for tf, tag, kind in results[:5]:
        print(f"   {tf:7.1f} TFLOPS  {tag} kind={kind}")
    assert kinds[1] > 0 and kinds[2] > 0 and direct > 0
