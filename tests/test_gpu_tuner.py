"""The autotune loop on the GPU, end to end: spawn-per-config compile processes, pickle hand-off, the
perf-tester process measuring with the C timing loop against the library GEMM, top-K JSON."""
import json
import os

import pytest

from codegendemo_amd.kcg.ConfigGenerator import make_config, save_to_json
from codegendemo_amd.kcg.KCGTask import ParallelTaskManager, PerfTester
from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig
from codegendemo_amd.kcg.Utils import PathManager

pytestmark = pytest.mark.gpu


def test_parallel_task_manager_on_gpu(tmp_path, monkeypatch):
    monkeypatch.setenv("KCG_WORK_DIR", str(tmp_path / "work"))
    PathManager.init(clearPkl=True, clearTmp=True, clearCache=True)
    M = N = K = 1024
    cfgs = [make_config(M, N, K, BM=64, BN=64, BK=16, TM=4, TN=4, is_atrans=at, shared_prefetch=sp, reg_prefetch=sp)
            for at in (0, 1) for sp in (0, 1)]
    cfgs.append(make_config(M, N, K, BM=128, BN=128, BK=16, TM=8, TN=8, is_atrans=0, shared_prefetch=1, reg_prefetch=1))
    cfgs.append(make_config(M, N, K, BM=32, BN=64, BK=8, TM=4, TN=4, warp_layout=(4, 16), is_atrans=1))   # SIMT kernel
    path = str(tmp_path / "tmp_json_0_6.json")
    save_to_json({"cfgs": cfgs}, path)
    perf = str(tmp_path / "perf")
    print("[case] tuner loop fp32 1024^3, 6 configs", flush=True)
    tm = ParallelTaskManager(len(cfgs), [path], perf, benchmarkcnt=5, warmupcnt=1, devId=0, keepTopNum=10,
                             nTorchEpsInitTest=5)
    tm.run(maxProcess=6, needCompile=True, needPerfTest=True)
    with open(perf + "_0.json") as f:
        res = json.load(f)["results"]
    assert len(res) == len(cfgs)                    # every kernel was correct against the library GEMM
    assert all(r["correct"] and r["kcgMs"] > 0 and r["torchMs"] > 0 and r["tflops"] > 1.0 for r in res)
    accs = [r["acc"] for r in res]
    assert accs == sorted(accs, reverse=True)
    got = {tuple(kernelArgFromConfig(r["config"]).values()) for r in res}
    assert got == {tuple(kernelArgFromConfig(c).values()) for c in cfgs}
    assert os.listdir(PathManager.pikle_dir()) == []


def test_perf_tester_fp16_in_process(tmp_path, monkeypatch):
    """PerfTester._test_perf with 16-bit inputs: relative tolerance against an fp32 product of the
    rounded inputs; direct-staging kernel."""
    monkeypatch.setenv("KCG_WORK_DIR", str(tmp_path / "work"))
    PathManager.init(clearCache=True)
    from tests.gemm_helpers import build_kernel
    PerfTester._a = PerfTester._b = None
    PerfTester.torch_eps = 0.0
    PerfTester.D = None
    cfg = make_config(1024, 1024, 1024, dtype=2, dtype_c=4, BM=128, BN=128, BK=64, TM=8, TN=8, is_atrans=0,
                      shared_prefetch=1, reg_prefetch=1)
    print("[case] PerfTester fp16 1024^3", flush=True)
    kpm, ui, kernel, info = build_kernel(cfg)
    assert info["lds_bytes"] == 0                   # static LDS stages: the direct-staging path was chosen
    PerfTester.setDevice(0)
    PerfTester._init_AB(kpm, ui)
    r = PerfTester._test_perf(kpm, ui, kernel, benchmarkCount=5, warmupCount=1, nTorchEpsInitTest=5)
    assert r.isCorrect and r.tflops > 10 and r.acc > 0
    PerfTester._a = PerfTester._b = PerfTester._aT = None
    PerfTester.D = None
    PerfTester.torch_eps = 0.0


ODD_BF16_CONFIG = make_config(1023, 1021, 1027, dtype=3, dtype_c=4, BM=128, BN=128, BK=32, TM=8, TN=8, is_atrans=1,
                              shared_prefetch=1, reg_prefetch=1)


def test_perf_tester_odd_extents_bf16_in_process(tmp_path, monkeypatch):
    """The tuner's own measurement and correctness gate on a problem the reference's checker rejects outright
    (matmul.py:293-298 wants M, N, K divisible by the tile): odd M, N and K, bf16, the `[K,M]` A layout."""
    monkeypatch.setenv("KCG_WORK_DIR", str(tmp_path / "work"))
    PathManager.init(clearCache=True)
    from tests.gemm_helpers import build_kernel
    PerfTester._a = PerfTester._b = None
    PerfTester.torch_eps = 0.0
    PerfTester.D = None
    print("[case] PerfTester bf16 1023x1021x1027", flush=True)
    kpm, ui, kernel, info = build_kernel(ODD_BF16_CONFIG)
    assert info["lds_bytes"] == 0                   # the direct-staging path
    PerfTester.setDevice(0)
    PerfTester._init_AB(kpm, ui)
    r = PerfTester._test_perf(kpm, ui, kernel, benchmarkCount=5, warmupCount=1, nTorchEpsInitTest=5)
    assert r.isCorrect and r.tflops > 10 and r.acc > 0
    PerfTester._a = PerfTester._b = PerfTester._aT = None
    PerfTester.D = None
    PerfTester.torch_eps = 0.0


@pytest.mark.parametrize("case", ["case_normal_0", "case_normal_1"])
def test_single_config_check_script(case, capsys):
    """python -m codegendemo_amd.kcg.test <case>: compile, one run, allclose(1e-2) against torch.matmul."""
    from codegendemo_amd.kcg import test as single
    print(f"[case] single-config check {case}", flush=True)
    assert single.main([case]) == 0
    out = capsys.readouterr().out
    assert "test correct!" in out and "speed up:" in out and "kernelName =  GEMM_MNK1024x" in out
