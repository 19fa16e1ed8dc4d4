"""The autotune loop's plumbing on the CPU: spawn-per-config compile processes, pickle hand-off, the
perf-tester process with its watchdog, the top-K result JSON and resume.  The per-kernel measurement is
injected (no GPU here); what is exercised is the control flow the reference has in KCGTask.py:226-457.
Failure handling is forced from the host: the injected measurement kills its own process once."""
import ctypes
import json
import multiprocessing
import os
import time

import pytest

from codegendemo_amd.kcg import KCGTask
from codegendemo_amd.kcg.ConfigGenerator import make_config, save_to_json
from codegendemo_amd.kcg.KCGTask import KernelTestResult, ParallelTaskManager, PerfTester, SerialCompileTask
from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig
from codegendemo_amd.kcg.Utils import PathManager, deserialize_from_file


def fake_perf(kpm, inConfig, packedKernel):
    """Stands in for PerfTester._test_perf: 'speed-up' is a pure function of the config."""
    assert os.path.isfile(inConfig.hsacoPath) and packedKernel.kernelName == inConfig.kernelFuncName
    r = KernelTestResult(kpm)
    r.isCorrect = kpm.BLOCK_SIZE_K != 8            # pretend the BK=8 kernel produced wrong results
    r.torch_elapseTimeMs = 1.0
    r.kcg_elapseTimeMs = 16.0 / kpm.BLOCK_SIZE_K
    r.acc = r.torch_elapseTimeMs / r.kcg_elapseTimeMs
    return r


def fake_perf_dies_once(kpm, inConfig, packedKernel):
    marker = os.path.join(os.environ["KCG_WORK_DIR"], "died_once")
    if not os.path.exists(marker):
        open(marker, "w").close()
        os._exit(7)                                # a faulting kernel takes the whole process down
    return fake_perf(kpm, inConfig, packedKernel)


@pytest.fixture()
def workdir(tmp_path, monkeypatch):
    monkeypatch.setenv("KCG_WORK_DIR", str(tmp_path / "work"))
    monkeypatch.setenv("KCG_CACHE_DIR", str(tmp_path / "codeobj"))
    PathManager.init(clearPkl=True, clearTmp=True, clearCache=True)
    return tmp_path


def _write_cfgs(path, cfgs):
    save_to_json({"cfgs": cfgs}, str(path))
    return str(path)


def test_compile_task_writes_pickle(workdir):
    lock = multiprocessing.get_context("spawn").Lock()
    kpms = [kernelArgFromConfig(make_config(256, 256, 128, BK=bk)) for bk in (16, 32)]
    bad = kernelArgFromConfig(make_config(256, 256, 128))
    bad.WARP_LAYOUT_M = 4
    out = SerialCompileTask().compile_kernels(lock, kpms + [bad], 0, 3, "unit", 0)
    assert len(out) == 2                                        # the invalid config is skipped, not fatal
    pkls = os.listdir(PathManager.pikle_dir())
    assert pkls == ["valid_kernels_unit_0_3.pkl"]
    back = deserialize_from_file(os.path.join(PathManager.pikle_dir(), pkls[0]))
    assert [t[0].BLOCK_SIZE_K for t in back] == [16, 32]
    assert back[0][2].m_launcher.m_kernelLib.m_kernelInfo is None and back[0][1].sharedMem() == back[0][2].shmSize
    # a truncated pickle reads as "no kernels" (Utils.py:44-51)
    p = os.path.join(PathManager.pikle_dir(), "broken.pkl")
    with open(p, "wb") as f:
        f.write(b"\x80\x04\x95")
    assert deserialize_from_file(p) == []


def test_parallel_task_manager_end_to_end(workdir):
    cfgs = [make_config(256, 256, 128, BK=bk, shared_prefetch=sp) for bk in (8, 16, 32) for sp in (0, 1)]
    cfgs.append(dict(make_config(256, 256, 128), WARP_LAYOUT_M=4))          # invalid: skipped by its compile process
    j1 = _write_cfgs(workdir / "tmp_json_0_4.json", cfgs[:4])
    j2 = _write_cfgs(workdir / "tmp_json_4_7.json", cfgs[4:])
    perf = str(workdir / "perfRecord")
    tm = ParallelTaskManager(len(cfgs), [j1, j2], perf, benchmarkcnt=3, warmupcnt=1, devId=0, keepTopNum=3,
                             perfTestFn=fake_perf)
    tm.run(maxProcess=3, needCompile=True, needPerfTest=True)
    with open(perf + "_0.json") as f:
        res = json.load(f)["results"]
    assert len(res) == 3                                                   # top-3 kept
    assert [r["config"]["BLOCK_SIZE_K"] for r in res[:2]] == [32, 32]      # sorted by speed-up
    assert all(r["correct"] for r in res) and all(r["config"]["BLOCK_SIZE_K"] != 8 for r in res)
    assert set(res[0].keys()) >= {"correct", "acc", "torchMs", "kcgMs", "config"}   # KCGTask.py:39-46
    assert res[0]["acc"] == pytest.approx(2.0)
    assert os.listdir(PathManager.pikle_dir()) == []                       # every hand-off file consumed
    # resume from a sub-JSON: only the second file is compiled
    tm2 = ParallelTaskManager(len(cfgs), [j1, j2], str(workdir / "perf2"), keepTopNum=10, perfTestFn=fake_perf)
    tm2.run(maxProcess=4, startFromSubjson=j2, needCompile=True, needPerfTest=True)
    with open(str(workdir / "perf2") + "_0.json") as f:
        res2 = json.load(f)["results"]
    assert sorted(r["config"]["SHARED_PREFETCH"] for r in res2) == [0, 1] and \
        all(r["config"]["BLOCK_SIZE_K"] == 32 for r in res2)


def test_watchdog_restarts_a_dead_perf_tester_and_resumes(workdir):
    ctx = multiprocessing.get_context("spawn")
    lock = ctx.Lock()
    mgr = ctx.Manager()
    end = mgr.Value(ctypes.c_int, 0)
    perf = str(workdir / "perfRecord")
    # results of an earlier life of the tester, already on disk
    prev = KernelTestResult(kernelArgFromConfig(make_config(256, 256, 128, BK=64)))
    prev.isCorrect, prev.acc, prev.torch_elapseTimeMs, prev.kcg_elapseTimeMs = True, 4.0, 1.0, 0.25
    with open(perf + "_0.json", "w") as f:
        json.dump(PerfTester.jsonfyBestPerfs([prev]), f)
    SerialCompileTask().compile_kernels(lock, [kernelArgFromConfig(make_config(256, 256, 128, BK=16))], 0, 1, "first", 0)
    mon = ctx.Process(target=KCGTask._perf_monitor,
                      args=(ctx, lock, end, perf, 3, 1, 0, 5, "", 1, fake_perf_dies_once, 3))
    mon.start()
    deadline = time.time() + 60
    while not os.path.exists(os.path.join(str(workdir / "work"), "died_once")) and time.time() < deadline:
        time.sleep(0.2)
    assert os.path.exists(os.path.join(str(workdir / "work"), "died_once"))
    SerialCompileTask().compile_kernels(lock, [kernelArgFromConfig(make_config(256, 256, 128, BK=32))], 0, 1, "second", 0)
    time.sleep(0.5)
    end.value = 1
    mon.join(60)
    assert not mon.is_alive() and mon.exitcode == 0
    with open(perf + "_0.json") as f:
        res = json.load(f)["results"]
    ks = [r["config"]["BLOCK_SIZE_K"] for r in res]
    assert 64 in ks and 32 in ks          # earlier top-K re-seeded from the JSON, new kernel measured after restart
    assert ks == sorted(ks, reverse=True)


def test_best_perf_bookkeeping():
    PerfTester.BestPerf = []
    rs = []
    for acc, ok in ((1.0, True), (3.0, True), (9.0, False), (2.0, True)):
        r = KernelTestResult(kernelArgFromConfig(make_config(256, 256, 128)))
        r.acc, r.isCorrect = acc, ok
        rs.append(r)
    best = PerfTester._getBestPerf(rs, topNum=2)
    assert [b.acc for b in best] == [3.0, 2.0]
    j = PerfTester.jsonfyBestPerfs(best)
    back = KernelTestResult(kernelArgFromConfig(make_config(8, 8, 8)))
    back.parseFromJson(j["results"][0])
    assert back.acc == 3.0 and back.kpm == rs[1].kpm
    PerfTester.BestPerf = []


def test_stored_library_time_is_keyed_by_shape_types_and_device(workdir):
    """The library GEMM time kept in _cache/benchmarkTorchEps.log is reused only for the shape, types and
    device it was measured for (a tuning file with mixed shapes must not inherit the first shape's time)."""
    os.makedirs(PathManager.default_cache_dir(), exist_ok=True)
    old_shape, old_eps = PerfTester._shape, PerfTester.torch_eps
    try:
        PerfTester._shape = (1024, 1024, 1024, 4, 4)
        with open(PerfTester._torchEpsStoreFile(), "w") as f:
            json.dump({"key": PerfTester._torch_eps_key(), "ms": 0.04}, f)
        PerfTester.torch_eps = 0.0
        assert PerfTester._read_torch_eps_from_file() and PerfTester.torch_eps == 0.04
        PerfTester._shape = (2048, 2048, 2048, 4, 4)
        PerfTester.torch_eps = 0.0
        assert not PerfTester._read_torch_eps_from_file() and PerfTester.torch_eps == 0.0
        with open(PerfTester._torchEpsStoreFile(), "w") as f:
            f.write("0.123")                                       # the reference's bare number: ignored
        assert not PerfTester._read_torch_eps_from_file()
    finally:
        PerfTester._shape, PerfTester.torch_eps = old_shape, old_eps
