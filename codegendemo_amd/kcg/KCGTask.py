"""The autotune loop: compile tasks, the perf-tester process, its watchdog, and the top-K result log.

Counterpart of Runtime/python/kcg/KCGTask.py.  Control flow and file formats are the reference's:

  ParallelTaskManager.run            (:424-457)  one spawned compile process per config, joined every
                                                 `maxProcess`; a watchdog process owns the perf tester
  SerialCompileTask.compile_kernels  (:305-318)  compile -> pickle [(kpm, UserInputs, CompiledKernel)]
                                                 into <work>/_pkls under the shared lock
  PerfTester.runPerfTests            (:226-271)  poll _pkls, time every kernel, keep the top-N by
                                                 speed-up, rewrite <perf_out>_0.json after each batch
  watchdog                           (:342-368)  restart the perf tester if it dies before the end
                                                 signal, re-seeding the top-N from the JSON so far

What differs, on purpose: inputs are seeded (the reference draws unseeded torch.randn, :85-87), the
timing loop runs in C with HIP events (kcg_benchmark) instead of one Python-level event pair per
launch, and correctness is judged with a tolerance that fits the dtype (fp32: 2e-6*K*max|a|*max|b|, a fiftieth of
the acceptance bar of the parity tests, so that a kernel that drops one k-step is never ranked; 16-bit inputs: 2e-2
of the result scale) instead of allclose(atol=rtol=1e-1) (:177).
"""
import ctypes
import glob
import json
import multiprocessing
import os
import time
from typing import List, Tuple

import numpy as np

from . import SeededInputs
from .CompiledKernelFactory import CompiledKernelFactory, EnumOperator, UserInputs
from .KCGCompiler import KCGCompiler
from .Operators.matmul import KernelArgMatmul, kernelArgFromConfig
from .Utils import PathManager, deserialize_from_file, serialize_to_file


class KernelTestResult:
    def __init__(self, kpm: KernelArgMatmul):
        self.kpm = kpm
        self.isCorrect = False
        self.acc = 0.0
        self.kcg_elapseTimeMs = 0.0
        self.torch_elapseTimeMs = 0.0
        self.diffRate = 0.0
        self.maxError = 0.0
        self.tflops = 0.0
        self.nSpills = 0          # scratch dwords per lane of the kernel that was timed (0: no register spills)
        self.lowOpt = False       # the kernel is the engine's -O1 rebuild of a build that ran out of registers

    def __str__(self):
        return "{" + f"correct : {self.isCorrect}, acc : {self.acc}, torchMs : {self.torch_elapseTimeMs}], config : {self.kpm}" + "}"

    def jsonfy(self) -> dict:
        # schema of the reference's result log (KCGTask.py:39-46) + the absolute throughput and which build the
        # timing belongs to (a kernel that spills registers, or the slower -O1 rebuild of one)
        return {"correct": bool(self.isCorrect), "acc": float(self.acc), "torchMs": float(self.torch_elapseTimeMs),
                "kcgMs": float(self.kcg_elapseTimeMs), "tflops": float(self.tflops), "nSpills": int(self.nSpills),
                "lowOpt": bool(self.lowOpt), "config": self.kpm.jsonfy()}

    def parseFromJson(self, jsonObj):
        self.isCorrect = jsonObj["correct"]
        self.acc = jsonObj["acc"]
        self.torch_elapseTimeMs = jsonObj["torchMs"]
        self.kcg_elapseTimeMs = jsonObj["kcgMs"]
        self.tflops = jsonObj.get("tflops", 0.0)
        self.nSpills = jsonObj.get("nSpills", 0)
        self.lowOpt = jsonObj.get("lowOpt", False)
        self.kpm = KernelArgMatmul(0, 0, 0, 1, 1, 1)
        self.kpm.assignWithJson(jsonObj["config"])


class PerfTester:
    _a = None            # logical [M,K] on the device
    _b = None
    _aT = None           # [K,M] copy for IS_ATRANS=1 kernels
    _shape = None
    torch_eps = 0.0      # baseline (torch.matmul -> hipBLASLt/rocBLAS) median ms
    D = None             # baseline result, the correctness reference inside the tuner
    tol = 0.0
    BestPerf = []        # List[KernelTestResult]
    torchDynamicEps = []
    check_dynamic_torch_perf = 2000
    currentDevId = 0
    seed = SeededInputs.SEED

    @staticmethod
    def _torchEpsStoreFile():
        return os.path.join(PathManager.default_cache_dir(), "benchmarkTorchEps.log")

    @staticmethod
    def _compare_with_error(tensor1, tensor2, abs_error=1e-2, rel_error=1e-2):
        import torch
        abs_diff = torch.abs(tensor1 - tensor2)
        rel_diff = abs_diff / (torch.abs(tensor1) + 1e-5)
        error_mask = (abs_diff > abs_error) & (rel_diff > rel_error)
        return torch.sum(error_mask).item(), torch.max(abs_diff).item()

    @staticmethod
    def setDevice(devId: int):
        if PerfTester.currentDevId != devId:
            PerfTester.currentDevId = devId
            PerfTester._a = PerfTester._b = PerfTester._aT = None
            PerfTester._shape = None

    @staticmethod
    def _init_AB(kpm: KernelArgMatmul, inConfig: UserInputs):
        """Seeded N(0,1) inputs in the config's input dtype (the reference: torch.randn)."""
        import torch
        dev = f"cuda:{PerfTester.currentDevId}"
        ta = inConfig.kernelParam.dtypeTorch('A')
        a = SeededInputs.normal((kpm.M, kpm.K), SeededInputs.STREAM_A, seed=PerfTester.seed)
        b = SeededInputs.normal((kpm.K, kpm.N), SeededInputs.STREAM_B, seed=PerfTester.seed)
        PerfTester._a = torch.from_numpy(a).to(device=dev, dtype=ta)
        PerfTester._b = torch.from_numpy(b).to(device=dev, dtype=ta)
        PerfTester._aT = PerfTester._a.t().contiguous()
        PerfTester._shape = (kpm.M, kpm.N, kpm.K, int(kpm.dtype('A')), int(kpm.dtype('C')))
        PerfTester.D = None
        PerfTester.torch_eps = 0.0
        amax = float(PerfTester._a.abs().max().item())
        bmax = float(PerfTester._b.abs().max().item())
        if int(kpm.dtype('A')) in (4, 8):
            # The tuner's own gate is 50 times tighter than the acceptance bar (1e-4 * K * max|a| * max|b|, which
            # the parity tests apply): a kernel that drops or repeats one k-step is off by up to max|a| * max|b|
            # in some element and must not be ranked, while correct kernels differ from the library by a few
            # 1e-4 at K = 4096 (rounding order only).
            PerfTester.tol = 2e-6 * kpm.K * amax * bmax
        else:
            PerfTester.tol = None   # relative, needs the result scale: set with D

    @staticmethod
    def _baseline(out_dtype):
        import torch
        d = torch.matmul(PerfTester._a, PerfTester._b)
        return d if d.dtype == out_dtype else d.to(out_dtype)

    @staticmethod
    def _inner_test_torch(out_dtype=None):
        import torch
        ev0 = torch.cuda.Event(enable_timing=True)
        ev1 = torch.cuda.Event(enable_timing=True)
        ev0.record()
        d = torch.matmul(PerfTester._a, PerfTester._b)
        ev1.record()
        torch.cuda.synchronize()
        return d, ev0.elapsed_time(ev1)

    @staticmethod
    def _init_torch_eps(nTorchEpsInitTest, out_dtype):
        import torch
        eps = []
        d = None
        for _ in range(max(1, nTorchEpsInitTest)):
            d, t = PerfTester._inner_test_torch()
            eps.append(t)
        if not PerfTester._read_torch_eps_from_file():
            PerfTester.torch_eps = float(np.median(eps))
        # the 16-bit baseline accumulates in fp32 inside the library but rounds its output to 16 bits;
        # for fp32-output kernels compare against an fp32 product of the same (already rounded) inputs
        if d.dtype != out_dtype:
            d = torch.matmul(PerfTester._a.to(torch.float32), PerfTester._b.to(torch.float32)).to(out_dtype)
        PerfTester.D = d
        if PerfTester.tol is None:
            PerfTester.tol = 2e-2 * float(torch.sqrt(torch.mean(d.to(torch.float32) ** 2)).item())
        os.makedirs(PathManager.default_cache_dir(), exist_ok=True)
        with open(PerfTester._torchEpsStoreFile(), "w") as f:
            json.dump({"key": PerfTester._torch_eps_key(), "ms": PerfTester.torch_eps}, f)

    @staticmethod
    def _torch_eps_key():
        """What a stored library time belongs to: shape, types and device (the reference's file holds a bare
        number, KCGTask.py:106-121, and would hand one shape's time to the next)."""
        return [int(x) for x in (PerfTester._shape or ())] + [int(PerfTester.currentDevId)]

    @staticmethod
    def _read_torch_eps_from_file():
        """The library time a previous perf process stored for this very shape, types and device (the watchdog's
        resume path); anything else in the file is ignored."""
        try:
            with open(PerfTester._torchEpsStoreFile(), "r") as f:
                doc = json.load(f)
            if doc.get("key") != PerfTester._torch_eps_key():
                return False
            PerfTester.torch_eps = float(doc["ms"])
        except (OSError, ValueError, TypeError, KeyError, AttributeError):
            return False
        return PerfTester.torch_eps > 0

    @staticmethod
    def _inner_test_kcg(a, b, c, packedKernel, start_event, end_event):
        """One launch between two events on torch's stream — the reference's per-sample measurement
        (KCGTask.py:124-130); kept for comparability, the tuner itself uses the C timing loop."""
        import torch
        start_event.record()
        packedKernel.run(a, b, c)
        end_event.record()
        torch.cuda.synchronize()
        return c, start_event.elapsed_time(end_event)

    @staticmethod
    def _test_perf(kpm: KernelArgMatmul, inConfig: UserInputs, packedKernel, benchmarkCount=5, warmupCount=1,
                   nTorchEpsInitTest=50) -> KernelTestResult:
        import torch
        result = KernelTestResult(kpm)
        result.lowOpt = bool(getattr(inConfig, "m_buildFlags", 0) & 1)       # _native.BUILD_LOW_OPT
        result.nSpills = int(packedKernel.n_spills)
        dev = f"cuda:{PerfTester.currentDevId}"
        tc = inConfig.kernelParam.dtypeTorch('C')
        a, b = PerfTester._a, PerfTester._b
        a_ = PerfTester._aT if kpm.isATranspose else a
        c = torch.full((kpm.M, kpm.N), float("nan"), dtype=tc, device=dev)
        for _ in range(warmupCount):
            torch.matmul(a, b)
            packedKernel.run(a_, b, c)
        torch.cuda.synchronize()
        if PerfTester.torch_eps <= 0 or PerfTester.D is None:
            PerfTester._init_torch_eps(nTorchEpsInitTest, tc)
        median_ms, _min_ms = packedKernel.benchmark(a_, b, c, warmup=0, iters=benchmarkCount, reps=0)
        torch.cuda.synchronize()
        diff = (c.to(torch.float32) - PerfTester.D.to(torch.float32)).abs()
        max_error = float(diff.max().item())   # NaN (unwritten output) compares false below
        result.maxError = max_error
        if max_error <= PerfTester.tol:
            result.isCorrect = True
            result.torch_elapseTimeMs = PerfTester.torch_eps
            result.kcg_elapseTimeMs = float(median_ms)
            result.acc = result.torch_elapseTimeMs / result.kcg_elapseTimeMs
            result.tflops = 2.0 * kpm.M * kpm.N * kpm.K / (median_ms * 1e-3) / 1e12
            print(f"[perf] {result.kcg_elapseTimeMs:.4f} ms  {result.tflops:.1f} TFLOPS  baseline {result.torch_elapseTimeMs:.4f} ms"
                  f"  speed up {result.acc:.3f}  maxerr {max_error:.3e}", flush=True)
        else:
            ndiff, _ = PerfTester._compare_with_error(PerfTester.D.to(torch.float32), c.to(torch.float32))
            result.diffRate = ndiff / (kpm.M * kpm.N)
            print(f"[perf] test fail! maxerror={max_error}, tol={PerfTester.tol}, diffrate={result.diffRate}", flush=True)
        return result

    @staticmethod
    def _getBestPerf(perfData: List[KernelTestResult], topNum=1) -> List[KernelTestResult]:
        for d in perfData:
            if d.isCorrect:
                PerfTester.BestPerf.append(d)
        PerfTester.BestPerf.sort(key=lambda x: x.acc, reverse=True)
        PerfTester.BestPerf = PerfTester.BestPerf[:topNum]
        return PerfTester.BestPerf

    @staticmethod
    def jsonfyBestPerfs(best_perfs: List[KernelTestResult]) -> dict:
        return {"results": [r.jsonfy() for r in best_perfs]}

    @staticmethod
    def check_torch_dynamic_perf(torchPerfLogName, index):
        t = [PerfTester._inner_test_torch()[1] for _ in range(10)]
        new_eps = float(np.median(t))
        PerfTester.torchDynamicEps.append(new_eps)
        with open(torchPerfLogName, mode="a+") as ff:
            ff.write(f"[{index}] - {new_eps};\n")
        return new_eps

    @staticmethod
    def _load_best_from_json(path):
        """Re-seed the top-N from the JSON written so far (restart after a crash, KCGTask.py:358-364)."""
        try:
            with open(path) as f:
                obj = json.load(f)
        except (OSError, ValueError):
            return
        for cfg in obj.get("results", []):
            ktr = KernelTestResult(KernelArgMatmul(0, 0, 0, 1, 1, 1))
            ktr.parseFromJson(cfg)
            PerfTester.BestPerf.append(ktr)

    @staticmethod
    def runPerfTests(lock, endsignal, outputPAth=None, benchmarkCount=5, warmupCount=1, device='0', topNum=6,
                     torchDynamicLogPath='', nTorchEpsInitTest=50, resume=False, pollSeconds=1.0, testFn=None):
        """Poll <work>/_pkls for compiled kernels until the end signal is set and the directory is
        empty.  `testFn` (default PerfTester._test_perf) turns (kpm, UserInputs, CompiledKernel) into
        a KernelTestResult; tests of the loop's plumbing inject their own."""
        if resume and outputPAth:
            PerfTester._load_best_from_json(outputPAth)
        testFn = testFn or PerfTester._test_perf
        counter = 0
        while True:
            with lock:
                pklFiles = sorted(glob.glob(PathManager.pikle_dir() + "/*.pkl"))
                valid_kernels = []
                for pkl in pklFiles:
                    valid_kernels += deserialize_from_file(pkl)
                    try:
                        os.remove(pkl)
                    except OSError as e:
                        print(f"exception occur when delete {pkl}: {e}")
            if not pklFiles:
                if endsignal.value > 0:
                    break
                time.sleep(pollSeconds)
                continue
            print(f"====== Glob .pkl files : {len(pklFiles)}, Valid Kernels : {len(valid_kernels)} ========", flush=True)
            perf_data = []
            PerfTester.setDevice(int(device))
            for (kpm, inConfig, packedKernel) in valid_kernels:
                counter += 1
                if testFn is PerfTester._test_perf:
                    shape = (kpm.M, kpm.N, kpm.K, int(kpm.dtype('A')), int(kpm.dtype('C')))
                    if PerfTester._a is None or PerfTester._shape != shape:
                        PerfTester._init_AB(kpm, inConfig)
                    perf_data.append(testFn(kpm, inConfig, packedKernel, benchmarkCount, warmupCount, nTorchEpsInitTest))
                    if torchDynamicLogPath and counter % int(PerfTester.check_dynamic_torch_perf) == 0:
                        PerfTester.check_torch_dynamic_perf(torchDynamicLogPath, counter)
                else:
                    perf_data.append(testFn(kpm, inConfig, packedKernel))
            PerfTester._getBestPerf(perf_data, topNum)
            if PerfTester.BestPerf and outputPAth is not None:
                tmp = outputPAth + ".tmp"
                with open(tmp, mode="w") as f:
                    json.dump(PerfTester.jsonfyBestPerfs(PerfTester.BestPerf), f, indent=4)
                os.replace(tmp, outputPAth)
        print(f"=====[ PerfTest Finished ] =======\n   - Best : {[str(b) for b in PerfTester.BestPerf[:1]]} ", flush=True)


class SerialCompileTask:
    def _task_compile_kernel(self, kpm: KernelArgMatmul, index: int, deviceId: int) -> Tuple:
        compiler = KCGCompiler()
        hsacoPath, kernelName, gx, gy, gz, bx, by, bz = compiler.compileKernel(kpm)[0]
        inConfig = UserInputs(hsacoPath, kernelName, kpm)
        inConfig.m_gridDims = [gx, gy, gz]
        inConfig.m_blockDims = [bx, by, bz]
        inConfig.m_ldsBytes = compiler.lastInfo["lds_bytes"]
        inConfig.operatorKind = EnumOperator.Matmul
        packedKernel = CompiledKernelFactory.getKernel(inConfig, deviceId)
        return (kpm, inConfig, packedKernel)

    def compile_kernels(self, lock, kernelArgs: List[KernelArgMatmul], lbs=0, ubs=-1, namePrefix='', deviceId=0) -> List:
        output_path = PathManager.pikle_dir() + f"/valid_kernels_{namePrefix}_{lbs}_{ubs}.pkl"
        if ubs < 0:
            lbs, ubs = 0, len(kernelArgs)
        valid_kernels = []
        for i in range(lbs, ubs):
            try:
                valid_kernels.append(self._task_compile_kernel(kernelArgs[i], i, deviceId))
            except Exception as e:   # an invalid or uncompilable config costs only itself
                print(f"[compile] config {i} skipped: {str(e)[:400]}", flush=True)
        if valid_kernels:
            os.makedirs(PathManager.pikle_dir(), exist_ok=True)
            with lock:
                tmp = output_path + ".part"
                serialize_to_file(tmp, valid_kernels)
                os.replace(tmp, output_path)     # the perf tester only ever sees complete files
        return valid_kernels


def _perf_monitor(ctx, lock, endSignal, perf_out_path, nBenchMark, nWarmup, devId, topNum, torchDynamicLogPath,
                  nTorchEpsInitTest, testFn, maxRestarts):
    """Watchdog: owns the perf-tester process and restarts it when it exits without the end signal."""
    outfilename = f"{perf_out_path}_0.json"
    restarts = 0
    resume = False
    while True:
        p = ctx.Process(target=PerfTester.runPerfTests,
                        args=(lock, endSignal, outfilename, nBenchMark, nWarmup, str(devId), topNum,
                              torchDynamicLogPath, nTorchEpsInitTest, resume, 1.0, testFn))
        p.start()
        p.join()
        if p.exitcode == 0 and endSignal.value == 1:
            return
        if p.exitcode == 0 and endSignal.value != 1:
            continue
        restarts += 1
        print(f"======= [W] PerfTester Broken (exit {p.exitcode}). Restart it ==========", flush=True)
        if restarts > maxRestarts:
            print("======= [E] PerfTester keeps dying; giving up ==========", flush=True)
            return
        resume = True


class ParallelTaskManager:
    def __init__(self, total_cfg_count, json_path_arr: List[str], perf_out_path: str, benchmarkcnt=5, warmupcnt=1,
                 devId=0, keepTopNum=1, torchDynamicLogPath='', nTorchEpsInitTest=50, perfTestFn=None, maxRestarts=8):
        self.ctx = multiprocessing.get_context('spawn')
        self.Process = self.ctx.Process
        self.lock = self.ctx.Lock()
        self.subProcList = []
        self.cfg_json_path_arr = json_path_arr
        self.CFG_COUNT = total_cfg_count
        self._manager = self.ctx.Manager()
        self.endSignal = self._manager.Value(ctypes.c_int, 0)
        self.perf_out_path = perf_out_path
        self.nBenchMark = benchmarkcnt
        self.nWarmup = warmupcnt
        self.devId = devId
        self.topNum = keepTopNum
        self.torchDynamicLogPath = torchDynamicLogPath
        self.nTorchEpsInitTest = nTorchEpsInitTest
        self.perfTestFn = perfTestFn
        self.maxRestarts = maxRestarts
        self.perfProcMonitor = None

    def _createSubProc(self, func, *params):
        p = self.Process(target=func, args=(*params,))
        p.start()
        self.subProcList.append(p)

    def _waitAll(self):
        for s in self.subProcList:
            s.join()
        self.subProcList.clear()

    def _get_kernelargMatmul(self, json_path: str) -> List[KernelArgMatmul]:
        with open(json_path, "r") as f:
            json_data = json.load(f)
        return [kernelArgFromConfig(cfg) for cfg in json_data["cfgs"]]

    def run(self, maxProcess=10, startFromSubjson='', needCompile=True, needPerfTest=True):
        PathManager.init()
        started = not startFromSubjson
        procCount = dealed = 0
        if needPerfTest:
            self.perfProcMonitor = self.Process(
                target=_perf_monitor,
                args=(self.ctx, self.lock, self.endSignal, self.perf_out_path, self.nBenchMark, self.nWarmup,
                      self.devId, self.topNum, self.torchDynamicLogPath, self.nTorchEpsInitTest, self.perfTestFn,
                      self.maxRestarts))
            self.perfProcMonitor.start()
        if needCompile:
            for jsonPath in self.cfg_json_path_arr:
                if not started:
                    if jsonPath != startFromSubjson:
                        continue
                    started = True
                print(f"=========== Dealing json : {jsonPath} ================", flush=True)
                kernelConfigs = self._get_kernelargMatmul(jsonPath)
                namePrefix = os.path.basename(jsonPath).split('.')[0]
                for i in range(len(kernelConfigs)):
                    self._createSubProc(SerialCompileTask().compile_kernels, self.lock, kernelConfigs, i, i + 1,
                                        namePrefix, self.devId)
                    procCount += 1
                    dealed += 1
                    if procCount >= maxProcess:
                        print(f"========= Wating for Compile tasks [{dealed}/{self.CFG_COUNT}]  ============", flush=True)
                        self._waitAll()
                        procCount = 0
            self._waitAll()
            print(f"========= All Compile tasks Finished [{dealed}] ! ============", flush=True)
        self.endSignal.value = 1
        if needPerfTest:
            self.perfProcMonitor.join()
