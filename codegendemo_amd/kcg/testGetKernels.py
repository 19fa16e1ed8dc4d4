"""Command-line driver of a tuning run (counterpart of Runtime/python/kcg/testGetKernels.py:1-69).

    python -m codegendemo_amd.kcg.testGetKernels <tuning_param_file> <cacheTuningSpaceFile> <onlyGenerateCfg> <splitBigJson>
           [--perf-out PATH] [--grid] [--max-process N] [--top K] [--device D]

The four positional arguments are the reference's (testGetKernels.py:31-35).  --grid keeps one layout
per (BM, BN, BK, TM, TN, prefetch) grid point instead of every valid layout.  Needs a GPU unless
onlyGenerateCfg >= 1.
"""
import argparse
import json
import os
import sys

from .ConfigGenerator import config_gen, read_params, save_to_json, sweep_grid_points
from .KCGTask import ParallelTaskManager
from .Utils import PathManager


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("tuning_param_file")
    ap.add_argument("cacheTuningSPaceFile")
    ap.add_argument("onlyGenerateCfg", type=int)
    ap.add_argument("splitBigJson", type=int)
    ap.add_argument("--perf-out", default="perfRecordlog")
    ap.add_argument("--grid", action="store_true")
    ap.add_argument("--max-process", type=int, default=8)
    ap.add_argument("--top", type=int, default=15)
    ap.add_argument("--device", type=int, default=0)
    ap.add_argument("--benchmark-count", type=int, default=20)
    args = ap.parse_args(argv)

    PathManager.init(clearPkl=True, clearTmp=True, clearCache=True)
    pre = ""
    if args.grid:
        cfgs, skipped = sweep_grid_points(read_params(args.tuning_param_file))
        pre = args.cacheTuningSPaceFile
        save_to_json({"cfgs": cfgs}, pre)
        print(f"grid: {len(cfgs)} configs, {len(skipped)} grid points skipped (no feasible layout)")
        for s in skipped:
            print("  skipped:", json.dumps(s))
    nProcess = args.max_process
    names, total = config_gen(args.tuning_param_file, preGeneratedJson=pre, singleLength=nProcess * 5,
                              cacheTuningSPaceFile="" if pre else args.cacheTuningSPaceFile,
                              splitBigJson=bool(args.splitBigJson) or True)
    print(f"==== config_gen Done: {total} configs in {len(names)} sub-JSONs ====")
    if args.onlyGenerateCfg >= 1:
        return 0
    tm = ParallelTaskManager(total, names, args.perf_out, benchmarkcnt=args.benchmark_count, warmupcnt=1,
                             devId=args.device, keepTopNum=args.top, torchDynamicLogPath="", nTorchEpsInitTest=20)
    tm.run(maxProcess=nProcess, startFromSubjson="", needCompile=True, needPerfTest=True)
    out = f"{args.perf_out}_0.json"
    if os.path.exists(out):
        with open(out) as f:
            best = json.load(f)["results"]
        print(f"==== best of {total}: {best[0]['tflops']:.1f} TFLOPS, speed-up {best[0]['acc']:.3f} over the library GEMM ====")
    return 0


if __name__ == "__main__":
    sys.exit(main())
