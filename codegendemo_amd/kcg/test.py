"""Single-config check: compile one tuning config, run it once on the GPU, compare with the library
GEMM and print the speed-up.  Counterpart of Runtime/python/kcg/test.py (cases :19-107, the check
:135-231): same steps (KCGCompiler.compileKernel -> UserInputs -> CompiledKernelFactory.getKernel ->
run(a or a^T, b, c) -> torch.matmul -> allclose(atol=rtol=1e-2, test.py:223)), same printed fields.
Differences: inputs are seeded, the config can also come from a JSON file, and the result is the
exit status.

    python -m codegendemo_amd.kcg.test [case_normal_0 | case_normal_1 | case_bad_0]
    python -m codegendemo_amd.kcg.test --config TunedConfigs/gemm_4096_fp16.json --index 0 [--count 20]
"""
import argparse
import json
import sys

import numpy as np

from .._native import InvalidConfigError
from .CompiledKernelFactory import CompiledKernelFactory, EnumOperator, UserInputs
from .KCGCompiler import KCGCompiler
from .Operators.matmul import KernelArgMatmul, kernelArgFromConfig
from .Utils import EnumKernelDType

# The reference's hand-written cases (test.py:19-107) as data: the fields each case sets on a
# KernelArgMatmul(1024, 1024, 1024, float32 x3).
CASES = {
    # 64x48x32 tile, 4x6 thread tile, split-U 2, 64-bit vectors, N = 1056 (22 block columns)
    "case_normal_0": dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=48, BLOCK_SIZE_K=32, THREAD_SIZE_M=4, THREAD_SIZE_N=6,
                          GLOB_LOAD_WIDTH_A=2, GLOB_LOAD_WIDTH_B=2, BLOCK_LAYOUT_M=2, BLOCK_LAYOUT_N=1,
                          WARP_LAYOUT_M=8, WARP_LAYOUT_N=8, WARP_SCATTER_WIDTH_A=2, WARP_SCATTER_WIDTH_B=2,
                          THREAD_SCATTER_WIDTH_A=2, THREAD_SCATTER_WIDTH_B=2, LOCAL_SPLIT_U=2, BLOCK_MAPPING=8,
                          WARP_SIZE=64, GLOB_STORE_WIDTH=2, isATranspose=1, M=1024, N=1056, K=1024),
    # 64x64x32 tile, 4x4 thread tile, 4x16 lanes
    "case_normal_1": dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=32, THREAD_SIZE_M=4, THREAD_SIZE_N=4,
                          GLOB_LOAD_WIDTH_A=4, GLOB_LOAD_WIDTH_B=4, BLOCK_LAYOUT_M=4, BLOCK_LAYOUT_N=1,
                          WARP_LAYOUT_M=4, WARP_LAYOUT_N=16, WARP_SCATTER_WIDTH_A=2, WARP_SCATTER_WIDTH_B=2,
                          THREAD_SCATTER_WIDTH_A=2, THREAD_SCATTER_WIDTH_B=2, LOCAL_SPLIT_U=1, BLOCK_MAPPING=8,
                          WARP_SIZE=64, GLOB_STORE_WIDTH=4, isATranspose=1, M=1024, N=1024, K=1024),
    # the shape of a Tensile kernel (MT256x32x8); as in the reference it sets tile sizes only, and the
    # layout it leaves behind does not multiply out to the tile: check() must reject it
    "case_bad_0": dict(BLOCK_SIZE_M=256, BLOCK_SIZE_N=32, BLOCK_SIZE_K=8, THREAD_SIZE_M=8, THREAD_SIZE_N=4,
                       BLOCK_LAYOUT_M=2, BLOCK_LAYOUT_N=2, WARP_LAYOUT_M=16, WARP_LAYOUT_N=4, WARP_SIZE=64,
                       isATranspose=0),
}


def make_case(name: str) -> KernelArgMatmul:
    kpm = KernelArgMatmul(1024, 1024, 1024, EnumKernelDType.float32, EnumKernelDType.float32, EnumKernelDType.float32)
    for field, value in CASES[name].items():
        setattr(kpm, field, value)
    return kpm


def compare_with_error(tensor1, tensor2, abs_error=1e-2, rel_error=1e-2):
    """(number of elements off by more than abs_error AND more than rel_error relative, largest
    absolute difference) -- test.py:124-133."""
    import torch
    abs_diff = torch.abs(tensor1 - tensor2)
    rel_diff = abs_diff / (torch.abs(tensor1) + 1e-5)
    diff_elements = int(torch.sum((abs_diff > abs_error) & (rel_diff > rel_error)).item())
    return diff_elements, float(abs_diff.max().item())


def test_correctness(kpm: KernelArgMatmul, deviceId: int = 0, benchmarkCount: int = 1, seed: int = 0x4B4347) -> bool:
    import torch
    kernelCompiler = KCGCompiler()
    hsacoPath, kernelName, gridDimX, gridDimY, gridDimZ, blockDimX, blockDimY, blockDimZ = kernelCompiler.compileKernel(kpm)[0]
    print("===== test info ========")
    for label, value in (("hsacoPath", hsacoPath), ("kernelName", kernelName), ("gridDimX", gridDimX),
                         ("gridDimY", gridDimY), ("gridDimZ", gridDimZ), ("blockDimX", blockDimX),
                         ("blockDimY", blockDimY), ("blockDimZ", blockDimZ)):
        print(label, "= ", value)
    inConfig = UserInputs(hsacoPath, kernelName, kpm)
    inConfig.m_gridDims = [gridDimX, gridDimY, gridDimZ]
    inConfig.m_blockDims = [blockDimX, blockDimY, blockDimZ]
    inConfig.m_ldsBytes = kernelCompiler.lastInfo["lds_bytes"]
    inConfig.operatorKind = EnumOperator.Matmul
    packedKernel = CompiledKernelFactory.getKernel(inConfig, deviceId)

    dev = f"cuda:{deviceId}"
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    ta, tc = kpm.dtypeTorch('A'), kpm.dtypeTorch('C')
    a = torch.randn(kpm.M, kpm.K, dtype=torch.float32, device=dev, generator=gen).to(ta)
    b = torch.randn(kpm.K, kpm.N, dtype=torch.float32, device=dev, generator=gen).to(ta)
    c = torch.empty(kpm.M, kpm.N, dtype=tc, device=dev)
    atrans = torch.transpose(a, 1, 0).contiguous()      # the kernel wants dense storage (test.py:168)
    print(f"python: M,N,K = {kpm.M},{kpm.N},{kpm.K}")
    print('transpose test' if kpm.isATranspose else 'normal test')
    first = atrans if kpm.isATranspose else a
    start_event = torch.cuda.Event(enable_timing=True)
    end_event = torch.cuda.Event(enable_timing=True)
    res, res1 = [], []
    for _ in range(benchmarkCount):
        start_event.record()
        packedKernel.run(first, b, c)
        end_event.record()
        torch.cuda.synchronize()
        res.append(start_event.elapsed_time(end_event))
    print(f"codegenDemo median time: {np.median(res)} ms")
    d = None
    for _ in range(benchmarkCount):
        start_event.record()
        d = torch.matmul(a, b)
        end_event.record()
        torch.cuda.synchronize()
        res1.append(start_event.elapsed_time(end_event))
    print(f"rocblas median time: {np.median(res1)} ms")
    print(f"speed up: {np.median(res1) / np.median(res)}")
    print("c=", c)
    print("d=", d)
    c32, d32 = c.to(torch.float32), d.to(torch.float32)
    ok = bool(torch.allclose(c32, d32, atol=1e-2, rtol=1e-2))
    if ok:
        print('test correct!')
    else:
        diff, max_error = compare_with_error(d32, c32)
        mn = kpm.M * kpm.N
        print(f'test fail! maxerror={max_error}, diff=[{diff} / {mn}], diffrate={diff / mn}')
    packedKernel.unload()
    return ok


def main(argv=None):
    ap = argparse.ArgumentParser(description="single-config check against the library GEMM")
    ap.add_argument("case", nargs="?", default="case_normal_0", choices=sorted(CASES))
    ap.add_argument("--config", help="JSON file: {\"cfgs\": [...]}, {\"results\": [{\"config\": ...}]} or one flat config")
    ap.add_argument("--index", type=int, default=0)
    ap.add_argument("--count", type=int, default=1, help="timed runs of each side (the reference uses 1)")
    ap.add_argument("--device", type=int, default=0)
    args = ap.parse_args(argv)
    if args.config:
        with open(args.config) as f:
            obj = json.load(f)
        entries = obj.get("cfgs") or obj.get("results") or [obj]
        cfg = entries[args.index]
        kpm = kernelArgFromConfig(cfg.get("config", cfg))
    else:
        kpm = make_case(args.case)
    try:
        kpm.check()                                      # test.py:230: an invalid config stops here
    except InvalidConfigError as e:
        print(e)
        return 2
    return 0 if test_correctness(kpm, args.device, args.count) else 1


if __name__ == "__main__":
    sys.exit(main())
