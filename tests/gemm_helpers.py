"""Shared helpers of the GPU parity tests: drive a config through the kcg API exactly the way the
reference's tuner does (compile -> UserInputs -> CompiledKernelFactory -> CompiledKernel.run)."""
import os

import numpy as np

from codegendemo_amd import _native
from codegendemo_amd.kcg import SeededInputs
from codegendemo_amd.kcg.CompiledKernelFactory import CompiledKernelFactory, EnumOperator, UserInputs
from codegendemo_amd.kcg.KCGCompiler import KCGCompiler
from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig

NP_OF = {2: np.float16, 4: np.float32, 8: np.float64}


def hiprtc_params():
    """The compilers the bit-exact gates run under: the hiprtc the process carries (in a Python process the ROCm
    that PyTorch bundles) and the system's (/opt/rocm: what a C program that links the library gets).  The
    direct-staging kernel counts its LDS reads by hand and hides its matrix instructions from the compiler, so its
    correctness has to be re-established per compiler; the two builds are separate cache entries."""
    import os
    import pytest
    return [pytest.param(None, id="process-hiprtc"),
            pytest.param(_native.SYSTEM_HIPRTC, id="system-hiprtc",
                         marks=pytest.mark.skipif(not os.path.exists(_native.SYSTEM_HIPRTC), reason="no system ROCm"))]


def build_kernel(config, kind=_native.KIND_AUTO, device=0, hiprtc=None, flags=None):
    """hiprtc: path of the hiprtc library that compiles (None: the process's own); flags: extra compiler options."""
    kpm = kernelArgFromConfig(config)
    comp = KCGCompiler(kind=kind)
    with _native.use_hiprtc(hiprtc), _native.use_flags(flags or os.environ.get("KCG_EXTRA_FLAGS")):
        path, name, gx, gy, gz, bx, by, bz = comp.compileKernel(kpm)[0]
    ui = UserInputs(path, name, kpm)
    ui.m_gridDims = [gx, gy, gz]
    ui.m_blockDims = [bx, by, bz]
    ui.m_ldsBytes = comp.lastInfo["lds_bytes"]
    ui.operatorKind = EnumOperator.Matmul
    return kpm, ui, CompiledKernelFactory.getKernel(ui, device), comp.lastInfo


def to_device(x, torch_dtype, device="cuda:0"):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).to(device=device, dtype=torch_dtype)


def run_gemm(config, a_mk, b_kn, kind=_native.KIND_AUTO, poison=True, hiprtc=None, flags=None):
    """a_mk: logical [M,K] fp32 numpy, b_kn: [K,N].  Returns (C as float64-free numpy in the config's
    C dtype upcast to fp32, info).  The output buffer is pre-filled with NaN so unwritten elements show."""
    import torch
    kpm, ui, kernel, info = build_kernel(config, kind, hiprtc=hiprtc, flags=flags)
    ta, tc = kpm.dtypeTorch('A'), kpm.dtypeTorch('C')
    a_dev = to_device(SeededInputs.a_operand(a_mk, kpm.isATranspose), ta)
    b_dev = to_device(b_kn, ta)
    c_dev = torch.empty((kpm.M, kpm.N), dtype=tc, device="cuda:0")
    if poison:
        # The same kernel first runs on NaN operands: LDS keeps its contents from launch to launch, so a
        # kernel that reads a staging buffer before its data has landed would otherwise find the right
        # values there whenever it (or a test with the same inputs) ran before, and pass by accident.
        kernel.run(torch.full_like(a_dev, float("nan")), torch.full_like(b_dev, float("nan")), c_dev)
        torch.cuda.synchronize()
        c_dev.fill_(float("nan"))
    kernel.run(a_dev, b_dev, c_dev)
    torch.cuda.synchronize()
    out = c_dev.to(torch.float64 if tc == torch.float64 else torch.float32).cpu().numpy()
    kernel.unload()
    return out, info


def quantize(x, dtype_code):
    """Round fp32 numpy data to the storage type of dtype_code and return it upcast to fp32
    (what the device sees)."""
    import torch
    if dtype_code == 4:
        return np.asarray(x, np.float32)
    if dtype_code == 8:
        return np.asarray(x, np.float64)
    tt = {2: torch.float16, 3: torch.bfloat16}[dtype_code]
    return torch.from_numpy(np.asarray(x, np.float32)).to(tt).to(torch.float32).numpy()


def fp32_tolerance(K, a, b):
    """max |err| <= 1e-4 * K * max|a| * max|b|."""
    return 1e-4 * K * float(np.abs(a).max()) * float(np.abs(b).max())
