"""UserInputs + CompiledKernelFactory (reference: Runtime/python/kcg/CompiledKernelFactory.py:6-73)."""
from enum import Enum

from .CompiledKernel import CompiledKernel
from .Operators.matmul import KernelArgMatmul, getMatmulSignature


class EnumOperator(Enum):
    Invalid = 0
    Matmul = 1
    Convolution = 2
    Poll = 3

    def __str__(self):
        return f"{self.name}"


class UserInputs:
    def __init__(self, hsaco_path: str, kernel_func_name: str, kernelParam: KernelArgMatmul):
        """The reference builds this from (path, name, config) alone (KCGTask.py:293-296) and recomputes the LDS
        size from the config (CompiledKernelFactory.py:30-44).  That formula does not describe this engine's
        kernels (padded rows in the scalar kernel, fp32 partial sums for 16-bit split-U, static LDS in the
        direct-staging kernel), so the size is taken from what the compile recorded beside the code object:
        a file read, no compile, nothing from the environment.  A path that is not a code object of the engine
        leaves m_ldsBytes unset, and sharedMem() then says so instead of guessing."""
        self.operatorKind = EnumOperator.Matmul
        self.hsacoPath = hsaco_path
        self.kernelFuncName = kernel_func_name
        self.kernelParam = kernelParam
        self.m_gridDims = [1, 1, 1]
        self.m_blockDims = [1, 1, 1]
        self.m_ldsBytes = None      # dynamic LDS of the launch
        self.m_buildFlags = 0       # kcg_build_flag bits of the code object (_native.BUILD_*)
        self.m_scratchBytes = -1    # scratch memory per lane (register spills); -1: unknown
        from .. import _native
        try:
            rec = _native.code_object_info(hsaco_path)
        except _native.KcgError:
            rec = None
        if rec is not None:
            self.m_ldsBytes = rec["lds_bytes"]
            self.m_buildFlags = rec["build_flags"]
            self.m_scratchBytes = rec["scratch_bytes"]

    def gridDims(self):
        return self.m_gridDims

    def blockDims(self):
        return self.m_blockDims

    def sharedMem(self):
        """Dynamic LDS bytes for the launch (no side effects)."""
        if self.m_ldsBytes is None:
            raise ValueError(f"UserInputs.sharedMem(): {self.hsacoPath} has no build record beside it (it was not written "
                             "by this engine's compile); set m_ldsBytes to the kernel's dynamic LDS size")
        return int(self.m_ldsBytes)

    def numCTA(self):
        n = 1
        for d in self.gridDims():
            n *= d
        return n


class CompiledKernelFactory:
    @staticmethod
    def getKernel(info: UserInputs, deviceId: int) -> CompiledKernel:
        if info.operatorKind == EnumOperator.Matmul:
            kp = info.kernelParam
            signature = getMatmulSignature(kp.dtypeTorch('A'), kp.dtypeTorch('B'), kp.dtypeTorch('C'))
            return CompiledKernel(info.hsacoPath, info.kernelFuncName, info.sharedMem(), signature,
                                  info.gridDims(), info.blockDims(), deviceId)
        return None
