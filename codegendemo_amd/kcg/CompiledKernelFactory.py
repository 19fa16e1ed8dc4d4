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
        self.operatorKind = EnumOperator.Matmul
        self.hsacoPath = hsaco_path
        self.kernelFuncName = kernel_func_name
        self.kernelParam = kernelParam
        self.m_gridDims = [1, 1, 1]
        self.m_blockDims = [1, 1, 1]
        self.m_ldsBytes = None      # set from the compile result when known

    def gridDims(self):
        return self.m_gridDims

    def blockDims(self):
        return self.m_blockDims

    def sharedMem(self):
        """Dynamic LDS bytes for the launch: what the kernel inside the code object needs, as the engine
        reported it at compile time (m_ldsBytes).  A driver written for the reference builds UserInputs from
        (path, name, config) alone (KCGTask.py:293-296) and relies on the reference's formula
        (CompiledKernelFactory.py:30-44) here; that formula does not describe this engine's kernels (padded
        rows in the scalar kernel, fp32 partial sums for 16-bit split-U, static LDS in the direct-staging
        kernel), so the engine is asked instead: the compile is a cache hit that returns the figure that
        belongs to exactly this code object.  A code object the engine would not produce for this config
        (another kernel family was forced) is refused rather than launched with a guessed size."""
        if self.m_ldsBytes is not None:
            return int(self.m_ldsBytes)
        from .. import _native
        info = _native.compile_matmul(self.kernelParam.values())
        if info["code_path"] != self.hsacoPath or info["kernel_name"] != self.kernelFuncName:
            raise ValueError("UserInputs.sharedMem(): the LDS size of this code object is unknown (it is not what "
                             "the engine builds for this config by default); set m_ldsBytes from the compile result")
        self.m_ldsBytes = info["lds_bytes"]
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
