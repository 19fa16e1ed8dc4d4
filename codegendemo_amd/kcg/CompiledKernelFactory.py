"""UserInputs + CompiledKernelFactory (reference: Runtime/python/kcg/CompiledKernelFactory.py:6-73)."""
from enum import Enum

from .CompiledKernel import CompiledKernel
from .Operators.matmul import KernelArgMatmul, getMatmulSignature
from .Utils import sizeof


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
        """Dynamic LDS bytes for the launch.  The compile result knows what the chosen kernel family
        needs; without it, the reference's formula (CompiledKernelFactory.py:30-44)."""
        if self.m_ldsBytes is not None:
            return int(self.m_ldsBytes)
        kp = self.kernelParam
        sizeAB = kp.BLOCK_SIZE_M * kp.BLOCK_SIZE_K * sizeof(kp.dtype('A')) \
            + kp.BLOCK_SIZE_N * kp.BLOCK_SIZE_K * sizeof(kp.dtype('B'))
        if kp.SHARED_PREFETCH > 0:
            sizeAB *= 2
        sizeC = -1
        if kp.LOCAL_SPLIT_U > 1:
            sizeC = kp.BLOCK_SIZE_M * kp.BLOCK_SIZE_N * kp.LOCAL_SPLIT_U * sizeof(kp.dtype('A'))
        return max(sizeAB, sizeC)

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
