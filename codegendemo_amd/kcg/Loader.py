"""HIPLoaderST: code object file -> module / function handles (reference: Runtime/python/kcg/Loader.py:64-105
and its C extension loaderCCode/hip.c:60-133, which the reference compiled with gcc at first use).
Here the loader is `kcg_load` of libkcg_gemm.so; the class keeps the reference's shape: a per-process
singleton whose loadBinary fills KernelLibFile.m_kernelInfo once."""
from .. import _native
from .Kernel import KernelLibFile, KernelRuntimeInfo


def is_hip() -> bool:
    return True


class HIPLoaderST(object):
    def __new__(cls):
        if not hasattr(cls, "instance"):
            cls.instance = super(HIPLoaderST, cls).__new__(cls)
        return cls.instance

    def __init__(self):
        _native.lib()                       # no library, no loader: fail here

    def loadBinary(self, kernelFile: KernelLibFile) -> KernelRuntimeInfo:
        if kernelFile.m_kernelInfo is None:
            mod, func, n_regs, n_spills = _native.load(kernelFile.m_filePath, kernelFile.m_kernelFuncName,
                                                       int(kernelFile.m_shmSize), int(kernelFile.m_device))
            kernelFile.m_kernelInfo = KernelRuntimeInfo(mod, func, n_regs, n_spills)
        return kernelFile.m_kernelInfo

    def unloadBinary(self, kernelFile: KernelLibFile) -> None:
        """Not in the reference (its modules are never unloaded, hip.c:86-125): a tuning sweep over
        thousands of kernels in one perf-tester process would otherwise keep every code object resident."""
        if kernelFile.m_kernelInfo is not None:
            _native.unload(kernelFile.m_kernelInfo.m_module)
            kernelFile.m_kernelInfo = None
