"""CompiledKernel: a lazily loaded, launchable GEMM kernel (reference: Runtime/python/kcg/CompiledKernel.py:6-23):
a HIPLauncher around a KernelLibFile, loaded by the HIPLoaderST singleton on first use.  Instances are
picklable before and after their first run: handles stay in the process that loaded them, and the
process that unpickles loads the code object again (they cross a process boundary in a .pkl,
KCGTask.py:305-318)."""
from .HIPLauncher import HIPLauncher
from .Loader import HIPLoaderST


class CompiledKernel:
    def __init__(self, kernelBinaryPath: str, kernelName: str, shmSize: int, kernel_signature,
                 gridDims: list, blockDims: list, device=0):
        self.signature = kernel_signature
        self.device = int(device)
        self.m_loader = HIPLoaderST()
        self.m_launcher = HIPLauncher(kernelBinaryPath, kernelName, shmSize, self.signature, gridDims, blockDims, device)

    # the launcher's view, under the names the rest of the package and its users read
    kernelBinaryPath = property(lambda self: self.m_launcher.m_kernelLib.m_filePath)
    kernelName = property(lambda self: self.m_launcher.m_kernelLib.m_kernelFuncName)
    shmSize = property(lambda self: self.m_launcher.m_kernelLib.m_shmSize)
    gridDims = property(lambda self: self.m_launcher.m_kernelLib.m_gridDims)
    blockDims = property(lambda self: self.m_launcher.m_kernelLib.m_blockDims)

    def _info(self):
        return self.m_loader.loadBinary(self.m_launcher.m_kernelLib)

    n_regs = property(lambda self: self._info().m_nRegs)
    n_spills = property(lambda self: self._info().m_nSpills)

    def __getstate__(self):
        st = dict(self.__dict__)
        st.pop("m_loader", None)            # a per-process singleton
        return st

    def __setstate__(self, st):
        self.__dict__.update(st)
        self.m_loader = HIPLoaderST()

    def run(self, *args, **kwargs):
        """Launch on torch's current stream of this kernel's device with (a, b, c)."""
        if self.m_launcher is not None:
            self.m_launcher.launchKernel(self.device, *args)

    def run_batched(self, a, b, c, batch, stride_a, stride_b, stride_c, alpha=1.0, beta=0.0):
        """Launch a kernel compiled in the batched-strided form (KCGCompiler(epilogue=...)): problem z of the
        batch uses the buffers z * stride_* elements further on; alpha and beta take effect in a kernel with
        the alpha-beta epilogue."""
        self.m_launcher.launchKernelBatched(self.device, a, b, c, batch, stride_a, stride_b, stride_c, alpha, beta)

    def benchmark(self, a, b, c, warmup=1, iters=20, reps=0):
        """HIP-event timing in C: (median_ms, min_ms) per launch."""
        return self.m_launcher.benchmarkKernel(self.device, a, b, c, warmup, iters, reps)

    def benchmark_batched(self, a, b, c, batch, stride_a, stride_b, stride_c, alpha=1.0, beta=0.0, warmup=1, iters=20, reps=0):
        """HIP-event timing in C of the batched launch: (median_ms, min_ms) per batch."""
        return self.m_launcher.benchmarkKernelBatched(self.device, a, b, c, batch, stride_a, stride_b, stride_c, alpha, beta,
                                                      warmup, iters, reps)

    def unload(self):
        self.m_loader.unloadBinary(self.m_launcher.m_kernelLib)
