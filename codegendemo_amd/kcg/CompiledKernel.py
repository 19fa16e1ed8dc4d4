"""CompiledKernel: a loaded (lazily) and launchable GEMM kernel.

Counterpart of Runtime/python/kcg/CompiledKernel.py (:6-23) with the loader (Loader.py:64-105,
loaderCCode/hip.c:60-133) and launcher (HIPLauncher.py:264-314) folded in: the reference gcc-built a
loader extension and a per-signature launch stub at run time; here both are entry points of
libkcg_gemm.so.  Instances are picklable before their first run and load the code object in the
process that first launches them (they cross a process boundary in a .pkl, KCGTask.py:305-318).
"""
from .. import _native


def _device_address(x):
    """int, None, or anything with .data_ptr() (HIPLauncher.py:148-187)."""
    if x is None:
        return 0
    if isinstance(x, int):
        return x
    return int(x.data_ptr())


class CompiledKernel:
    def __init__(self, kernelBinaryPath: str, kernelName: str, shmSize: int, kernel_signature,
                 gridDims: list, blockDims: list, device=0):
        self.kernelBinaryPath = kernelBinaryPath
        self.kernelName = kernelName
        self.shmSize = int(shmSize)
        self.signature = kernel_signature
        self.gridDims = [int(x) for x in gridDims]
        self.blockDims = [int(x) for x in blockDims]
        self.device = int(device)
        self._module = 0
        self._function = 0
        self.n_regs = None
        self.n_spills = None

    # ---- pickling: handles are per process ----------------------------------------------------
    def __getstate__(self):
        st = dict(self.__dict__)
        st["_module"] = 0
        st["_function"] = 0
        return st

    def _ensure_loaded(self):
        if not self._function:
            self._module, self._function, self.n_regs, self.n_spills = _native.load(
                self.kernelBinaryPath, self.kernelName, self.shmSize, self.device)
        return self._function

    def _stream(self):
        import torch
        return torch.cuda.current_stream(self.device).cuda_stream

    def run(self, *args, **kwargs):
        """Launch on torch's current stream of this kernel's device with (a, b, c)."""
        if len(args) != 3:
            raise TypeError(f"GEMM kernel takes 3 device buffers (a, b, c), got {len(args)}")
        fn = self._ensure_loaded()
        a, b, c = (_device_address(x) for x in args)
        _native.launch(fn, self.gridDims, self.blockDims, self.shmSize, self._stream(), a, b, c)

    def benchmark(self, a, b, c, warmup=1, iters=20, reps=0):
        """HIP-event timing in C: (median_ms, min_ms) per launch."""
        fn = self._ensure_loaded()
        a, b, c = (_device_address(x) for x in (a, b, c))
        return _native.benchmark(fn, self.gridDims, self.blockDims, self.shmSize, self._stream(), a, b, c,
                                 warmup, iters, reps)

    def unload(self):
        if self._module:
            _native.unload(self._module)
        self._module = 0
        self._function = 0
