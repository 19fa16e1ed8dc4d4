"""HIPLauncher: launches a loaded GEMM kernel on torch's current stream (reference:
Runtime/python/kcg/HIPLauncher.py:264-314).  The reference generated and gcc-compiled a CPython launch
stub per kernel signature (`launch(gridX, ..., stream, function, hooks, A, B, C)`, :107-238); here the
launch is `kcg_launch` of libkcg_gemm.so.  Pointer arguments may be ints, None or objects with
.data_ptr() (:148-187)."""
from .. import _native
from .Kernel import EnumBackendType, KernelLibFile, operand_bytes
from .Loader import HIPLoaderST
from .Utils import DeviceInfo


def _device_address(x):
    if x is None:
        return 0
    if isinstance(x, int):
        return x
    return int(x.data_ptr())


class HIPLauncher:
    def __init__(self, kernelBinaryPath, kernelFuncName, shmSize, signature: dict, gridDims: list, blockDims: list,
                 device=0):
        self.m_kernelLib = KernelLibFile(kernelBinaryPath, EnumBackendType.HIP, kernelFuncName, shmSize, signature,
                                         gridDims, blockDims, device)
        self._need = operand_bytes(kernelFuncName)

    def _function(self):
        return HIPLoaderST().loadBinary(self.m_kernelLib).m_function

    def _check_operands(self, args, batch=1, strides=(0, 0, 0)):
        """A buffer smaller than what the kernel will touch would be a memory fault on the device: refuse it
        on the host.  Only objects that say how large they are (tensors) can be checked."""
        if len(args) != 3:
            raise TypeError(f"GEMM kernel takes 3 device buffers (a, b, c), got {len(args)}")
        if self._need is None:
            return
        for label, x, need, stride in zip("abc", args, self._need, strides):
            if hasattr(x, "numel") and hasattr(x, "element_size"):
                have = int(x.numel()) * int(x.element_size())
                need = need + (int(batch) - 1) * int(stride) * int(x.element_size())
                if have < need:
                    raise ValueError(f"operand {label}: {have} bytes, but {self.m_kernelLib.m_kernelFuncName[:60]}... "
                                     f"accesses {need} bytes")
                if hasattr(x, "is_contiguous") and not x.is_contiguous():
                    raise ValueError(f"operand {label} must be contiguous")

    @staticmethod
    def _check_strides(args, batch, strides):
        """Every problem's buffers must be as aligned as the first one's: the kernels move 16-byte vectors
        (kcg_launch_batched refuses such strides too; here the message names the operand)."""
        for label, x, stride in zip("abc", args, strides):
            if batch > 1 and hasattr(x, "element_size") and (int(stride) * int(x.element_size())) % 16:
                raise ValueError(f"stride_{label} = {stride} elements is not a multiple of 16 bytes")

    def launchKernel(self, devId: int, *args):
        if self.m_kernelLib.m_kernelFuncName.endswith(("EX_", "EXab_")):
            raise TypeError("a kernel in the batched-strided form takes strides, alpha and beta: use run_batched")
        self._check_operands(args)
        fn = self._function()
        a, b, c = (_device_address(x) for x in args)
        _native.launch(fn, self.m_kernelLib.m_gridDims, self.m_kernelLib.m_blockDims, self.m_kernelLib.m_shmSize,
                       DeviceInfo.get_cuda_stream(devId), a, b, c)

    def launchKernelBatched(self, devId: int, a, b, c, batch, stride_a, stride_b, stride_c, alpha=1.0, beta=0.0):
        if not self.m_kernelLib.m_kernelFuncName.endswith(("EX_", "EXab_")):
            raise TypeError("this kernel was not compiled in the batched-strided form (KCGCompiler(epilogue=...))")
        if batch > 0:
            self._check_operands((a, b, c), batch, (stride_a, stride_b, stride_c))
            self._check_strides((a, b, c), batch, (stride_a, stride_b, stride_c))
        fn = self._function()
        a, b, c = (_device_address(x) for x in (a, b, c))
        _native.launch_batched(fn, self.m_kernelLib.m_gridDims, self.m_kernelLib.m_blockDims, self.m_kernelLib.m_shmSize,
                               DeviceInfo.get_cuda_stream(devId), a, b, c, batch, stride_a, stride_b, stride_c, alpha, beta)

    def benchmarkKernel(self, devId: int, a, b, c, warmup=1, iters=20, reps=0):
        """The timing loop of PerfTester in C (kcg_benchmark): (median_ms, min_ms) per launch."""
        self._check_operands((a, b, c))
        fn = self._function()
        a, b, c = (_device_address(x) for x in (a, b, c))
        return _native.benchmark(fn, self.m_kernelLib.m_gridDims, self.m_kernelLib.m_blockDims, self.m_kernelLib.m_shmSize,
                                 DeviceInfo.get_cuda_stream(devId), a, b, c, warmup, iters, reps)

    def benchmarkKernelBatched(self, devId: int, a, b, c, batch, stride_a, stride_b, stride_c, alpha=1.0, beta=0.0,
                               warmup=1, iters=20, reps=0):
        """The same timing loop around the batched launch (kcg_benchmark_batched): (median_ms, min_ms) per batch."""
        if not self.m_kernelLib.m_kernelFuncName.endswith(("EX_", "EXab_")):
            raise TypeError("this kernel was not compiled in the batched-strided form (KCGCompiler(epilogue=...))")
        self._check_operands((a, b, c), batch, (stride_a, stride_b, stride_c))
        self._check_strides((a, b, c), batch, (stride_a, stride_b, stride_c))
        fn = self._function()
        a, b, c = (_device_address(x) for x in (a, b, c))
        return _native.benchmark_batched(fn, self.m_kernelLib.m_gridDims, self.m_kernelLib.m_blockDims, self.m_kernelLib.m_shmSize,
                                         DeviceInfo.get_cuda_stream(devId), a, b, c, batch, stride_a, stride_b, stride_c,
                                         alpha, beta, warmup, iters, reps)
