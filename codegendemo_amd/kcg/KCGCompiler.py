"""KCGCompiler: config -> compiled gfx950 code object.

Counterpart of Runtime/python/kcg/KCGCompiler.py (:5-45) + compile_kernel_matmul (src/main.cc:315-357):
the reference imported a CPython extension and forwarded 31 ints; this loads the C-ABI library with
ctypes and forwards the same 31 ints.  The return shape is the reference's:
[(codeObjectPath, kernelName, gridX, gridY, gridZ, blockX, blockY, blockZ)].
"""
from .. import _native
from .Operators.matmul import KernelArgMatmul


class KCGCompiler:
    def __init__(self, arch: str = "gfx950", kind: int = _native.KIND_AUTO, epilogue=None):
        """epilogue None: the reference's three-pointer kernel.  _native.EPILOGUE_NONE / EPILOGUE_ALPHA_BETA: the
        batched-strided kernel form (C_z = A_z B_z, or alpha * A_z B_z + beta * C_z), run with
        CompiledKernel.run_batched."""
        _native.lib()            # fail here, loudly, if the native library is missing
        self.arch = arch
        self.kind = kind
        self.epilogue = epilogue
        self.lastInfo = None     # full kcg_kernel_info of the last compile (lds_bytes, kind, cache_hit)

    def compile_kernel_matmul(self, *ints):
        """The raw 31-integer entry point (argument order of src/main.cc:64-96)."""
        info = _native.compile_matmul(ints, self.arch, self.kind, self.epilogue)
        self.lastInfo = info
        g, b = info["grid"], info["block"]
        return [(info["code_path"], info["kernel_name"], g[0], g[1], g[2], b[0], b[1], b[2])]

    def compileKernel(self, param: KernelArgMatmul) -> list:
        return self.compile_kernel_matmul(*param.values())
