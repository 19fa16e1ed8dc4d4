"""Kernel file descriptor and run-time handles (reference: Runtime/python/kcg/Kernel.py:44-83).

The reference's Kernel.py also carries a Triton-style `@kcg_kernel` function wrapper whose only use on
this path is to derive the pointer signature of the GEMM kernel; that signature is produced by
Operators.matmul.getMatmulSignature here."""
import hashlib
import re
from enum import IntEnum

# GEMM_MNK<M>x<N>x<K>_DTabc<a>x<b>x<c>_AT<t>_...   (kernel-name format of src/main.cc:119-145)
_NAME = re.compile(r"^GEMM_MNK(\d+)x(\d+)x(\d+)_DTabc([a-z0-9]+)x([a-z0-9]+)x([a-z0-9]+)_AT(\d)_")
_DTYPE_BYTES = {"float16": 2, "bfloat16": 2, "float32": 4, "float64": 8}


class EnumBackendType(IntEnum):
    CUDA = 1
    HIP = 2
    INVALID = 3


class KernelRuntimeInfo:
    def __init__(self, module, func, regs, spills):
        self.m_module = module
        self.m_function = func
        self.m_nRegs = regs
        self.m_nSpills = spills


def operand_bytes(kernelFuncName: str):
    """Bytes the kernel reads from A and B and writes to C, from the shape and types in its name;
    None for a name in another format."""
    m = _NAME.match(kernelFuncName)
    if not m or any(t not in _DTYPE_BYTES for t in m.group(4, 5, 6)):
        return None
    M, N, K = (int(x) for x in m.group(1, 2, 3))
    sa, sb, sc = (_DTYPE_BYTES[t] for t in m.group(4, 5, 6))
    return M * K * sa, K * N * sb, M * N * sc


class KernelLibFile:
    def __init__(self, filePath: str, backendType: EnumBackendType, kernelFuncName, sharedMemSize, signature,
                 gridDims: list, blockDims: list, device=0):
        self.m_filePath = filePath
        self.m_backendType = backendType
        self.m_kernelInfo = None            # KernelRuntimeInfo once the loader has run (per process)
        self.m_signature = signature
        self.m_kernelFuncName = kernelFuncName
        self.m_shmSize = int(sharedMemSize)
        self.m_device = int(device)
        self.m_gridDims = [int(x) for x in gridDims]
        self.m_blockDims = [int(x) for x in blockDims]

    def hash(self) -> str:
        """md5 of the code object file, first 10 hex digits (calculate_file_hash, Utils.py:240-262)."""
        with open(self.m_filePath, "rb") as f:
            return hashlib.md5(f.read()).hexdigest()[:10]

    def signature_str(self) -> str:
        return "".join(str(v) for v in self.m_signature.values())

    def __getstate__(self):                 # module / function handles belong to the process that loaded them
        st = dict(self.__dict__)
        st["m_kernelInfo"] = None
        return st
