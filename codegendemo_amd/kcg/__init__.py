"""Host-side mirror of the reference's `Runtime/python/kcg` package for the GEMM hot path.

Module and class names follow the reference so that drivers written against it (testGetKernels.py
style) read the same: Utils, Operators.matmul, KCGCompiler, CompiledKernelFactory, CompiledKernel,
KCGTask, ConfigGenerator.  Underneath, everything goes through libkcg_gemm.so (ctypes).
"""
