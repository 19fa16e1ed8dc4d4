"""codegendemo_amd — MI355X (gfx950) GEMM engine behind the KCG operator API.

`codegendemo_amd.kcg` mirrors the reference's `Runtime/python/kcg` package for the GEMM hot path
(same class and function names, same JSON formats); `codegendemo_amd._native` is the ctypes binding of
`libkcg_gemm.so`, whose C ABI is declared in `include/kcg_gemm.h`.
"""
from . import _native  # noqa: F401

__all__ = ["_native", "kcg"]
