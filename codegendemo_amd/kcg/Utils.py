"""Keywords, dtype codes, paths and small helpers shared by the kcg modules.

Mirrors Runtime/python/kcg/Utils.py of the reference for what the GEMM path uses:
ConfigKeywords (:359-390), EnumKernelDType/ToTorchType/sizeof (:198-221), get_dtype_from_int (:392-400),
DeviceInfo (:264-297), PathManager (:300-356) and the pickle helpers (:31-51).  The keyword strings are
not retyped here: they are read from the native library, which holds the single table
(include/Common/Utils.h:186-217 of the reference).
"""
import os
import pickle
from enum import IntEnum
from pathlib import Path
from typing import Dict, List  # noqa: F401  (re-exported, the reference's modules star-import them)

from .. import _native


class EnumKernelDType(IntEnum):
    float8 = 1
    float16 = 2
    bfloat16 = 3   # addition of this engine; the reference has no bf16 code
    float32 = 4
    float64 = 8
    float128 = 16
    int8 = 31
    int16 = 32
    int32 = 34
    int64 = 38

    def __str__(self):
        return f"{self.name}"


def ToTorchType(t):
    import torch
    return {
        EnumKernelDType.float16: torch.float16,
        EnumKernelDType.bfloat16: torch.bfloat16,
        EnumKernelDType.float32: torch.float32,
        EnumKernelDType.float64: torch.float64,
    }.get(EnumKernelDType(int(t)))


def ToNumpyType(t):
    import numpy as np
    return {
        EnumKernelDType.float16: np.float16,
        EnumKernelDType.float32: np.float32,
        EnumKernelDType.float64: np.float64,
    }.get(EnumKernelDType(int(t)))


def sizeof(t) -> int:
    """Bytes per element (reference: int(t) % 30, which this agrees with for every code it defines)."""
    assert t is not None
    t = int(t)
    if t == int(EnumKernelDType.bfloat16):
        return 2
    return t % 30


def get_dtype_from_int(dtype: int):
    try:
        return EnumKernelDType(int(dtype))
    except ValueError:
        return None


class _Keywords:
    """ConfigKeywords: KEY_* attributes generated from the native keyword table."""

    _attr = {
        "BLOCK_SIZE_M": "KEY_BLOCK_SIZE_M", "BLOCK_SIZE_N": "KEY_BLOCK_SIZE_N", "BLOCK_SIZE_K": "KEY_BLOCK_SIZE_K",
        "THREAD_SIZE_M": "KEY_THREAD_SIZE_M", "THREAD_SIZE_N": "KEY_THREAD_SIZE_N", "WARP_SIZE": "KEY_WARP_SIZE",
        "BLOCK_LAYOUT_M": "KEY_BLOCK_LAYOUT_M", "BLOCK_LAYOUT_N": "KEY_BLOCK_LAYOUT_N",
        "WARP_LAYOUT_M": "KEY_WARP_LAYOUT_M", "WARP_LAYOUT_N": "KEY_WARP_LAYOUT_N",
        "DATATYPE_A": "KEY_DTYPE_A", "DATATYPE_B": "KEY_DTYPE_B", "DATATYPE_C": "KEY_DTYPE_C",
        "M_SIZE": "KEY_M", "N_SIZE": "KEY_N", "K_SIZE": "KEY_K", "IS_ATRANS": "KEY_IS_A_TRANSPOSE",
    }

    def __init__(self):
        self.ORDER = tuple(_native.keywords())          # ABI order (src/main.cc:64-96)
        for kw in self.ORDER:
            setattr(self, self._attr.get(kw, "KEY_" + kw), kw)


ConfigKeywords = _Keywords()


def serialize_to_file(path, obj):
    with open(path, "wb") as f:
        pickle.dump(obj, f)


def deserialize_from_file(path):
    """A truncated or unreadable pickle yields [] (reference: Utils.py:44-51)."""
    try:
        with open(path, "rb") as f:
            return pickle.load(f)
    except (EOFError, pickle.UnpicklingError, OSError):
        return []


def delete_files_in_directory(directory):
    if not os.path.isdir(directory):
        return
    for name in os.listdir(directory):
        p = os.path.join(directory, name)
        if os.path.isfile(p):
            os.remove(p)


class DeviceInfo:
    @staticmethod
    def get_cuda_stream(idx=None):
        import torch
        if idx is None:
            idx = DeviceInfo.get_current_device()
        return torch.cuda.current_stream(idx).cuda_stream

    @staticmethod
    def get_current_device():
        import torch
        return torch.cuda.current_device()

    @staticmethod
    def set_current_device(idx):
        import torch
        torch.cuda.set_device(idx)

    @staticmethod
    def get_warp_size():
        return 64


class PathManager:
    """Working directories of a tuning run.  Root = $KCG_WORK_DIR or ./_kcg_work (the reference used
    fixed directories under its checkout: _pkls, _tmp, _cache, _override, _dump)."""

    @staticmethod
    def project_dir() -> str:
        return os.environ.get("KCG_WORK_DIR", os.path.join(os.getcwd(), "_kcg_work"))

    @staticmethod
    def pikle_dir() -> str:
        return os.path.join(PathManager.project_dir(), "_pkls")

    @staticmethod
    def tmp_dir() -> str:
        return os.path.join(PathManager.project_dir(), "_tmp")

    @staticmethod
    def default_cache_dir() -> str:
        return os.path.join(PathManager.project_dir(), "_cache")

    @staticmethod
    def default_override_dir() -> str:
        return os.path.join(PathManager.project_dir(), "_override")

    @staticmethod
    def default_dump_dir() -> str:
        return os.path.join(PathManager.project_dir(), "_dump")

    @staticmethod
    def kcg_compiler_path() -> str:
        return _native.LIB_PATH

    @staticmethod
    def init(clearPkl=False, clearDump=False, clearOverride=False, clearCache=False, clearTmp=False):
        dirs = [(PathManager.pikle_dir(), clearPkl), (PathManager.default_cache_dir(), clearCache),
                (PathManager.default_override_dir(), clearOverride), (PathManager.default_dump_dir(), clearDump),
                (PathManager.tmp_dir(), clearTmp)]
        for d, clear in dirs:
            Path(d).mkdir(parents=True, exist_ok=True)
            if clear:
                delete_files_in_directory(d)
