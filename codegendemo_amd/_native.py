"""ctypes binding of libkcg_gemm.so (C ABI: include/kcg_gemm.h).

The library is looked up next to this file.  It is never built implicitly on import: a missing
library raises, so that a GPU run cannot silently proceed without the native engine.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libkcg_gemm.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

CFG_LEN = 31
KIND_AUTO, KIND_SIMT, KIND_MFMA = 0, 1, 2
KCG_OK = 0
EPILOGUE_NONE, EPILOGUE_ALPHA_BETA = 0, 1
ERR_INVALID_CONFIG, ERR_COMPILE, ERR_IO, ERR_HIP, ERR_ARGUMENT = -1, -2, -3, -4, -5


class KcgError(RuntimeError):
    """A failure reported by libkcg_gemm.so; `.status` is the negative kcg_status."""

    def __init__(self, status, message):
        super().__init__(message)
        self.status = status


class InvalidConfigError(KcgError, ValueError):
    pass


class MatmulCfg(ctypes.Structure):
    _fields_ = [("v", ctypes.c_int32 * CFG_LEN)]


class KernelInfo(ctypes.Structure):
    _fields_ = [
        ("code_path", ctypes.c_char * 1024),
        ("kernel_name", ctypes.c_char * 512),
        ("grid", ctypes.c_int32 * 3),
        ("block", ctypes.c_int32 * 3),
        ("lds_bytes", ctypes.c_int32),
        ("kind", ctypes.c_int32),
        ("cache_hit", ctypes.c_int32),
        ("build_flags", ctypes.c_int32),
        ("scratch_bytes", ctypes.c_int32),
        ("vgprs", ctypes.c_int32),
        ("sgpr_spills", ctypes.c_int32),
    ]


# kcg_build_flag bits
BUILD_LOW_OPT, BUILD_DIAGNOSTIC, BUILD_DIRECT_DECLINED, BUILD_META_UNKNOWN = 1, 2, 4, 8
SYSTEM_HIPRTC = "/opt/rocm/lib/libhiprtc.so.7"


EXPORTS = (
    "kcg_cfg_keyword", "kcg_dtype_size", "kcg_check_config", "kcg_select_kind", "kcg_kernel_name",
    "kcg_launch_dims", "kcg_reference_lds_bytes", "kcg_block_mapping", "kcg_compile_matmul",
    "kcg_instantiation_source", "kcg_load", "kcg_launch", "kcg_benchmark", "kcg_unload",
    "kcg_device_info", "kcg_last_error", "kcg_version", "kcg_compile_matmul_ex", "kcg_launch_batched",
    "kcg_benchmark_batched", "kcg_code_object_info", "kcg_compiler_identity",
)

_lib = None


def build_library(verbose=False):
    """Compile libkcg_gemm.so in-tree with hipcc (used by __graft_entry__.build())."""
    out = subprocess.run(["make", "-B", "-C", CSRC_DIR], capture_output=True, text=True)
    if verbose or out.returncode != 0:
        print(out.stdout)
        print(out.stderr)
    if out.returncode != 0:
        raise RuntimeError("building libkcg_gemm.so failed")
    global _lib
    _lib = None
    return LIB_PATH


def _preload_process_hip_runtime():
    """A process must talk to ONE HIP runtime.  The PyTorch wheel bundles its own libamdhip64 /
    libhiprtc next to libtorch_hip.so; device buffers and streams handed to the engine come from that
    runtime, so when torch is installed its copies are loaded first and libkcg_gemm.so (which binds
    HIP lazily and prefers an already-loaded runtime) uses them.  Without torch the system ROCm is used."""
    try:
        import torch
    except ImportError:
        return None
    libdir = os.path.join(os.path.dirname(torch.__file__), "lib")
    loaded = []
    for name in ("libamdhip64.so", "libhiprtc.so"):
        p = os.path.join(libdir, name)
        if os.path.exists(p):
            ctypes.CDLL(p, mode=ctypes.RTLD_GLOBAL)
            loaded.append(p)
    return loaded


def lib():
    global _lib
    if _lib is not None:
        return _lib
    _preload_process_hip_runtime()
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` (or __graft_entry__.build()); "
            "there is no fallback path without the native library")
    L = ctypes.CDLL(LIB_PATH)
    i32p = ctypes.POINTER(ctypes.c_int32)
    u64p = ctypes.POINTER(ctypes.c_uint64)
    cfgp = ctypes.POINTER(MatmulCfg)
    L.kcg_last_error.restype = ctypes.c_char_p
    L.kcg_version.restype = ctypes.c_char_p
    L.kcg_cfg_keyword.restype = ctypes.c_char_p
    L.kcg_cfg_keyword.argtypes = [ctypes.c_int]
    L.kcg_dtype_size.argtypes = [ctypes.c_int]
    L.kcg_check_config.argtypes = [cfgp, ctypes.c_int]
    L.kcg_select_kind.argtypes = [cfgp]
    L.kcg_kernel_name.argtypes = [cfgp, ctypes.c_char_p, ctypes.c_int]
    L.kcg_launch_dims.argtypes = [cfgp, i32p, i32p]
    L.kcg_reference_lds_bytes.argtypes = [cfgp]
    L.kcg_block_mapping.argtypes = [cfgp, ctypes.c_int, ctypes.c_int, i32p, i32p]
    L.kcg_compile_matmul.argtypes = [cfgp, ctypes.c_char_p, ctypes.c_int, ctypes.POINTER(KernelInfo)]
    L.kcg_instantiation_source.argtypes = [cfgp, ctypes.c_int, ctypes.c_char_p, ctypes.c_int]
    L.kcg_load.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int, u64p, u64p, i32p, i32p]
    L.kcg_launch.argtypes = [ctypes.c_uint64, i32p, i32p, ctypes.c_int, ctypes.c_uint64,
                             ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64]
    L.kcg_benchmark.argtypes = [ctypes.c_uint64, i32p, i32p, ctypes.c_int, ctypes.c_uint64,
                                ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64,
                                ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float)]
    L.kcg_compile_matmul_ex.argtypes = [cfgp, ctypes.c_char_p, ctypes.c_int, ctypes.c_int, ctypes.POINTER(KernelInfo)]
    L.kcg_launch_batched.argtypes = [ctypes.c_uint64, i32p, i32p, ctypes.c_int, ctypes.c_uint64,
                                     ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_int32,
                                     ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_float, ctypes.c_float]
    L.kcg_benchmark_batched.argtypes = L.kcg_launch_batched.argtypes + [ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                                        ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float)]
    L.kcg_code_object_info.argtypes = [ctypes.c_char_p, ctypes.POINTER(KernelInfo)]
    L.kcg_compiler_identity.argtypes = [ctypes.c_char_p, ctypes.c_int]
    L.kcg_unload.argtypes = [ctypes.c_uint64]
    L.kcg_device_info.argtypes = [ctypes.c_int, i32p, i32p, i32p, ctypes.c_char_p, ctypes.c_int]
    _lib = L
    return L


def last_error():
    return lib().kcg_last_error().decode("utf-8", "replace")


def check(status):
    """Raise the Python exception matching a negative kcg_status."""
    if status >= 0:
        return status
    msg = last_error()
    if status == ERR_INVALID_CONFIG:
        raise InvalidConfigError(status, msg)
    raise KcgError(status, msg)


def keywords():
    L = lib()
    return [L.kcg_cfg_keyword(i).decode() for i in range(CFG_LEN)]


def make_cfg(values):
    """values: sequence of 31 ints in ABI order."""
    values = [int(v) for v in values]
    if len(values) != CFG_LEN:
        raise ValueError(f"expected {CFG_LEN} config integers, got {len(values)}")
    c = MatmulCfg()
    for i, v in enumerate(values):
        c.v[i] = v
    return c


def _dims(d):
    return (ctypes.c_int32 * 3)(*[int(x) for x in d])


def check_config(values, kind=KIND_AUTO):
    c = make_cfg(values)
    return check(lib().kcg_check_config(ctypes.byref(c), kind))


def is_valid_config(values, kind=KIND_AUTO):
    c = make_cfg(values)
    return lib().kcg_check_config(ctypes.byref(c), kind) == KCG_OK


def select_kind(values):
    c = make_cfg(values)
    return check(lib().kcg_select_kind(ctypes.byref(c)))


def kernel_name(values):
    c = make_cfg(values)
    buf = ctypes.create_string_buffer(1024)
    check(lib().kcg_kernel_name(ctypes.byref(c), buf, len(buf)))
    return buf.value.decode()


def launch_dims(values):
    c = make_cfg(values)
    g, b = _dims((0, 0, 0)), _dims((0, 0, 0))
    check(lib().kcg_launch_dims(ctypes.byref(c), g, b))
    return list(g), list(b)


def reference_lds_bytes(values):
    c = make_cfg(values)
    return lib().kcg_reference_lds_bytes(ctypes.byref(c))


def block_mapping(values, bid, xcd_remap=False):
    c = make_cfg(values)
    by, bx = ctypes.c_int32(), ctypes.c_int32()
    check(lib().kcg_block_mapping(ctypes.byref(c), bid, int(bool(xcd_remap)), ctypes.byref(by), ctypes.byref(bx)))
    return by.value, bx.value


def instantiation_source(values, kind=KIND_AUTO):
    c = make_cfg(values)
    n = check(lib().kcg_instantiation_source(ctypes.byref(c), kind, None, 0))
    buf = ctypes.create_string_buffer(n + 1)
    check(lib().kcg_instantiation_source(ctypes.byref(c), kind, buf, n + 1))
    return buf.value.decode()


def _info_dict(info):
    return {
        "code_path": info.code_path.decode(),
        "kernel_name": info.kernel_name.decode(),
        "grid": list(info.grid),
        "block": list(info.block),
        "lds_bytes": info.lds_bytes,
        "kind": info.kind,
        "cache_hit": bool(info.cache_hit),
        "build_flags": info.build_flags,
        "low_opt": bool(info.build_flags & BUILD_LOW_OPT),
        "diagnostic": bool(info.build_flags & BUILD_DIAGNOSTIC),
        "direct_declined": bool(info.build_flags & BUILD_DIRECT_DECLINED),
        "scratch_bytes": info.scratch_bytes,
        "vgprs": info.vgprs,
        "sgpr_spills": info.sgpr_spills,
    }


def compile_matmul(values, arch="gfx950", kind=KIND_AUTO, epilogue=None):
    """-> dict(code_path, kernel_name, grid, block, lds_bytes, kind, cache_hit, build_flags, low_opt, diagnostic,
    direct_declined, scratch_bytes, vgprs, sgpr_spills).
    epilogue None: the reference's three-pointer kernel; EPILOGUE_NONE / EPILOGUE_ALPHA_BETA: the
    batched-strided kernel form (launch it with launch_batched)."""
    c = make_cfg(values)
    info = KernelInfo()
    if epilogue is None:
        check(lib().kcg_compile_matmul(ctypes.byref(c), arch.encode(), kind, ctypes.byref(info)))
    else:
        check(lib().kcg_compile_matmul_ex(ctypes.byref(c), arch.encode(), kind, int(epilogue), ctypes.byref(info)))
    return _info_dict(info)


def code_object_info(code_path):
    """What the compile recorded beside a code object it wrote: dict with lds_bytes, kind, build_flags, ... (the
    fields of compile_matmul that belong to the file; kernel_name, grid and block are not among them)."""
    info = KernelInfo()
    check(lib().kcg_code_object_info(str(code_path).encode(), ctypes.byref(info)))
    d = _info_dict(info)
    for k in ("kernel_name", "grid", "block", "cache_hit"):
        d.pop(k)
    return d


def compiler_identity():
    """"hiprtc:<library path>:<size>" of the compiler the next compile uses ($KCG_HIPRTC_LIB selects another)."""
    buf = ctypes.create_string_buffer(2048)
    check(lib().kcg_compiler_identity(buf, len(buf)))
    return buf.value.decode()


class use_flags:
    """Context manager: compiles inside it get `flags` (a string) as $KCG_EXTRA_FLAGS (None or "": none)."""

    def __init__(self, flags):
        self.flags = flags

    def __enter__(self):
        self.old = os.environ.get("KCG_EXTRA_FLAGS")
        if self.flags:
            os.environ["KCG_EXTRA_FLAGS"] = self.flags
        else:
            os.environ.pop("KCG_EXTRA_FLAGS", None)
        return self

    def __exit__(self, *exc):
        if self.old is None:
            os.environ.pop("KCG_EXTRA_FLAGS", None)
        else:
            os.environ["KCG_EXTRA_FLAGS"] = self.old
        return False


class use_hiprtc:
    """Context manager: compiles inside it use the hiprtc library at `path` (None: the process's own).  The
    library reads $KCG_HIPRTC_LIB at every compile and keeps such a compiler in a link namespace of its own."""

    def __init__(self, path):
        self.path = path

    def __enter__(self):
        self.old = os.environ.get("KCG_HIPRTC_LIB")
        if self.path:
            os.environ["KCG_HIPRTC_LIB"] = self.path
        else:
            os.environ.pop("KCG_HIPRTC_LIB", None)
        return self

    def __exit__(self, *exc):
        if self.old is None:
            os.environ.pop("KCG_HIPRTC_LIB", None)
        else:
            os.environ["KCG_HIPRTC_LIB"] = self.old
        return False


def load(code_path, kernel_name_, lds_bytes, device):
    mod, fn = ctypes.c_uint64(), ctypes.c_uint64()
    regs, spills = ctypes.c_int32(), ctypes.c_int32()
    check(lib().kcg_load(code_path.encode(), kernel_name_.encode(), int(lds_bytes), int(device),
                         ctypes.byref(mod), ctypes.byref(fn), ctypes.byref(regs), ctypes.byref(spills)))
    return mod.value, fn.value, regs.value, spills.value


def launch(function, grid, block, lds_bytes, stream, a, b, c):
    check(lib().kcg_launch(function, _dims(grid), _dims(block), int(lds_bytes), int(stream), int(a), int(b), int(c)))


def launch_batched(function, grid, block, lds_bytes, stream, a, b, c, batch, stride_a, stride_b, stride_c, alpha=1.0, beta=0.0):
    check(lib().kcg_launch_batched(function, _dims(grid), _dims(block), int(lds_bytes), int(stream), int(a), int(b), int(c),
                                   int(batch), int(stride_a), int(stride_b), int(stride_c), float(alpha), float(beta)))


def benchmark(function, grid, block, lds_bytes, stream, a, b, c, warmup=1, iters=20, reps=0):
    """-> (median_ms, min_ms) per launch"""
    med, mn = ctypes.c_float(), ctypes.c_float()
    check(lib().kcg_benchmark(function, _dims(grid), _dims(block), int(lds_bytes), int(stream), int(a), int(b),
                              int(c), int(warmup), int(iters), int(reps), ctypes.byref(med), ctypes.byref(mn)))
    return med.value, mn.value


def benchmark_batched(function, grid, block, lds_bytes, stream, a, b, c, batch, stride_a, stride_b, stride_c, alpha=1.0, beta=0.0,
                      warmup=1, iters=20, reps=0):
    """-> (median_ms, min_ms) per launch of the whole batch"""
    med, mn = ctypes.c_float(), ctypes.c_float()
    check(lib().kcg_benchmark_batched(function, _dims(grid), _dims(block), int(lds_bytes), int(stream), int(a), int(b), int(c),
                                      int(batch), int(stride_a), int(stride_b), int(stride_c), float(alpha), float(beta),
                                      int(warmup), int(iters), int(reps), ctypes.byref(med), ctypes.byref(mn)))
    return med.value, mn.value


def unload(module):
    check(lib().kcg_unload(module))


def device_info(device=0):
    cu, clk, lds = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int32()
    name = ctypes.create_string_buffer(256)
    check(lib().kcg_device_info(device, ctypes.byref(cu), ctypes.byref(clk), ctypes.byref(lds), name, len(name)))
    return {"cu_count": cu.value, "clock_khz": clk.value, "lds_per_block": lds.value, "arch": name.value.decode()}
