"""The C ABI itself: every function include/kcg_gemm.h declares is exported by libkcg_gemm.so, the
struct layouts agree, and the entry points that need a GPU fail cleanly (status + message) without one.
No compute call is made here."""
import ctypes
import os
import re

import pytest

from codegendemo_amd import _native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    with open(os.path.join(ROOT, "include", "kcg_gemm.h")) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kcg_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    names = declared_functions()
    assert len(names) >= 17
    lib = _native.lib()
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/kcg_gemm.h but not exported"
    assert set(names) == set(_native.EXPORTS)


def test_library_does_not_link_a_hip_runtime():
    """HIP is bound lazily so the process keeps a single runtime (the host program's)."""
    import subprocess
    out = subprocess.run(["readelf", "-d", _native.LIB_PATH], capture_output=True, text=True).stdout
    needed = re.findall(r"NEEDED.*\[(.*?)\]", out)
    assert not [n for n in needed if "amdhip" in n or "hiprtc" in n or "torch" in n], needed


def test_struct_layouts():
    assert ctypes.sizeof(_native.MatmulCfg) == 31 * 4
    assert ctypes.sizeof(_native.KernelInfo) == 1024 + 512 + 4 * (3 + 3 + 3 + 4)
    assert _native.lib().kcg_dtype_size(2) == 2 and _native.lib().kcg_dtype_size(3) == 2
    assert _native.lib().kcg_dtype_size(4) == 4 and _native.lib().kcg_dtype_size(8) == 8
    assert _native.lib().kcg_dtype_size(99) == 0
    assert _native.lib().kcg_cfg_keyword(31) is None and _native.lib().kcg_cfg_keyword(-1) is None


def test_error_channel_without_gpu():
    lib = _native.lib()
    # missing code object: IO error, message names the path (reference: fopen NULL -> silent NULL, hip.c:79-81)
    with pytest.raises(_native.KcgError) as ei:
        _native.load("/nonexistent/kernel.hsaco", "k", 0, 0)
    assert ei.value.status == _native.ERR_IO and "/nonexistent/kernel.hsaco" in str(ei.value)
    # null handles / null pointers
    with pytest.raises(_native.KcgError) as ei:
        _native.launch(0, [1, 1, 1], [64, 1, 1], 0, 0, 1, 2, 3)
    assert ei.value.status == _native.ERR_ARGUMENT
    assert lib.kcg_check_config(None, 0) == _native.ERR_ARGUMENT
    assert lib.kcg_compile_matmul(None, b"gfx950", 0, None) == _native.ERR_ARGUMENT
    with pytest.raises(_native.KcgError):
        _native.unload(0)
    with pytest.raises(_native.KcgError) as ei:
        _native.benchmark(1, [1, 1, 1], [64, 1, 1], 0, 0, 1, 2, 3, iters=0)
    assert ei.value.status == _native.ERR_ARGUMENT
    # unknown kernel kind
    from codegendemo_amd.kcg.ConfigGenerator import make_config
    from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig
    v = kernelArgFromConfig(make_config(256, 256, 128)).values()
    with pytest.raises(_native.KcgError) as ei:
        _native.compile_matmul(v, kind=7)
    assert ei.value.status == _native.ERR_ARGUMENT


def test_empty_grid_launch_is_a_no_op():
    """HIPLauncher.py:138: a launch with an empty grid is skipped."""
    _native.launch(1234, [0, 1, 1], [64, 1, 1], 0, 0, 1, 2, 3)


def test_last_error_is_per_thread():
    import threading
    lib = _native.lib()
    lib.kcg_check_config(None, 0)
    assert _native.last_error() != ""
    seen = {}

    def worker():
        seen["msg"] = _native.last_error()

    t = threading.Thread(target=worker)
    t.start()
    t.join()
    assert seen["msg"] == ""


def test_direct_staging_build_that_spills_falls_back_to_register_staging(tmp_path, monkeypatch):
    """The direct-staging kernel reads LDS asynchronously behind the compiler's back; a build whose
    fragments would be spilled to scratch memory must never be used.  The library notices it in the code
    object's metadata, remembers it with a marker file and builds the register-staged kernel instead."""
    from codegendemo_amd.kcg.ConfigGenerator import make_config
    from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig
    monkeypatch.setenv("KCG_CACHE_DIR", str(tmp_path))
    # 8 waves of 128x128 accumulators: 256 registers per lane cannot hold accumulators and fragments
    cfg = make_config(4096, 4096, 4096, dtype=2, dtype_c=4, BM=256, BN=512, BK=32, TM=16, TN=16, is_atrans=0,
                      shared_prefetch=1, reg_prefetch=1)
    values = kernelArgFromConfig(cfg).values()
    info = _native.compile_matmul(values, "gfx950", _native.KIND_MFMA)
    assert info["lds_bytes"] == 2 * (256 + 512) * 32 * 2 and not info["cache_hit"]     # dynamic LDS of the register-staged kernel
    assert sorted(f.rsplit(".", 1)[1] for f in os.listdir(tmp_path)) == ["buildinfo", "hsaco", "spills"]
    assert info["direct_declined"] and info["vgprs"] > 0
    assert "static constexpr bool DIRECT = false;" not in _native.instantiation_source(values, _native.KIND_MFMA)
    again = _native.compile_matmul(values, "gfx950", _native.KIND_MFMA)                 # marker + cache: nothing is compiled
    assert again["cache_hit"] and again["code_path"] == info["code_path"]
    assert again["direct_declined"] and again["vgprs"] == info["vgprs"] > 0                # the record survives the cache


def test_register_staged_build_that_spills_is_rebuilt_at_a_lower_optimisation_level(tmp_path, monkeypatch):
    """A scalar or register-staged kernel that needs scratch memory is built a second time at -O1 and that
    build is the one kept ($KCG_SPILL_REBUILD=0 keeps the first; the switch is part of the cache key).  A
    kernel without spills is built once, whatever the switch says."""
    monkeypatch.setenv("KCG_CACHE_DIR", str(tmp_path))
    # fp32 scalar kernel, one wave on a 32x32x64 tile, edge tiles everywhere: spills at -O3 (a case of the random samples)
    spilling = [32, 32, 64, 4, 4, 64, 1, 1, 8, 8, 4, 4, 4, 4, 4, 4, 1, 2, 4, 4, 1, 1, 1, 1, 4, 4, 4, 435, 401, 487, 1]
    calm = [64, 64, 16, 4, 4, 64, 2, 2, 8, 8, 4, 4, 4, 4, 4, 4, 1, 8, 4, 4, 0, 0, 0, 1, 4, 4, 4, 1024, 1024, 1024, 1]

    infos = []

    def build(values):
        info = _native.compile_matmul(values, "gfx950", _native.KIND_SIMT)
        infos.append(info)
        with open(info["code_path"], "rb") as f:
            return info["code_path"], f.read()

    p_spill, code_spill = build(spilling)
    p_calm, code_calm = build(calm)
    # the caller can see which build it got, from the compile and from the record beside the code object
    assert infos[0]["low_opt"] and infos[0]["build_flags"] & _native.BUILD_LOW_OPT and not infos[1]["low_opt"]
    assert _native.code_object_info(p_spill)["low_opt"] and not _native.code_object_info(p_calm)["low_opt"]
    assert _native.compile_matmul(spilling, "gfx950", _native.KIND_SIMT)["low_opt"]        # cache hit: still said
    monkeypatch.setenv("KCG_SPILL_REBUILD", "0")
    p_spill_first, code_spill_first = build(spilling)
    p_calm_first, code_calm_first = build(calm)
    assert p_spill != p_spill_first and p_calm != p_calm_first          # the switch is part of the cache key
    assert code_spill != code_spill_first                               # the kept build is another one
    assert code_calm == code_calm_first                                 # nothing to rebuild
    assert not infos[2]["low_opt"] and infos[2]["scratch_bytes"] > 0    # the first build kept: it spills, and says so


def test_builds_that_are_wrong_on_purpose_must_be_asked_for_twice(tmp_path, monkeypatch):
    """-DKCG_DIAG_... switches make the direct-staging kernel leave work out (to time what is left): its C is
    wrong.  $KCG_EXTRA_FLAGS alone does not get such a kernel: KCG_ALLOW_DIAG=1 must be set as well, and the
    compile result then says what it is."""
    from codegendemo_amd.kcg.ConfigGenerator import make_config
    from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig
    monkeypatch.setenv("KCG_CACHE_DIR", str(tmp_path))
    values = kernelArgFromConfig(make_config(256, 256, 256, BM=64, BN=64, BK=16, TM=4, TN=4, is_atrans=0,
                                             shared_prefetch=1, reg_prefetch=1)).values()
    plain = _native.compile_matmul(values)
    assert not plain["diagnostic"] and _native.last_error() == ""
    monkeypatch.setenv("KCG_EXTRA_FLAGS", "-DKCG_DIAG_NO_FETCH=1")
    with pytest.raises(_native.KcgError, match="KCG_ALLOW_DIAG") as ei:
        _native.compile_matmul(values)
    assert ei.value.status == _native.ERR_ARGUMENT
    monkeypatch.setenv("KCG_ALLOW_DIAG", "1")
    diag = _native.compile_matmul(values)
    assert diag["diagnostic"] and diag["code_path"] != plain["code_path"] and diag["kernel_name"] == plain["kernel_name"]
    assert _native.last_error().startswith("note: diagnostic build")
    assert _native.code_object_info(diag["code_path"])["diagnostic"]
    assert _native.compile_matmul(values)["diagnostic"]                  # from the cache: still marked
    monkeypatch.setenv("KCG_EXTRA_FLAGS", "-DKCG_TIMELINE=1")            # time stamps: C stays right, no fence
    assert not _native.compile_matmul(values)["diagnostic"]


def test_a_second_compiler_in_the_same_process(tmp_path, monkeypatch):
    """$KCG_HIPRTC_LIB selects another hiprtc, loaded in a link namespace of its own (it brings its own compiler
    library instead of sharing the one the process has loaded under the same name).  The compiler's identity is
    part of the cache key: the two builds of one config are two files."""
    system = _native.SYSTEM_HIPRTC
    if not os.path.exists(system):
        pytest.skip("no system ROCm")
    monkeypatch.setenv("KCG_CACHE_DIR", str(tmp_path))
    calm = [64, 64, 16, 4, 4, 64, 2, 2, 8, 8, 4, 4, 4, 4, 4, 4, 1, 8, 4, 4, 0, 0, 0, 1, 4, 4, 4, 1024, 1024, 1024, 1]
    own_id = _native.compiler_identity()
    own = _native.compile_matmul(calm)
    with _native.use_hiprtc(system):
        other_id = _native.compiler_identity()
        other = _native.compile_matmul(calm)
        assert not other["cache_hit"] and _native.compile_matmul(calm)["cache_hit"]
    assert os.path.realpath(system) in other_id
    assert _native.compiler_identity() == own_id
    if own_id != other_id:                      # (a process without torch uses the system's compiler by default)
        assert own["code_path"] != other["code_path"]

    def producer(path):
        with open(path, "rb") as f:
            m = re.search(rb"clang version [0-9.]+", f.read())
        return m.group(0) if m else None

    import torch
    if "torch/lib" in own_id:
        assert producer(own["code_path"]) != producer(other["code_path"])   # really two compilers
    with _native.use_hiprtc(str(tmp_path / "no_such_libhiprtc.so")):
        with pytest.raises(_native.KcgError, match="KCG_HIPRTC_LIB"):
            _native.compile_matmul(calm)


def test_launch_refuses_misaligned_operand_addresses():
    """The kernels move 16-byte vectors: an operand address that is not 16-byte aligned is refused before anything
    is launched (the check comes before the first HIP call, so it can be seen without a GPU)."""
    with pytest.raises(_native.KcgError, match="16-byte aligned"):
        _native.launch(0x1000, [1, 1, 1], [64, 1, 1], 0, 0, 0x10000, 0x20004, 0x30000)
    with pytest.raises(_native.KcgError, match="16-byte aligned"):
        _native.launch_batched(0x1000, [1, 1, 1], [64, 1, 1], 0, 0, 0x10008, 0x20000, 0x30000, 2, 64, 64, 64)
