"""The Python operator API mirrors the reference's kcg package: same records, same JSON, same call
shapes (CPU only)."""
import json
import os
import pickle

import numpy as np
import pytest

from codegendemo_amd import _native
from codegendemo_amd.kcg import SeededInputs as SI
from codegendemo_amd.kcg.CompiledKernelFactory import CompiledKernelFactory, EnumOperator, UserInputs
from codegendemo_amd.kcg.ConfigGenerator import config_gen, get_cfgs, iter_cfgs, make_config
from codegendemo_amd.kcg.KCGCompiler import KCGCompiler
from codegendemo_amd.kcg.Operators.matmul import (KernelArgMatmul, TuningSpaceChecker_Matmul, getMatmulSignature,
                                                  kernelArgFromConfig)
from codegendemo_amd.kcg.Utils import ConfigKeywords, EnumKernelDType, PathManager, ToTorchType, sizeof
from tests import fixtures


def test_enum_codes_and_sizes():
    """Utils.py:198-221 / Utils.h:110-120: float16=2, float32=4, float64=8; sizeof = code % 30."""
    assert int(EnumKernelDType.float16) == 2 and int(EnumKernelDType.float32) == 4 and int(EnumKernelDType.float64) == 8
    assert sizeof(EnumKernelDType.float32) == 4 and sizeof(EnumKernelDType.float16) == 2
    assert sizeof(EnumKernelDType.int32) == 4 and sizeof(EnumKernelDType.bfloat16) == 2
    import torch
    assert ToTorchType(EnumKernelDType.float16) is torch.float16
    assert ToTorchType(4) is torch.float32 and ToTorchType(3) is torch.bfloat16


def test_kernel_arg_defaults_follow_the_reference_constructor():
    """matmul.py:77-108."""
    k = KernelArgMatmul(1024, 512, 256, EnumKernelDType.float32, EnumKernelDType.float32, EnumKernelDType.float32)
    assert (k.BLOCK_SIZE_M, k.BLOCK_SIZE_N, k.BLOCK_SIZE_K, k.THREAD_SIZE_M, k.THREAD_SIZE_N) == (64, 64, 16, 4, 4)
    assert (k.WARP_SIZE, k.BLOCK_LAYOUT_M, k.BLOCK_LAYOUT_N, k.WARP_LAYOUT_M, k.WARP_LAYOUT_N) == (64, 4, 1, 16, 4)
    assert (k.M, k.N, k.K, k.isATranspose, k.UNROLL_NUM) == (1024, 512, 256, 1, 1)
    assert k.GLOB_LOAD_WIDTH_A == 0 and k.LOCAL_SPLIT_U == 0 and k.SHARED_PREFETCH == 0
    assert k.dtype('A') == 4 and k.dtypeTorch('C') is ToTorchType(4)


def test_json_round_trip_over_reference_configs():
    for cfg in fixtures.best_combs_1024()[::9]:
        k = kernelArgFromConfig(cfg)
        j = k.jsonfy()
        assert j == cfg
        assert list(j.keys()) == list(cfg.keys())      # same key order as the reference writes
        k2 = KernelArgMatmul(0, 0, 0, 1, 1, 1)
        k2.assignWithJson(json.loads(json.dumps(j)))
        assert k2 == k and k2.values() == k.values()
        json.loads(str(k))                              # __str__ is JSON text like the reference's


def test_values_are_in_abi_order():
    cfg = fixtures.best_combs_1024()[3]
    k = kernelArgFromConfig(cfg)
    assert k.values() == [cfg[kw] for kw in _native.keywords()]


def test_check_raises_with_reason():
    k = kernelArgFromConfig(make_config(1024, 1024, 1024))
    k.check()
    k.WARP_LAYOUT_N = 4
    with pytest.raises(ValueError):
        k.check()


def test_signature():
    import torch
    assert getMatmulSignature(torch.float32, torch.float32, torch.float32) == {0: "*fp32", 1: "*fp32", 2: "*fp32"}
    assert getMatmulSignature(torch.float16, torch.float16, torch.float32) == {0: "*fp16", 1: "*fp16", 2: "*fp32"}


def test_compiler_return_shape_and_factory(tmp_path, monkeypatch):
    """compile_kernel_matmul returns [(path, name, gx, gy, gz, bx, by, bz)] (src/main.cc:335-348)."""
    monkeypatch.setenv("KCG_CACHE_DIR", str(tmp_path / "c"))
    kpm = kernelArgFromConfig(make_config(1024, 1024, 1024, shared_prefetch=1))
    res = KCGCompiler().compileKernel(kpm)
    assert isinstance(res, list) and len(res) == 1 and len(res[0]) == 8
    path, name, gx, gy, gz, bx, by, bz = res[0]
    assert os.path.isfile(path) and name.startswith("GEMM_MNK1024x1024x1024_DTabcfloat32xfloat32xfloat32_AT1_")
    assert (gx, gy, gz, bx, by, bz) == (256, 1, 1, 256, 1, 1)
    assert KCGCompiler().compile_kernel_matmul(*kpm.values()) == res
    ui = UserInputs(path, name, kpm)
    # a reference-style driver never sets m_ldsBytes (KCGTask.py:293-296): it comes from the record the compile
    # left beside the code object, not from the reference's formula, and reading it compiles nothing
    comp = KCGCompiler()
    comp.compileKernel(kpm)
    assert ui.m_ldsBytes == ui.sharedMem() == comp.lastInfo["lds_bytes"] == 2 * (64 + 64) * 16 * 4
    assert ui.m_buildFlags == 0 and ui.m_scratchBytes == 0
    # where formula and kernel disagree (row padding of the scalar kernel for A[M,K]) the engine's figure wins, also
    # for a kernel family that was forced: the record belongs to the file, not to the config
    kpm0 = kernelArgFromConfig(make_config(1024, 1024, 1024, shared_prefetch=1, is_atrans=0))
    comp.kind = 1
    p0, n0 = comp.compileKernel(kpm0)[0][:2]
    forced_lds = comp.lastInfo["lds_bytes"]
    comp.kind = 0
    p1, n1 = comp.compileKernel(kpm0)[0][:2]
    assert p0 != p1 and forced_lds != comp.lastInfo["lds_bytes"]
    assert UserInputs(p0, n0, kpm0).sharedMem() == forced_lds
    assert UserInputs(p1, n1, kpm0).sharedMem() == comp.lastInfo["lds_bytes"]
    # a code object the engine did not write: the size is unknown and sharedMem() says so (no guess, no compile)
    alien = tmp_path / "alien.hsaco"
    alien.write_bytes(b"x")
    stranger = UserInputs(str(alien), n0, kpm0)
    assert stranger.m_ldsBytes is None
    with pytest.raises(ValueError):
        stranger.sharedMem()
    stranger.m_ldsBytes = 4096
    assert stranger.sharedMem() == 4096
    ui.m_gridDims, ui.m_blockDims = [gx, gy, gz], [bx, by, bz]
    assert ui.numCTA() == 256 and ui.operatorKind == EnumOperator.Matmul
    kernel = CompiledKernelFactory.getKernel(ui, 0)
    assert kernel.signature == {0: "*fp32", 1: "*fp32", 2: "*fp32"}
    # picklable before first run, handles never travel (KCGTask.py:305-318)
    from codegendemo_amd.kcg.Kernel import EnumBackendType, KernelRuntimeInfo
    from codegendemo_amd.kcg.Loader import HIPLoaderST
    lib = kernel.m_launcher.m_kernelLib                     # KernelLibFile (Kernel.py:52-71)
    assert lib.m_backendType == EnumBackendType.HIP and lib.m_shmSize == ui.sharedMem() and lib.m_device == 0
    assert lib.signature_str() == "*fp32*fp32*fp32" and len(lib.hash()) == 10
    assert kernel.m_loader is HIPLoaderST() and HIPLoaderST() is HIPLoaderST()      # per-process singleton
    lib.m_kernelInfo = KernelRuntimeInfo(11, 22, 0, 0)
    k2 = pickle.loads(pickle.dumps((kpm, ui, kernel)))[2]
    assert k2.m_launcher.m_kernelLib.m_kernelInfo is None and k2.m_loader is HIPLoaderST()
    assert k2.kernelBinaryPath == path and k2.gridDims == [256, 1, 1] and k2.kernelName == name
    lib.m_kernelInfo = None
    with pytest.raises(TypeError):
        k2.run(1, 2)


def test_launcher_refuses_operands_smaller_than_the_kernel_accesses(tmp_path, monkeypatch):
    """The kernel name carries M, N, K and the element types: a tensor with fewer bytes than the kernel
    will touch is refused on the host (on the device it would be a memory fault)."""
    import torch
    from codegendemo_amd.kcg.HIPLauncher import HIPLauncher
    from codegendemo_amd.kcg.Kernel import operand_bytes
    name = _native.kernel_name(kernelArgFromConfig(make_config(512, 256, 128, dtype=2, dtype_c=4)).values())
    assert operand_bytes(name) == (512 * 128 * 2, 128 * 256 * 2, 512 * 256 * 4)
    assert operand_bytes("some_other_kernel") is None
    launcher = HIPLauncher(str(tmp_path / "missing.hsaco"), name, 0, {}, [8, 1, 1], [256, 1, 1], 0)
    a = torch.zeros(512, 128, dtype=torch.float16)
    b = torch.zeros(128, 256, dtype=torch.float16)
    with pytest.raises(ValueError, match="operand c: .* accesses 524288 bytes"):
        launcher.launchKernel(0, a, b, torch.zeros(512, 256, dtype=torch.float16))
    with pytest.raises(ValueError, match="operand a must be contiguous"):
        launcher.launchKernel(0, torch.zeros(128, 512, dtype=torch.float16).t(), b, torch.zeros(512, 256))
    with pytest.raises(_native.KcgError):                   # sizes fine: it gets as far as the (missing) code object
        launcher.launchKernel(0, a, b, torch.zeros(512, 256))


def test_tuning_space_checkers():
    chk = TuningSpaceChecker_Matmul
    good = make_config(1024, 1024, 1024)
    assert chk.check_warp(dict(good)) and chk.check_size(dict(good)) and chk.check_shm_size(dict(good))
    assert not chk.check_warp(dict(good, WARP_LAYOUT_M=4))
    assert not chk.check_size(dict(good, BLOCK_LAYOUT_M=1))
    assert not chk.check_size(dict(good, WARP_SCATTER_WIDTH_A=1, THREAD_SCATTER_WIDTH_A=2))
    assert chk.check_size(dict(good, K_SIZE=1000))                               # edge tiles are allowed here …
    assert not chk.check_size(dict(good, K_SIZE=1000), allow_edge_tiles=False)   # … the reference rule rejects them
    big = make_config(4096, 4096, 4096, BM=256, BN=256, BK=64, TM=8, TN=8, dtype=2, dtype_c=4, shared_prefetch=1)
    assert chk.check_shm_size(dict(big))                                         # 128 KiB fits gfx950's 160 KiB
    assert not chk.check_shm_size(dict(big, BLOCK_SIZE_K=128))
    # DATATYPE_C alone is expanded to A/B (matmul.py:259-263)
    c = {k: v for k, v in good.items() if k not in ("DATATYPE_A", "DATATYPE_B")}
    assert chk.check_shm_size(c) and c["DATATYPE_A"] == 4 and c["DATATYPE_B"] == 4


def test_get_cfgs_on_reference_tuning_space():
    """GEMM_single_test.json describes one point; GEMM_configs_1024.json a large space whose every
    emitted point must pass the engine predicate."""
    spaces = fixtures.tuning_spaces()
    single = list(iter_cfgs(spaces["GEMM_single_test.json"]))
    assert len(single) == 1 and single[0]["BLOCK_SIZE_N"] == 64 and single[0]["WARP_LAYOUT_N"] == 16
    space = dict(spaces["GEMM_configs_1024.json"])
    for k in ("UNROLL_NUM", "BLOCK_MAPPING", "GLOB_STORE_WIDTH", "REDUCE_C_CONTINUOUS", "LOAD_CONTINUOUS",
              "WARP_SCATTER_WIDTH_A", "WARP_SCATTER_WIDTH_B", "THREAD_SCATTER_WIDTH_A", "THREAD_SCATTER_WIDTH_B"):
        space[k] = space[k][:1]      # keep the enumeration small for a unit test
    stats = {}
    cfgs = list(iter_cfgs(space, stats=stats))
    assert 0 < len(cfgs) < stats["enumerated"]
    for c in cfgs[::17]:
        assert _native.is_valid_config([c[k] for k in ConfigKeywords.ORDER])


def test_config_gen_splits_into_sub_jsons(tmp_path, monkeypatch):
    monkeypatch.setenv("KCG_WORK_DIR", str(tmp_path / "work"))
    PathManager.init(clearTmp=True)
    space = {k: [v] for k, v in make_config(2048, 2048, 2048).items()}
    space["BLOCK_SIZE_K"] = [8, 16, 32]
    space["SHARED_PREFETCH"] = [0, 1]
    tuning = tmp_path / "space.json"
    tuning.write_text(json.dumps(space))
    cache = tmp_path / "combs.json"
    names, total = config_gen(str(tuning), "", 4, str(cache), splitBigJson=True)
    assert total == 6 and len(names) == 2
    assert [len(json.load(open(n))["cfgs"]) for n in names] == [4, 2]
    assert len(json.load(open(cache))["cfgs"]) == 6
    names2, total2 = config_gen("", str(cache), 6, "", splitBigJson=True)      # reuse the pre-generated file
    assert total2 == 6 and len(names2) == 1
    assert get_cfgs(str(tuning))[0]["M_SIZE"] == 2048


def test_seeded_inputs_are_deterministic_and_well_formed():
    u1 = SI.uniform((64, 48), SI.STREAM_A)
    u2 = SI.uniform((64, 48), SI.STREAM_A)
    assert np.array_equal(u1, u2) and u1.dtype == np.float32
    assert not np.array_equal(u1, SI.uniform((64, 48), SI.STREAM_B))
    assert u1.min() >= -1.0 and u1.max() < 1.0
    assert np.array_equal(SI.uniform((4096,), 1)[:100], SI.uniform((100,), 1))      # counter-based: prefix-stable
    # fixture: integer-exact stream, must never change across machines or numpy versions
    assert SI.checksum(SI.uniform((1024, 1024), SI.STREAM_A)) == SI.checksum(SI.uniform((1024 * 1024,), SI.STREAM_A))
    big = SI.uniform((1 << 20,), 7)
    assert abs(float(big.mean())) < 5e-3 and abs(float(big.var()) - 1.0 / 3.0) < 5e-3
    n = SI.normal((1 << 20,), 8, std=0.5)
    assert abs(float(n.mean())) < 5e-3 and abs(float(n.std()) - 0.5) < 5e-3
    s = SI.small_ints((1000,), 9, lim=4)
    assert set(np.unique(s)).issubset(set(np.arange(-4, 5, dtype=np.float32))) and len(np.unique(s)) == 9
    a = SI.uniform((5, 7), 3)
    assert SI.a_operand(a, 1).shape == (7, 5) and np.array_equal(SI.a_operand(a, 1), a.T)


def test_uniform_stream_golden_values():
    """First values of stream A, committed so the generator cannot drift silently."""
    got = SI.raw_bits(4, SI.STREAM_A).tolist()
    with open(os.path.join(fixtures.GOLDEN, "seeded_inputs.json")) as f:
        want = json.load(f)
    assert got == want["raw_bits_stream1_first4"]
    assert SI.checksum(SI.uniform((256, 256), SI.STREAM_A)) == want["checksum_uniform_256x256_stream1"]
    assert SI.checksum(SI.uniform((256, 256), SI.STREAM_B)) == want["checksum_uniform_256x256_stream2"]


def test_single_config_check_cases(capsys):
    """The hand-written cases of the reference's test.py (:19-107): the two normal ones are valid configs
    with the launch geometry its comments state; the 'bad' one is refused before anything is compiled."""
    from codegendemo_amd.kcg import test as single
    k0 = single.make_case("case_normal_0")
    k0.check()
    assert (k0.M, k0.N, k0.K, k0.LOCAL_SPLIT_U, k0.isATranspose) == (1024, 1056, 1024, 2, 1)
    grid, block = _native.launch_dims(k0.values())
    assert grid[0] == 16 * 22 and block[0] == 256            # matmul.cpp:2448-2449
    single.make_case("case_normal_1").check()
    assert single.main(["case_bad_0"]) == 2
    assert "invalid config" in capsys.readouterr().out
