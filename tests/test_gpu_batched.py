"""GPU parity of the batched / strided kernel form and the alpha-beta epilogue (kcg_compile_matmul_ex +
kcg_launch_batched) against the CPU oracle (oracle_matmul_f32_batched_ab): bit for bit on small-integer
inputs with alpha, beta chosen so that every scaled value stays exact, for each kernel family (scalar,
register-staged matrix-core with and without split-U, direct staging in fp32 and fp16), both A layouts, edge
shapes, padded strides and an operand shared by the whole batch; within the fp32 bar on real-valued data."""
import numpy as np
import pytest

from codegendemo_amd import _native
from codegendemo_amd.kcg import SeededInputs as SI
from codegendemo_amd.kcg.CompiledKernelFactory import CompiledKernelFactory, EnumOperator, UserInputs
from codegendemo_amd.kcg.ConfigGenerator import make_config
from codegendemo_amd.kcg.KCGCompiler import KCGCompiler
from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig
from tests.gemm_helpers import fp32_tolerance, quantize, to_device

pytestmark = pytest.mark.gpu

SIMT, MFMA = _native.KIND_SIMT, _native.KIND_MFMA
NONE, AB = _native.EPILOGUE_NONE, _native.EPILOGUE_ALPHA_BETA

DIRECT = dict(shared_prefetch=1, reg_prefetch=1)
# (tag, kind, make_config kwargs, batch)
CASES = [
    ("simt", SIMT, dict(M=128, N=192, K=64), 3),
    ("simt-at0-edge", SIMT, dict(M=100, N=72, K=50, is_atrans=0), 2),
    ("simt-lsu2", SIMT, dict(M=128, N=128, K=64, lsu=2), 2),
    ("mfma", MFMA, dict(M=128, N=192, K=64, is_atrans=0), 3),
    ("mfma-edge", MFMA, dict(M=200, N=136, K=100), 2),
    ("mfma-lsu2-at0", MFMA, dict(M=128, N=128, K=128, lsu=2, is_atrans=0, BK=32), 2),
    ("f32-direct", MFMA, dict(M=256, N=256, K=272, BM=128, BN=128, TM=8, TN=8, BK=16, is_atrans=0, **DIRECT), 3),
    ("f32-direct-edge-at1", MFMA, dict(M=200, N=136, K=104, BM=128, BN=64, TM=8, TN=4, BK=16, is_atrans=1, **DIRECT), 2),
    ("f16-direct", MFMA, dict(M=256, N=256, K=192, dtype=2, dtype_c=4, BM=128, BN=128, TM=8, TN=8, BK=64, is_atrans=0, **DIRECT), 2),
    ("bf16-mfma-at1", MFMA, dict(M=128, N=128, K=96, dtype=3, dtype_c=4, BM=64, BN=64, BK=32, is_atrans=1), 2),
    # odd extents: rows off 4-byte boundaries, and the last chunk of every problem's A and B fetched from further down
    ("f16-direct-odd", MFMA, dict(M=254, N=249, K=203, dtype=2, dtype_c=4, BM=128, BN=128, TM=8, TN=8, BK=64, is_atrans=0, **DIRECT), 3),
    ("bf16-direct-odd-at1", MFMA, dict(M=125, N=131, K=128, dtype=3, dtype_c=4, BM=64, BN=64, TM=4, TN=4, BK=32, is_atrans=1, **DIRECT), 2),
]


def configs_to_build():
    """(config, kind, epilogue) of every kernel this file launches (precompiled by the build step)."""
    out = []
    for _tag, kind, kw, _batch in CASES:
        out += [(make_config(**kw), kind, NONE), (make_config(**kw), kind, AB)]
    out.append((make_config(**REAL_CASE), MFMA, AB))
    return out


REAL_CASE = dict(M=512, N=384, K=520, BM=128, BN=128, TM=8, TN=8, BK=8, is_atrans=0, **DIRECT)


def build(config, kind, epilogue):
    kpm = kernelArgFromConfig(config)
    comp = KCGCompiler(kind=kind, epilogue=epilogue)
    path, name, gx, gy, gz, bx, by, bz = comp.compileKernel(kpm)[0]
    ui = UserInputs(path, name, kpm)
    ui.m_gridDims, ui.m_blockDims = [gx, gy, gz], [bx, by, bz]
    ui.m_ldsBytes = comp.lastInfo["lds_bytes"]
    ui.operatorKind = EnumOperator.Matmul
    return kpm, CompiledKernelFactory.getKernel(ui, 0), comp.lastInfo


def run_batched(config, kind, epilogue, a, b, c0, strides, alpha, beta):
    """a: [batch, M, K] logical, b: [batch or 1, K, N], c0: flat fp32 buffer of batch problems at stride_c.
    Returns the C buffer after the launch (flat fp32)."""
    import torch
    kpm, kernel, info = build(config, kind, epilogue)
    batch = a.shape[0]
    sa, sb, sc = strides
    ta = kpm.dtypeTorch('A')
    a_flat = np.zeros((batch - 1) * sa + kpm.M * kpm.K, np.float32)
    for z in range(batch):
        a_flat[z * sa:z * sa + kpm.M * kpm.K] = SI.a_operand(a[z], kpm.isATranspose).ravel()
    b_flat = np.zeros((batch - 1) * sb + kpm.K * kpm.N, np.float32)
    for z in range(b.shape[0]):
        b_flat[z * sb:z * sb + kpm.K * kpm.N] = b[z].ravel()
    a_dev, b_dev = to_device(a_flat, ta), to_device(b_flat, ta)
    c_dev = to_device(c0, torch.float32)
    # first on NaN operands (LDS keeps its contents between launches: a fragment read too early must not find
    # the right values there), into a scratch result
    kernel.run_batched(torch.full_like(a_dev, float("nan")), torch.full_like(b_dev, float("nan")), torch.empty_like(c_dev),
                       batch, sa, sb, sc, alpha, beta)
    torch.cuda.synchronize()
    kernel.run_batched(a_dev, b_dev, c_dev, batch, sa, sb, sc, alpha, beta)
    torch.cuda.synchronize()
    out = c_dev.cpu().numpy()
    kernel.unload()
    return out, a_flat, b_flat, info


@pytest.mark.parametrize("tag,kind,kw,batch", CASES, ids=[c[0] for c in CASES])
def test_batched_alpha_beta_bit_exact_on_integers(oracle, tag, kind, kw, batch):
    cfg = make_config(**kw)
    M, N, K, at = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"], cfg["IS_ATRANS"]
    a = np.stack([SI.small_ints((M, K), 400 + z) for z in range(batch)])
    b = np.stack([SI.small_ints((K, N), 500 + z) for z in range(batch)])
    pad8 = lambda x: (x + 7) // 8 * 8
    sa, sb, sc = pad8(M * K) + 16, pad8(K * N) + 32, pad8(M * N) + 8   # padded strides (kept 16-byte aligned for every type)
    c0 = SI.small_ints((batch * sc,), 600).astype(np.float32)
    for alpha, beta in ((2.0, -3.0), (1.0, 1.0), (-0.5, 0.0)):
        print(f"[case] {tag} kind={kind} {M}x{N}x{K} batch={batch} alpha={alpha} beta={beta}", flush=True)
        c_in = c0.copy()
        if beta == 0.0:
            c_in[:] = np.nan                                           # beta == 0: C must not be read
        got, a_flat, b_flat, info = run_batched(cfg, kind, AB, a, b, c_in, (sa, sb, sc), alpha, beta)
        assert info["kind"] == kind and info["kernel_name"].endswith("EXab_")
        want = oracle.batched_ab(a_flat, b_flat, c_in, M, N, K, at, batch, (sa, sb, sc), alpha, beta)
        for z in range(batch):
            g, w = got[z * sc:z * sc + M * N], want[z * sc:z * sc + M * N]
            bad = np.argwhere(g != w)
            assert bad.size == 0, f"{tag} problem {z}: {len(bad)} mismatches, first at {bad[:5].ravel().tolist()}"
            if z + 1 < batch:                                          # the padding between problems is not touched
                pad_g, pad_w = got[z * sc + M * N:(z + 1) * sc], c_in[z * sc + M * N:(z + 1) * sc]
                assert np.array_equal(pad_g, pad_w, equal_nan=True)


@pytest.mark.parametrize("tag,kind,kw,batch", [CASES[0], CASES[3], CASES[6], CASES[8]], ids=["simt", "mfma", "f32-direct", "f16-direct"])
def test_batched_without_epilogue_and_shared_b(oracle, tag, kind, kw, batch):
    """The batched form without the epilogue equals per-problem products; stride_b = 0 shares B."""
    cfg = make_config(**kw)
    M, N, K, at = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"], cfg["IS_ATRANS"]
    a = np.stack([SI.small_ints((M, K), 700 + z) for z in range(batch)])
    b = SI.small_ints((K, N), 800)[None]
    sa, sc = M * K, M * N
    c_in = np.full(batch * sc, np.nan, np.float32)
    print(f"[case] {tag} no-epilogue kind={kind} {M}x{N}x{K} batch={batch} shared B", flush=True)
    got, _, _, info = run_batched(cfg, kind, NONE, a, b, c_in, (sa, 0, sc), 123.0, 456.0)   # alpha, beta ignored
    assert info["kernel_name"].endswith("EX_")
    for z in range(batch):
        want = oracle.matmul(a[z], b[0], a_trans=False)
        assert np.array_equal(got[z * sc:(z + 1) * sc].reshape(M, N), want), f"{tag} problem {z}"


def test_alpha_beta_on_real_valued_data(oracle):
    """Uniform inputs, alpha = 0.75, beta = -1.25 through the direct-staging kernel: within the fp32 bar
    1e-4 * K * max|a| * max|b| (scaled by |alpha|) plus the rounding of beta * C0."""
    cfg = make_config(**REAL_CASE)
    M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
    batch, alpha, beta = 2, 0.75, -1.25
    a = np.stack([SI.uniform((M, K), 900 + z) for z in range(batch)])
    b = np.stack([SI.uniform((K, N), 910 + z) for z in range(batch)])
    c0 = SI.uniform((batch * M * N,), 920)
    strides = (M * K, K * N, M * N)
    print(f"[case] real-valued alpha-beta {M}x{N}x{K} batch={batch}", flush=True)
    got, a_flat, b_flat, _ = run_batched(cfg, MFMA, AB, a, b, c0, strides, alpha, beta)
    want = oracle.batched_ab(a_flat, b_flat, c0, M, N, K, 0, batch, strides, alpha, beta)
    tol = abs(alpha) * fp32_tolerance(K, a, b) + 1e-6
    assert float(np.abs(got - want).max()) <= tol


def test_launch_batched_argument_checks():
    cfg = make_config(M=128, N=192, K=64)
    kpm, kernel, info = build(cfg, SIMT, AB)
    import torch
    a = torch.zeros(2 * 128 * 64, device="cuda:0")
    b = torch.zeros(2 * 64 * 192, device="cuda:0")
    c = torch.zeros(2 * 128 * 192, device="cuda:0")
    with pytest.raises(_native.KcgError):
        kernel.run_batched(a, b, c, 2, 128 * 64, 64 * 192, 0)              # two problems on one C
    with pytest.raises(_native.KcgError):
        kernel.run_batched(a, b, c, 70000, 0, 0, 0)
    with pytest.raises(ValueError):
        kernel.run_batched(a, b, c, 3, 128 * 64, 64 * 192, 128 * 192)      # buffers hold two problems, not three
    with pytest.raises(ValueError):
        kernel.run_batched(a, b, c, 2, 128 * 64 - 2, 64 * 192, 128 * 192)  # second problem's A not 16-byte aligned
    with pytest.raises(TypeError):
        kernel.run(a, b, c)                                                # the three-pointer launch does not fit this kernel
    kernel.run_batched(a, b, c, 0, 0, 0, 0)                                # empty batch: nothing launched
    torch.cuda.synchronize()
    # the C ABI itself knows which form a function it loaded has, and refuses the other launch call
    ui = kernel.m_launcher.m_kernelLib
    fn = kernel.m_launcher._function()
    with pytest.raises(_native.KcgError, match="kcg_launch_batched"):
        _native.launch(fn, ui.m_gridDims, ui.m_blockDims, ui.m_shmSize, 0, a.data_ptr(), b.data_ptr(), c.data_ptr())
    kernel.unload()
    _, plain, _ = build(cfg, SIMT, None)
    with pytest.raises(TypeError):
        plain.run_batched(a, b, c, 1, 0, 0, 0)
    ui = plain.m_launcher.m_kernelLib
    fn = plain.m_launcher._function()
    with pytest.raises(_native.KcgError, match="kcg_launch"):
        _native.launch_batched(fn, ui.m_gridDims, ui.m_blockDims, ui.m_shmSize, 0, a.data_ptr(), b.data_ptr(), c.data_ptr(),
                               1, 0, 0, 0)
    plain.unload()


def test_batched_benchmark_times_the_whole_batch(oracle):
    """kcg_benchmark_batched: the C timing loop around the batched launch; C afterwards is the batch's result."""
    import torch
    tag, kind, kw, batch = CASES[8]
    cfg = make_config(**kw)
    M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
    kpm, kernel, info = build(cfg, kind, AB)
    a = np.stack([SI.small_ints((M, K), 1000 + z) for z in range(batch)])
    b = np.stack([SI.small_ints((K, N), 1100 + z) for z in range(batch)])
    a_dev = to_device(a.reshape(-1), kpm.dtypeTorch('A'))
    b_dev = to_device(b.reshape(-1), kpm.dtypeTorch('A'))
    c_dev = torch.full((batch * M * N,), float("nan"), dtype=torch.float32, device="cuda:0")
    print(f"[case] batched benchmark {tag} {M}x{N}x{K} batch={batch}", flush=True)
    med, mn = kernel.benchmark_batched(a_dev, b_dev, c_dev, batch, M * K, K * N, M * N, alpha=2.0, beta=0.0, warmup=2, iters=5, reps=3)
    torch.cuda.synchronize()
    assert 0 < mn <= med < 100.0
    got = c_dev.cpu().numpy().reshape(batch, M, N)
    for z in range(batch):
        assert np.array_equal(got[z], 2.0 * oracle.matmul(a[z], b[z], a_trans=False))
    # every problem of a batch must start 16-byte aligned: strides that are not are refused, by the Python launcher
    # (which names the operand) and by the C entry points themselves, before anything is launched
    with pytest.raises(ValueError, match="stride_a"):
        kernel.benchmark_batched(a_dev, b_dev, c_dev, batch, M * K - 1, K * N, M * N)
    with pytest.raises(ValueError, match="stride_c"):
        kernel.run_batched(a_dev, b_dev, c_dev, batch, M * K, K * N, M * N - 2)
    fn = kernel._info().m_function
    for strides in ((M * K - 1, K * N, M * N), (M * K, K * N - 2, M * N), (M * K, K * N, M * N - 3)):
        with pytest.raises(_native.KcgError, match="multiples of 16 bytes"):
            _native.launch_batched(fn, kernel.gridDims, kernel.blockDims, kernel.shmSize, 0, a_dev.data_ptr(), b_dev.data_ptr(),
                                   c_dev.data_ptr(), batch, *strides)
    _native.launch_batched(fn, kernel.gridDims, kernel.blockDims, kernel.shmSize, 0, a_dev.data_ptr(), b_dev.data_ptr(),
                           c_dev.data_ptr(), 1, M * K - 1, K * N - 1, M * N - 1)      # one problem: the strides are not used
    torch.cuda.synchronize()
    kernel.unload()
    plain = build(make_config(M=128, N=192, K=64), SIMT, None)[1]          # a three-pointer kernel
    with pytest.raises(TypeError):
        plain.benchmark_batched(a_dev, b_dev, c_dev, 1, 0, 0, 0)
