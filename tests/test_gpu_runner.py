"""The stand-alone C++ runner (naive device GEMM + compare kernel + event timing), both argument forms:
the twin of the reference's runkernel.cpp / matmul.cpp main programs."""
import json
import os
import subprocess

import pytest

from codegendemo_amd import _native
from codegendemo_amd.kcg.ConfigGenerator import make_config
from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig

pytestmark = pytest.mark.gpu

RUNNER = os.path.join(os.path.dirname(_native.LIB_PATH), "kcg_runner")

CASES = {
    "f32-mfma": (make_config(1024, 1024, 1024, BM=64, BN=64, BK=16, TM=4, TN=4, is_atrans=0), "mfma"),
    "f32-simt-at": (make_config(1024, 1024, 1024, BM=64, BN=64, BK=16, TM=4, TN=4, is_atrans=1), "simt"),
    "f16-direct": (make_config(1024, 1024, 1024, dtype=2, dtype_c=4, BM=128, BN=128, BK=64, TM=8, TN=8, is_atrans=0,
                               shared_prefetch=1, reg_prefetch=1), "auto"),
}


TIMELINE_CASE = make_config(2048, 2048, 2048, dtype=2, dtype_c=4, BM=256, BN=256, BK=64, TM=16, TN=16, is_atrans=0,
                            shared_prefetch=1, reg_prefetch=1)


def runner_inputs(M, N, K):
    """The runner's operands: a 64-bit LCG (seed 0x4B4347) fills the logical A[M,K] and then B[K,N] in row-major
    order with uniform values on [-1, 1) (kcg_runner.hip: lcg_uniform)."""
    import numpy as np
    n = M * K + K * N
    mask = (1 << 64) - 1
    s = 0x4B4347
    out = np.empty(n, np.float32)
    for i in range(n):
        s = (s * 6364136223846793005 + 1442695040888963407) & mask
        out[i] = ((s >> 40) - (1 << 23)) / float(1 << 23)
    return out[:M * K].reshape(M, K), out[M * K:].reshape(K, N)


def _run(args):
    assert os.path.exists(RUNNER), "kcg_runner is not built (make -C codegendemo_amd/csrc runner)"
    p = subprocess.run([RUNNER] + [str(a) for a in args], capture_output=True, text=True, timeout=120)
    print(p.stdout, p.stderr, flush=True)
    return p


@pytest.mark.parametrize("case", list(CASES))
def test_runner_config_mode(case, tmp_path, oracle):
    """The runner checks the kernel against its own naive device GEMM (the reference runner's contract); the
    result it dumps is checked here against the CPU oracle on the same inputs as well."""
    import numpy as np
    from tests.gemm_helpers import fp32_tolerance, quantize
    cfg, kind = CASES[case]
    path = tmp_path / "cfg.json"
    path.write_text(json.dumps({"cfgs": [make_config(256, 256, 256, BM=64, BN=64, BK=16, TM=4, TN=4), cfg]}))
    print(f"[case] kcg_runner --config {case}", flush=True)
    dump = tmp_path / "c.bin"
    p = _run(["--config", path, "--index", 1, "--kind", kind, "--iters", 5, "--dump-c", dump])
    assert p.returncode == 0
    assert "no error!" in p.stdout and "tflops" in p.stdout
    M, N, K, dt = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"], cfg["DATATYPE_A"]
    a, b = runner_inputs(M, N, K)
    a, b = quantize(a, dt), quantize(b, dt)              # what the device sees
    want = oracle.matmul(a, b, a_trans=False)
    got = np.fromfile(dump, np.float32).reshape(M, N)
    err = float(np.abs(got - want).max())
    if dt == 4:
        assert err <= fp32_tolerance(K, a, b)
    else:
        assert err <= 2e-2 * float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))


def test_runner_timeline_mode(tmp_path):
    """--timeline: the direct-staging kernel built with its in-kernel time stamps; the phases of a launch come
    out in order, every wave reports, and the eight XCDs share the blocks evenly."""
    path = tmp_path / "cfg.json"
    path.write_text(json.dumps({"cfgs": [TIMELINE_CASE]}))
    print("[case] kcg_runner --timeline 2", flush=True)
    p = _run(["--config", path, "--dist", "normal", "--iters", 5, "--timeline", 2])
    assert p.returncode == 0 and "no error!" in p.stdout
    t = json.loads(p.stdout[p.stdout.index('{"timeline"'):])["timeline"]
    assert t["waves"] == 64 * 4 and t["level"] == 2
    u = t["us_after_first_block_start"]
    order = ["block_start", "first_tile_landed", "k_loop_done", "stores_issued", "stores_acknowledged"]
    for x, y in zip(order, order[1:]):
        assert u[x]["mean"] <= u[y]["mean"] and u[x]["last"] <= u[y]["last"]
    assert u["stores_acknowledged"]["last"] <= t["launch_period_us"] * 1.5
    assert 500 < t["k_loop_shader_clock_mhz"]["mean"] <= 2500
    assert 0.0 <= t["barrier_wait_pct_of_k_loop_cycles"]["mean"] < 50.0
    assert [x["waves"] for x in t["by_xcd"]] == [32] * 8


def test_runner_reference_argument_list():
    """M N K gridX blockX code-object kernel-name ldsBytes dtype isATrans — runkernel.cpp's contract."""
    cfg, _ = CASES["f32-mfma"]
    info = _native.compile_matmul(kernelArgFromConfig(cfg).values(), "gfx950", _native.KIND_MFMA)
    print("[case] kcg_runner positional", flush=True)
    p = _run([1024, 1024, 1024, info["grid"][0], info["block"][0], info["code_path"], info["kernel_name"],
              info["lds_bytes"], 4, 0])
    assert p.returncode == 0 and "no error!" in p.stdout


def test_runner_reports_a_wrong_kernel():
    """Launched with A declared transposed although the kernel reads it row-major, the compare kernel
    must count errors and the exit status must say so (every access stays in bounds: M == K)."""
    cfg, _ = CASES["f32-mfma"]
    info = _native.compile_matmul(kernelArgFromConfig(cfg).values(), "gfx950", _native.KIND_MFMA)
    p = _run([1024, 1024, 1024, info["grid"][0], info["block"][0], info["code_path"], info["kernel_name"],
              info["lds_bytes"], 4, 1])
    assert p.returncode == 1 and "error!" in p.stdout and "no error!" not in p.stdout


def test_runner_mfma_peak_mode():
    """Sustained matrix-core rate on register operands: the figure on zeros is close to the published
    peak, the one on normal(0, 0.5) data is lower on a power-limited part, never higher."""
    p = _run(["--mfma-peak", "f16"])
    assert p.returncode == 0
    r = json.loads(p.stdout.strip().splitlines()[-1])["mfma_peak"]
    for shape in ("16x16x32", "32x32x16"):
        assert 500.0 < r["normal(0,0.5)"][shape] <= r["zeros"][shape] * 1.02 < 2516.6 * 1.05


def test_runner_launch_cost_mode():
    """Fixed costs per launch: an empty kernel's back-to-back period is a few microseconds, and writing
    64 MiB (the fp32 result of a 4096 x 4096 product) takes at least what 8 TB/s of HBM allow."""
    p = _run(["--launch-cost"])
    assert p.returncode == 0
    lines = p.stdout.strip().splitlines()
    f = json.loads(lines[-2])["fetch_behind_stores"]
    # a fetch lands, and is reported, no earlier behind 32 stores of the same wave than alone; the counter never
    # reports before the data is there
    assert 0 < f["alone"]["data_visible_in_lds"] <= f["alone"]["vmcnt_0"]
    assert f["alone"]["data_visible_in_lds"] <= f["behind_32_stores"]["data_visible_in_lds"] <= f["behind_32_stores"]["vmcnt_0"]
    r = json.loads(lines[-1])["launch_cost"]
    per = r["period_us"]
    assert 0.5 < per["empty_1_block"] < 50.0 and 0.5 < per["empty_256_blocks"] < 50.0
    assert per["write_64MiB"] > (64 << 20) / 8e12 * 1e6
    assert 1000.0 < r["write_GBps"] < 12000.0      # HBM peak is 8 TB/s; the figure subtracts a launch period, so leave room
