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


def _run(args):
    assert os.path.exists(RUNNER), "kcg_runner is not built (make -C codegendemo_amd/csrc runner)"
    p = subprocess.run([RUNNER] + [str(a) for a in args], capture_output=True, text=True, timeout=120)
    print(p.stdout, p.stderr, flush=True)
    return p


@pytest.mark.parametrize("case", list(CASES))
def test_runner_config_mode(case, tmp_path):
    cfg, kind = CASES[case]
    path = tmp_path / "cfg.json"
    path.write_text(json.dumps({"cfgs": [make_config(256, 256, 256, BM=64, BN=64, BK=16, TM=4, TN=4), cfg]}))
    print(f"[case] kcg_runner --config {case}", flush=True)
    p = _run(["--config", path, "--index", 1, "--kind", kind, "--iters", 5])
    assert p.returncode == 0
    assert "no error!" in p.stdout and "tflops" in p.stdout


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
    r = json.loads(p.stdout.strip().splitlines()[-1])["launch_cost"]
    per = r["period_us"]
    assert 0.5 < per["empty_1_block"] < 50.0 and 0.5 < per["empty_256_blocks"] < 50.0
    assert per["write_64MiB"] > (64 << 20) / 8e12 * 1e6
    assert 1000.0 < r["write_GBps"] < 12000.0      # HBM peak is 8 TB/s; the figure subtracts a launch period, so leave room
