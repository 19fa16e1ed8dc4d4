"""The stand-alone runner's host side without a GPU: reading a config out of a {"cfgs": [...]} file or a
single flat object, compiling it through the library (--compile-only), usage and error exits."""
import json
import os
import subprocess

import pytest

from codegendemo_amd import _native
from codegendemo_amd.kcg.ConfigGenerator import make_config
from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig

RUNNER = os.path.join(os.path.dirname(_native.LIB_PATH), "kcg_runner")

pytestmark = pytest.mark.skipif(not os.path.exists(RUNNER), reason="kcg_runner is not built (make -C codegendemo_amd/csrc runner)")


def _run(args, env=None):
    return subprocess.run([RUNNER] + [str(a) for a in args], capture_output=True, text=True, timeout=120,
                          env=dict(os.environ, **(env or {})))


def test_compile_only_picks_the_indexed_config(tmp_path):
    first = make_config(256, 256, 256, BM=64, BN=64, BK=16, TM=4, TN=4)
    second = make_config(512, 256, 128, BM=64, BN=64, BK=16, TM=4, TN=4, is_atrans=0)
    path = tmp_path / "cfgs.json"
    path.write_text(json.dumps({"cfgs": [first, second]}))
    p = _run(["--config", path, "--index", 1, "--kind", "simt", "--compile-only", 1], {"KCG_CACHE_DIR": str(tmp_path / "cache")})
    assert p.returncode == 0, p.stderr
    assert _native.kernel_name(kernelArgFromConfig(second).values()) in p.stdout and "SIMT kernel" in p.stdout
    assert sorted(f.rsplit(".", 1)[1] for f in os.listdir(tmp_path / "cache")) == ["buildinfo", "hsaco"]
    # a single flat object works too, and a second run is a cache hit
    flat = tmp_path / "one.json"
    flat.write_text(json.dumps(second))
    p = _run(["--config", flat, "--kind", "simt", "--compile-only", 1], {"KCG_CACHE_DIR": str(tmp_path / "cache")})
    assert p.returncode == 0 and "cache hit" in p.stdout


def test_bad_inputs_exit_with_a_message(tmp_path):
    assert _run([]).returncode == 2
    p = _run(["--config", tmp_path / "missing.json"])
    assert p.returncode == 2 and "cannot read config" in p.stderr
    bad = tmp_path / "bad.json"
    cfg = make_config(256, 256, 256)
    del cfg["BLOCK_SIZE_K"]
    bad.write_text(json.dumps({"cfgs": [cfg]}))
    p = _run(["--config", bad])
    assert p.returncode == 2 and "BLOCK_SIZE_K" in p.stderr
    invalid = tmp_path / "invalid.json"
    invalid.write_text(json.dumps(dict(make_config(256, 256, 256), WARP_LAYOUT_M=4)))   # 4 x 8 lanes is no wave
    p = _run(["--config", invalid, "--compile-only", 1])
    assert p.returncode == 2 and "compile failed" in p.stderr
