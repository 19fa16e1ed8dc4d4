"""The fetch map of the direct-staging kernel, walked on the host with the kernel's own code.

FetchMap (kcg_device_direct.h) says which 16 bytes of A and B every lane's fetch instructions bring to LDS; it is
written as host-callable code, so tests/kcg_fetch_check.h, appended to the `struct Cfg` of an instantiation stub and
compiled for the host, can walk every block, K tile, wave, instruction and lane of a problem and check that no
fetch leaves the operand buffers (the extents below put the ends of rows and of the buffers at every position
inside a 16-byte chunk, with rows that start 2, 4, ... bytes off a 16-byte boundary) and that every element that
exists lands where the fragment reads look for it.  The checker also lists the kernel's LDS read instructions in the
order the K loop issues them and checks every counted wait (s_waitcnt lgkmcnt(n), n from StreamPlan::allowed) against that
list: a fragment a row is about to use must have at least n reads issued behind it, or the wait would let the row start
before the fragment has arrived.  No GPU needed: the parity tests on the GPU pin the rest."""
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from codegendemo_amd import _native
from codegendemo_amd.kcg.ConfigGenerator import make_config
from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "codegendemo_amd", "csrc")
HIPCC = "/opt/rocm/bin/hipcc"
DIRECT = dict(shared_prefetch=1, reg_prefetch=1)
# (dtype, tile kwargs)
TILES = [
    (2, dict(BM=128, BN=128, TM=8, TN=8, BK=64)),
    (2, dict(BM=64, BN=64, TM=4, TN=4, BK=32)),
    (3, dict(BM=32, BN=64, TM=4, TN=8, BK=32, warp_layout=(8, 8))),      # one wave
    (4, dict(BM=128, BN=64, TM=8, TN=4, BK=16)),
    (4, dict(BM=64, BN=128, TM=4, TN=8, BK=32)),
    (4, dict(BM=32, BN=32, TM=4, TN=4, BK=16)),                          # one wave, 16x16 tiles
]


def cases():
    out = []
    for dtype, tile in TILES:
        g = 16 // (2 if dtype in (2, 3) else 4)
        bm, bn, bk = tile["BM"], tile["BN"], tile["BK"]
        ks = [bk, bk + 1, bk + g - 1, bk + g, bk + g + 1, 2 * bk - 1, 2 * bk, 3 * bk + g // 2 + 1, 5 * bk + 2]
        mns = [(bm - 1, 2 * bn + 1), (bm, bn), (bm + 1, bn - 1), (2 * bm + g // 2, bn + g - 1), (2 * bm - g + 1, 2 * bn - 2),
               (bm + 2, 3 * bn - g - 1), (2 * bm, bn + 1), (bm // 2 + 1, bn // 2 + 3), (3 * bm - 1, bn)]
        for at in (0, 1):
            for i, k in enumerate(ks):
                m, n = mns[(i + at) % len(mns)]
                out.append(make_config(m, n, k, dtype=dtype, dtype_c=4, is_atrans=at, **tile, **DIRECT))
    return out


def ag_cases():
    """Shapes for the build that reads A straight from global memory (-DKCG_A_GLOBAL=1: A [M,K], whole K tiles):
    full tiles, edge tiles in M and N, and block rows of which whole wave rows lie beyond M."""
    out = []
    for dtype, tile in TILES:
        bm, bn, bk = tile["BM"], tile["BN"], tile["BK"]
        for m, n, k in ((bm, bn, bk), (2 * bm, bn + 3, 3 * bk), (bm + 1, 2 * bn, 2 * bk), (bm - 1, bn, 5 * bk), (2 * bm - 17, bn - 1, 4 * bk),
                        (bm // 2 - 1, bn, bk), (bm + bm // 4 + 2, bn, 2 * bk), (1, bn, 2 * bk), (3 * bm - bm // 2, 2 * bn - 8, 6 * bk)):
            out.append(make_config(m, n, k, dtype=dtype, dtype_c=4, is_atrans=0, **tile, **DIRECT))
    return out


def run_check(job):
    index, cfg, workdir = job[:3]
    flags = list(job[3]) if len(job) > 3 else []
    values = kernelArgFromConfig(cfg).values()
    stub = _native.instantiation_source(values, _native.KIND_MFMA)
    if "DIRECT = true" not in stub:
        return index, "not a direct-staging instantiation"
    # the stub without its kernel entry (a host-only build has no device code to register) + the checker's main()
    src = stub.split('extern "C" __global__')[0] + '\n#include "kcg_fetch_check.h"\n'
    path = os.path.join(workdir, f"check_{index}")
    with open(path + ".hip", "w") as f:
        f.write(src)
    p = subprocess.run([HIPCC, "--cuda-host-only", "-O1", "-std=c++17", "-include", "hip/hip_runtime.h", "-I", CSRC, "-I", HERE] + flags + [
                        "-o", path, path + ".hip"], capture_output=True, text=True)
    if p.returncode:
        return index, "compile failed: " + p.stderr[-1500:]
    p = subprocess.run([path], capture_output=True, text=True)
    return index, (p.stdout + p.stderr).strip()


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_every_fetch_stays_inside_the_operands_and_lands_where_it_is_read(tmp_path):
    jobs = [(i, cfg, str(tmp_path)) for i, cfg in enumerate(cases())]
    with ThreadPoolExecutor(max_workers=8) as pool:
        results = list(pool.map(run_check, jobs))
    moved = 0
    for index, text in results:
        cfg = jobs[index][1]
        shape = (cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"], cfg["IS_ATRANS"], cfg["DATATYPE_A"], cfg["BLOCK_SIZE_M"], cfg["BLOCK_SIZE_N"], cfg["BLOCK_SIZE_K"])
        assert text.startswith("ok:"), f"case {index} (M, N, K, A layout, type, tile = {shape}): {text}"
        moved += int(text.split("chunks,")[1].split()[0])
    assert moved > 0          # the sample reaches the chunks at the end of a matrix


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_every_load_of_a_from_global_memory_stays_inside_a(tmp_path):
    """The same walk for the build that loads A fragments straight from global memory: every lane's 16 bytes lie
    inside A (also for waves whose rows all lie beyond M) and are the lane's row and k values where the row exists.
    The checker also lists the counted memory operations of a wave in the order the K loop issues them and
    compares every wait count of the kernel's compile-time schedule (VmSchedule) with it: no wait may allow more
    operations in flight than were issued behind the one it waits for, and the waits for A fragments are exact."""
    jobs = [(i, cfg, str(tmp_path), ("-DKCG_A_GLOBAL=1",)) for i, cfg in enumerate(ag_cases())]
    with ThreadPoolExecutor(max_workers=8) as pool:
        results = list(pool.map(run_check, jobs))
    for index, text in results:
        cfg = jobs[index][1]
        shape = (cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"], cfg["DATATYPE_A"], cfg["BLOCK_SIZE_M"], cfg["BLOCK_SIZE_N"], cfg["BLOCK_SIZE_K"])
        assert text.startswith("ok:"), f"case {index} (M, N, K, type, tile = {shape}): {text}"
