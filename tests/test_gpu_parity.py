"""GPU parity tests: the HIP kernels, driven through the C ABI, against the CPU oracle on the same
seeded inputs.  Integer-valued inputs must match bit for bit (every product and partial sum is exact
in fp32, so summation order cannot matter); real-valued fp32 inputs must satisfy
max|err| <= 1e-4*K*max|a|*max|b|; 16-bit inputs <= 2e-2 relative to the result scale."""
import numpy as np
import pytest

from codegendemo_amd import _native
from codegendemo_amd.kcg import SeededInputs as SI
from codegendemo_amd.kcg.ConfigGenerator import make_config
from tests.gemm_helpers import fp32_tolerance, hiprtc_params, quantize, run_gemm

pytestmark = pytest.mark.gpu

SIMT, MFMA = _native.KIND_SIMT, _native.KIND_MFMA


def _exact_case(oracle, cfg, kind, tag):
    M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
    a = SI.small_ints((M, K), SI.STREAM_A)
    b = SI.small_ints((K, N), SI.STREAM_B)
    print(f"[case] {tag} kind={kind} {M}x{N}x{K} cfg={ {k: cfg[k] for k in ('BLOCK_SIZE_M','BLOCK_SIZE_N','BLOCK_SIZE_K','THREAD_SIZE_M','THREAD_SIZE_N','LOCAL_SPLIT_U','IS_ATRANS','SHARED_PREFETCH','REG_PREFETCH','LOAD_CONTINUOUS','DATATYPE_A')} }", flush=True)
    got, info = run_gemm(cfg, a, b, kind)
    assert info["kind"] == kind
    if "direct" in tag and kind == MFMA:
        assert info["lds_bytes"] == 0, "expected the direct-staging kernel (static LDS)"
    want = oracle.matmul(a, b, a_trans=False)
    assert not np.isnan(got).any(), "some C elements were never written"
    bad = np.argwhere(got != want)
    assert bad.size == 0, f"{tag}: {len(bad)} mismatches, first at {bad[:5].tolist()}"


# (kind, kwargs) — small problems, every structural code path of both kernel families
EXACT_CASES = [
    ("simt-base", SIMT, dict(M=256, N=256, K=128)),
    ("simt-atrans0", SIMT, dict(M=256, N=256, K=128, is_atrans=0)),
    ("simt-lc0", SIMT, dict(M=256, N=256, K=128, load_continuous=0)),
    ("simt-shmp", SIMT, dict(M=256, N=256, K=128, shared_prefetch=1)),
    ("simt-regp", SIMT, dict(M=256, N=256, K=128, reg_prefetch=1)),
    ("simt-both", SIMT, dict(M=256, N=256, K=128, shared_prefetch=1, reg_prefetch=1, is_atrans=0)),
    ("simt-lsu2", SIMT, dict(M=256, N=256, K=128, lsu=2)),
    ("simt-lsu2-rc0", SIMT, dict(M=256, N=256, K=128, lsu=2, reduce_c_continuous=0, shared_prefetch=1)),
    ("simt-scatter1", SIMT, dict(M=256, N=256, K=128, scatter=1)),
    ("simt-scatter2", SIMT, dict(M=256, N=256, K=128, scatter=2, TM=8, TN=8, BM=128, BN=128)),
    ("simt-wl4x16", SIMT, dict(M=256, N=256, K=128, warp_layout=(4, 16), BM=32, BN=64, BK=8)),
    ("simt-edge", SIMT, dict(M=200, N=136, K=100)),
    ("simt-edge-at0", SIMT, dict(M=200, N=136, K=100, is_atrans=0, shared_prefetch=1)),
    ("simt-odd", SIMT, dict(M=131, N=67, K=37, is_atrans=0, lsu=2)),
    ("simt-f64", SIMT, dict(M=256, N=256, K=128, dtype=8, scatter=2)),
    ("simt-f64-at0-both", SIMT, dict(M=256, N=192, K=136, dtype=8, scatter=2, is_atrans=0, shared_prefetch=1, reg_prefetch=1, BK=8)),
    ("simt-f64-lsu2-edge", SIMT, dict(M=200, N=136, K=100, dtype=8, scatter=1, lsu=2)),
    ("mfma-base", MFMA, dict(M=256, N=256, K=128)),
    ("mfma-atrans0", MFMA, dict(M=256, N=256, K=128, is_atrans=0)),
    ("mfma-shmp", MFMA, dict(M=256, N=256, K=128, shared_prefetch=1)),
    ("mfma-regp", MFMA, dict(M=256, N=256, K=128, reg_prefetch=1, BK=32)),
    ("mfma-both-at0", MFMA, dict(M=256, N=256, K=128, shared_prefetch=1, reg_prefetch=1, is_atrans=0, BK=32)),
    ("mfma-lsu2", MFMA, dict(M=256, N=256, K=128, lsu=2)),
    ("mfma-lsu2-at0", MFMA, dict(M=256, N=256, K=128, lsu=2, is_atrans=0, shared_prefetch=1, BK=32)),
    ("mfma-128x128", MFMA, dict(M=256, N=256, K=128, BM=128, BN=128, TM=8, TN=8, shared_prefetch=1, reg_prefetch=1)),
    ("mfma-128x64-at0", MFMA, dict(M=256, N=256, K=128, BM=128, BN=64, TM=8, TN=4, is_atrans=0)),
    ("mfma-16x16", MFMA, dict(M=256, N=256, K=128, warp_layout=(4, 16), BM=32, BN=64, BK=16)),
    ("mfma-16x16-at0", MFMA, dict(M=256, N=256, K=128, warp_layout=(16, 4), BM=64, BN=32, BK=32, is_atrans=0)),
    ("mfma-glw2", MFMA, dict(M=256, N=256, K=128, glw=2)),
    ("mfma-glw1-at0", MFMA, dict(M=256, N=256, K=128, glw=1, is_atrans=0)),
    ("mfma-edge", MFMA, dict(M=200, N=136, K=100)),
    ("mfma-edge-at0", MFMA, dict(M=200, N=136, K=100, is_atrans=0, shared_prefetch=1)),
    ("mfma-odd", MFMA, dict(M=131, N=67, K=37, is_atrans=0)),
    ("mfma-odd-at1", MFMA, dict(M=131, N=67, K=37, is_atrans=1, lsu=2, BK=32)),
    ("mfma-64x48", MFMA, dict(M=256, N=192, K=128, BM=64, BN=48, BK=32, TM=4, TN=6, scatter=2, glw=2, gsw=2, lsu=2)),
    ("simt-64x48", SIMT, dict(M=256, N=192, K=128, BM=64, BN=48, BK=32, TM=4, TN=6, scatter=2, glw=2, gsw=2, lsu=2)),
    # fp32 through the direct-staging kernel (both prefetch flags + LOAD_CONTINUOUS): 4, 2 and 3 LDS stages,
    # both A layouts, long K (steady-state loop), 32x32 and 16x16 matrix-core tiles, 8 waves
    ("f32-direct-128-at0", MFMA, dict(M=256, N=256, K=256, BM=128, BN=128, TM=8, TN=8, BK=16, is_atrans=0,
                                      shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-128-at1-longk", MFMA, dict(M=256, N=256, K=1040, BM=128, BN=128, TM=8, TN=8, BK=16, is_atrans=1,
                                            shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-256-2st", MFMA, dict(M=256, N=512, K=1024, BM=256, BN=256, TM=16, TN=16, BK=32, is_atrans=0,
                                      shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-256x128-3st-at1", MFMA, dict(M=512, N=256, K=1056, BM=256, BN=128, TM=16, TN=8, BK=32, is_atrans=1,
                                              shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-bk8", MFMA, dict(M=256, N=256, K=520, BM=128, BN=128, TM=8, TN=8, BK=8, is_atrans=0,
                                  shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-mf16-8w", MFMA, dict(M=256, N=256, K=544, BM=128, BN=64, TM=8, TN=2, BK=32, is_atrans=0,
                                      shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-mf16-8w-at1", MFMA, dict(M=256, N=256, K=544, BM=128, BN=64, TM=8, TN=2, BK=32, is_atrans=1,
                                          shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-kt1", MFMA, dict(M=256, N=256, K=16, BM=128, BN=128, TM=8, TN=8, BK=16, is_atrans=0,
                                  shared_prefetch=1, reg_prefetch=1)),                    # a single K tile
    ("f32-direct-kt2-at1", MFMA, dict(M=256, N=256, K=64, BM=128, BN=128, TM=8, TN=8, BK=32, is_atrans=1,
                                      shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-1wave", MFMA, dict(M=256, N=256, K=1056, BM=128, BN=128, TM=16, TN=16, BK=32, is_atrans=0,
                                    shared_prefetch=1, reg_prefetch=1)),
    # direct staging with edge tiles: a partial last K tile (fetched by tile KT-NST, by tile 0, or in the
    # prologue), rows and columns beyond M and N, both A layouts, both matrix-core tile sizes
    ("f32-direct-ktail", MFMA, dict(M=256, N=256, K=1000, BM=128, BN=64, TM=8, TN=4, BK=16, is_atrans=0,
                                    shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-ktail-bk32-at1", MFMA, dict(M=256, N=256, K=1000, BM=128, BN=128, TM=8, TN=8, BK=32, is_atrans=1,
                                             shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-ktail-tile0", MFMA, dict(M=256, N=256, K=72, BM=128, BN=64, TM=8, TN=4, BK=16, is_atrans=0,
                                          shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-ktail-prologue-at1", MFMA, dict(M=256, N=256, K=24, BM=128, BN=64, TM=8, TN=4, BK=16, is_atrans=1,
                                                 shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-edge-mn", MFMA, dict(M=200, N=136, K=104, BM=128, BN=64, TM=8, TN=4, BK=16, is_atrans=0,
                                      shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-edge-mn-at1", MFMA, dict(M=200, N=136, K=104, BM=128, BN=64, TM=8, TN=4, BK=16, is_atrans=1,
                                          shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-edge-256", MFMA, dict(M=260, N=516, K=1064, BM=256, BN=256, TM=16, TN=16, BK=32, is_atrans=0,
                                       shared_prefetch=1, reg_prefetch=1)),
    # 32-wide block tiles (one wave of 32x32, two of 32x32 side by side): 8 chunks per tile row
    ("f32-direct-32x32-1wave", MFMA, dict(M=96, N=160, K=272, BM=32, BN=32, TM=4, TN=4, BK=16, is_atrans=1,
                                          shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-32x64-edge", MFMA, dict(M=100, N=136, K=108, BM=32, BN=64, TM=4, TN=4, BK=32, is_atrans=0,
                                         shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-64x32-at1", MFMA, dict(M=128, N=96, K=520, BM=64, BN=32, TM=8, TN=4, BK=8, is_atrans=1,
                                        shared_prefetch=1, reg_prefetch=1)),
    # block tiles that are not powers of two (whole groups of 16 chunks per tile row): 192 columns, 192 rows in
    # both A layouts, edges in M, N and K
    ("f32-direct-64x192", MFMA, dict(M=256, N=768, K=544, BM=64, BN=192, TM=4, TN=12, BK=32, is_atrans=0,
                                     shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-192x64-at1-edge", MFMA, dict(M=500, N=200, K=1000, BM=192, BN=64, TM=12, TN=4, BK=16, is_atrans=1,
                                              shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-192x128-at0-edge", MFMA, dict(M=388, N=516, K=264, BM=192, BN=128, TM=12, TN=8, BK=32, is_atrans=0,
                                               shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-128x192-8w", MFMA, dict(M=512, N=1536, K=1000, BM=128, BN=192, TM=8, TN=6, BK=32, is_atrans=0,
                                         scatter=2, shared_prefetch=1, reg_prefetch=1)),
    # K remainders that end inside a k-step: the lanes holding k >= K clear their fragments
    ("f32-direct-kpart", MFMA, dict(M=256, N=256, K=1004, BM=128, BN=64, TM=8, TN=4, BK=16, is_atrans=0,
                                    shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-kpart-bk32-at1", MFMA, dict(M=200, N=136, K=1020, BM=128, BN=128, TM=8, TN=8, BK=32, is_atrans=1,
                                             shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-mf16-kpart-at1", MFMA, dict(M=252, N=248, K=572, BM=128, BN=64, TM=8, TN=2, BK=32, is_atrans=1,
                                             shared_prefetch=1, reg_prefetch=1)),
    ("f32-direct-mf16-ktail", MFMA, dict(M=252, N=248, K=560, BM=128, BN=64, TM=8, TN=2, BK=32, is_atrans=0,
                                         shared_prefetch=1, reg_prefetch=1)),
    # scalar kernel, edge tiles under register pressure (16-wide thread tiles, a one-wave block with 192
    # staging registers): shapes that returned wrong values when the compiler was allowed to park vector
    # registers in accumulation registers
    ("simt-edge-16x8-both", SIMT, dict(M=244, N=376, K=112, BM=128, BN=128, BK=16, TM=16, TN=8, is_atrans=1,
                                       shared_prefetch=1, reg_prefetch=1, block_mapping=0, reduce_c_continuous=0)),
    ("simt-edge-1wave-8x16", SIMT, dict(M=124, N=124, K=133, BM=64, BN=128, BK=64, TM=8, TN=16, is_atrans=1,
                                        shared_prefetch=1, reg_prefetch=1, block_mapping=2, load_continuous=0,
                                        scatter=2, glw=1)),
    ("simt-edge-1wave-8x16-glw4", SIMT, dict(M=124, N=124, K=136, BM=64, BN=128, BK=64, TM=8, TN=16, is_atrans=1,
                                             shared_prefetch=1, reg_prefetch=1, block_mapping=2, load_continuous=0,
                                             scatter=2, glw=4)),
    ("simt-edge-16x8-unaligned", SIMT, dict(M=127, N=509, K=33, BM=128, BN=256, BK=16, TM=16, TN=8, is_atrans=1,
                                            shared_prefetch=1, block_mapping=2, reduce_c_continuous=0)),
    ("simt-edge-16x16-lsu2", SIMT, dict(M=124, N=253, K=66, BM=128, BN=128, BK=16, TM=16, TN=16, is_atrans=1,
                                        shared_prefetch=1, reg_prefetch=1, lsu=2, reduce_c_continuous=0)),
    # fp64 on the matrix cores (16x16x4 instructions, two k values per 16-byte chunk)
    ("mfma-f64", MFMA, dict(M=256, N=256, K=128, dtype=8, scatter=2)),
    ("mfma-f64-at0-both", MFMA, dict(M=256, N=192, K=136, dtype=8, scatter=2, is_atrans=0, shared_prefetch=1,
                                     reg_prefetch=1, BK=8)),
    ("mfma-f64-128x128", MFMA, dict(M=256, N=256, K=256, dtype=8, scatter=2, BM=128, BN=128, TM=8, TN=8, BK=16,
                                    is_atrans=0, shared_prefetch=1, reg_prefetch=1)),
    ("mfma-f64-lsu2-edge", MFMA, dict(M=200, N=136, K=100, dtype=8, scatter=1, lsu=2)),
    ("mfma-bm0", MFMA, dict(M=512, N=256, K=64, block_mapping=0)),
    ("mfma-bm4", MFMA, dict(M=512, N=384, K=64, block_mapping=4)),
]


@pytest.mark.parametrize("tag,kind,kw", EXACT_CASES, ids=[c[0] for c in EXACT_CASES])
def test_exact_small_integers_fp32(oracle, tag, kind, kw):
    _exact_case(oracle, make_config(**kw), kind, tag)


HALF_CASES = [
    ("f16-at0", dict(M=256, N=256, K=128, dtype=2, dtype_c=4, is_atrans=0, BK=32)),
    ("f16-at1", dict(M=256, N=256, K=128, dtype=2, dtype_c=4, is_atrans=1, BK=32)),
    ("f16-128-shmp", dict(M=256, N=256, K=256, dtype=2, dtype_c=4, is_atrans=0, BM=128, BN=128, TM=8, TN=8, BK=64,
                          shared_prefetch=1, reg_prefetch=1)),
    ("f16-16x16", dict(M=256, N=256, K=128, dtype=2, dtype_c=4, is_atrans=0, warp_layout=(4, 16), BM=32, BN=64, BK=32)),
    ("f16-edge", dict(M=200, N=136, K=100, dtype=2, dtype_c=4, is_atrans=0, BK=32)),
    ("f16-glw4", dict(M=256, N=256, K=128, dtype=2, dtype_c=4, is_atrans=1, BK=32, glw=4)),
    ("f16-out16", dict(M=256, N=256, K=128, dtype=2, is_atrans=0, BK=32)),
    ("f16-direct-at1", dict(M=256, N=256, K=256, dtype=2, dtype_c=4, is_atrans=1, BM=128, BN=128, TM=8, TN=8, BK=64,
                            shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-128x384", dict(M=256, N=768, K=544, dtype=2, dtype_c=4, is_atrans=0, BM=128, BN=384, TM=8, TN=12, BK=32,
                                shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-384x128-at1-edge", dict(M=776, N=248, K=552, dtype=2, dtype_c=4, is_atrans=1, BM=384, BN=128, TM=12, TN=8,
                                         BK=32, shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-bk32", dict(M=256, N=384, K=224, dtype=2, dtype_c=4, is_atrans=0, BM=128, BN=128, TM=8, TN=8, BK=32,
                             shared_prefetch=1, reg_prefetch=1)),
    ("f16-wl4x16-shmp", dict(M=256, N=256, K=256, dtype=2, dtype_c=4, is_atrans=0, warp_layout=(4, 16), BM=64, BN=64,
                              BK=32, shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-16x16-at1", dict(M=256, N=256, K=256, dtype=2, dtype_c=4, is_atrans=1, warp_layout=(16, 4), BM=64,
                                  BN=64, BK=64, shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-256", dict(M=512, N=512, K=512, dtype=2, dtype_c=4, is_atrans=0, BM=256, BN=256, TM=16, TN=16, BK=64,
                            shared_prefetch=1, reg_prefetch=1, block_mapping=4)),
    ("f16-direct-256x128-8w", dict(M=512, N=512, K=192, dtype=2, dtype_c=4, is_atrans=1, BM=256, BN=128, TM=8, TN=8,
                                   BK=64, shared_prefetch=1, reg_prefetch=1)),
    ("bf16-direct", dict(M=256, N=256, K=256, dtype=3, dtype_c=4, is_atrans=0, BM=128, BN=128, TM=8, TN=8, BK=64,
                         shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-out16", dict(M=256, N=256, K=128, dtype=2, is_atrans=0, BM=128, BN=128, TM=8, TN=8, BK=64,
                              shared_prefetch=1, reg_prefetch=1)),
    # long K: the steady-state part of the direct-staging K loop (groups of NST tiles) with 4, 2, 3 and 4
    # LDS stages, tile counts that leave 1..NST tiles for the unrolled rest
    ("f16-direct-longk-4st", dict(M=256, N=256, K=2048, dtype=2, dtype_c=4, is_atrans=0, BM=128, BN=128, TM=8, TN=8,
                                  BK=64, shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-longk-2st", dict(M=256, N=512, K=1024, dtype=2, dtype_c=4, is_atrans=0, BM=256, BN=256, TM=16, TN=16,
                                  BK=64, shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-longk-3st-at1", dict(M=512, N=256, K=1088, dtype=2, dtype_c=4, is_atrans=1, BM=256, BN=128, TM=16,
                                      TN=8, BK=64, shared_prefetch=1, reg_prefetch=1)),
    ("bf16-direct-longk-bk32", dict(M=512, N=256, K=1056, dtype=3, dtype_c=4, is_atrans=0, BM=256, BN=256, TM=16, TN=16,
                                    BK=32, shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-longk-8w", dict(M=256, N=256, K=1600, dtype=2, dtype_c=4, is_atrans=0, BM=256, BN=256, TM=8, TN=16,
                                 BK=32, shared_prefetch=1, reg_prefetch=1)),
    # the direct-staging kernel's other shapes: 32x32x16 instructions (K tile of 16), two rows of
    # matrix-core tiles per wave (the minimum of its row-streaming loop), both A layouts
    ("f16-direct-bk16-mf32", dict(M=256, N=256, K=400, dtype=2, dtype_c=4, is_atrans=0, BM=128, BN=128, TM=8, TN=8,
                                  BK=16, shared_prefetch=1, reg_prefetch=1)),
    ("bf16-direct-bk16-mf32-at1", dict(M=256, N=256, K=400, dtype=3, dtype_c=4, is_atrans=1, BM=128, BN=128, TM=8, TN=8,
                                       BK=16, shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-2rows", dict(M=192, N=128, K=736, dtype=2, dtype_c=4, is_atrans=0, BM=64, BN=64, TM=4, TN=4,
                              BK=32, shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-2rows-at1", dict(M=192, N=128, K=736, dtype=2, dtype_c=4, is_atrans=1, BM=64, BN=64, TM=4, TN=4,
                                  BK=32, shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-kt1", dict(M=256, N=256, K=64, dtype=2, dtype_c=4, is_atrans=0, BM=128, BN=128, TM=8, TN=8, BK=64,
                            shared_prefetch=1, reg_prefetch=1)),                          # a single K tile
    ("bf16-direct-kt3-at1", dict(M=256, N=256, K=96, dtype=3, dtype_c=4, is_atrans=1, BM=128, BN=128, TM=8, TN=8, BK=32,
                                 shared_prefetch=1, reg_prefetch=1)),
    # one wave per block: 32 fetch instructions per wave and tile limit the number of stages in flight
    ("f16-direct-1wave", dict(M=256, N=256, K=1088, dtype=2, dtype_c=4, is_atrans=0, BM=128, BN=128, TM=16, TN=16,
                              BK=64, shared_prefetch=1, reg_prefetch=1)),
    # edge tiles through the direct-staging kernel: partial last K tile, rows/columns beyond M and N
    ("f16-direct-ktail", dict(M=256, N=256, K=992, dtype=2, dtype_c=4, is_atrans=0, BM=128, BN=128, TM=8, TN=8, BK=64,
                              shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-32x32-1wave-at1", dict(M=96, N=160, K=288, dtype=2, dtype_c=4, is_atrans=1, BM=32, BN=32, TM=4, TN=4,
                                        BK=32, shared_prefetch=1, reg_prefetch=1)),
    ("bf16-direct-32x64-edge", dict(M=104, N=136, K=200, dtype=3, dtype_c=4, is_atrans=0, BM=32, BN=64, TM=4, TN=4,
                                    BK=64, shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-kpart", dict(M=256, N=256, K=1000, dtype=2, dtype_c=4, is_atrans=0, BM=128, BN=128, TM=8, TN=8, BK=64,
                              shared_prefetch=1, reg_prefetch=1)),
    ("bf16-direct-kpart-at1", dict(M=200, N=136, K=72, dtype=3, dtype_c=4, is_atrans=1, BM=128, BN=128, TM=8, TN=8, BK=64,
                                   shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-kpart-mf32", dict(M=256, N=256, K=408, dtype=2, dtype_c=4, is_atrans=0, BM=128, BN=128, TM=8, TN=8, BK=16,
                                   shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-edge-at1", dict(M=200, N=136, K=160, dtype=2, dtype_c=4, is_atrans=1, BM=128, BN=128, TM=8, TN=8,
                                 BK=64, shared_prefetch=1, reg_prefetch=1)),
    ("bf16-direct-256-edge", dict(M=264, N=520, K=1120, dtype=3, dtype_c=4, is_atrans=0, BM=256, BN=256, TM=16, TN=16,
                                  BK=64, shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-edge-out16", dict(M=200, N=136, K=96, dtype=2, is_atrans=0, BM=128, BN=128, TM=8, TN=8, BK=64,
                                   shared_prefetch=1, reg_prefetch=1)),
    # 16-bit output behind an edge predicate with 32x32x16 instructions: the epilogue's conversions must not
    # be scheduled in front of the wait states that follow the last matrix instruction
    ("bf16-direct-edge-out16-mf32", dict(M=40, N=128, K=48, dtype=3, dtype_c=3, is_atrans=1, BM=64, BN=128, BK=16, TM=8,
                                         TN=8, shared_prefetch=1, reg_prefetch=1)),
    ("f16-direct-edge-out16-mf32-at0", dict(M=48, N=120, K=32, dtype=2, dtype_c=2, is_atrans=0, BM=64, BN=128, BK=16,
                                            TM=8, TN=8, shared_prefetch=1, reg_prefetch=1)),
    ("bf16-at0", dict(M=256, N=256, K=128, dtype=3, dtype_c=4, is_atrans=0, BK=32)),
    ("bf16-at1-lsu2", dict(M=256, N=256, K=128, dtype=3, dtype_c=4, is_atrans=1, BK=64, lsu=2)),
]


@pytest.mark.parametrize("tag,kw", HALF_CASES, ids=[c[0] for c in HALF_CASES])
@pytest.mark.parametrize("kind", [MFMA, SIMT], ids=["mfma", "simt"])
def test_exact_small_integers_16bit(oracle, tag, kw, kind):
    """Integers in [-2,2] are exact in fp16/bf16 and sums of K <= 2048 products of them (|sum| <= 8192)
    are exact in fp32; the fp16-output cases keep K <= 256 so that their sums (<= 1024) stay exact."""
    cfg = make_config(**kw)
    M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
    lim = 2
    a = SI.small_ints((M, K), SI.STREAM_A, lim=lim)
    b = SI.small_ints((K, N), SI.STREAM_B, lim=lim)
    print(f"[case] {tag} kind={kind} {M}x{N}x{K}", flush=True)
    got, info = run_gemm(cfg, a, b, kind)
    assert info["kind"] == kind
    if "direct" in tag and kind == MFMA:
        assert info["lds_bytes"] == 0, "expected the direct-staging kernel (static LDS)"
    want = oracle.matmul(a, b, a_trans=False)
    assert not np.isnan(got).any()
    bad = np.argwhere(got != want)
    assert bad.size == 0, f"{tag}: {len(bad)} mismatches, first at {bad[:5].tolist()}"


def extra_build_configs():
    """(config, kind) pairs of the full-size tests below, so a build step can precompile them."""
    out = []
    for kind in (SIMT, MFMA):
        for at in (0, 1):
            out.append((make_config(1024, 1024, 1024, BM=64, BN=64, BK=16, TM=4, TN=4, is_atrans=at), kind))
    for kind, kw in CONFIG4_KERNELS:
        out.append((make_config(4096, 1536, 1000, **kw), kind))
    for kw in CONFIG5_KERNELS:
        out.append((make_config(4096, 4096, 4096, dtype=2, dtype_c=4, is_atrans=0, **kw), MFMA))
    bf16 = dict(_tuned("gemm_4096_fp16.json"))
    bf16["DATATYPE_A"] = bf16["DATATYPE_B"] = 3
    out.append((bf16, 0))
    out += [(cfg, MFMA) for _tag, cfg in spilling_fp64_twins()]
    out += [(make_config(*shape, **kw), MFMA) for _tag, shape, kw in LARGE_CASES]
    return out


# fp64, one wave on a 64x64x64 tile with both prefetch flags, edge tiles in M and N and a partial last K tile:
# the register-staged kernel cannot fit the register file (512 registers and scratch memory besides), and its
# build at the usual optimisation level returned wrong sums in the last block column
SPILLING_FP64_CONFIG = dict(zip(_native.keywords(), [64, 64, 64, 4, 16, 64, 1, 1, 16, 4, 2, 2, 2, 2, 2, 2, 1, 4, 2, 4, 1, 1,
                                                      0, 1, 8, 8, 8, 8, 208, 592, 0]))

# beyond the BASELINE sizes: eight times the work of config 3 / 5, extents that are no multiples of anything
LARGE_CASES = (
    ("fp16-8192", (8192, 8192, 8192), dict(dtype=2, dtype_c=4, BM=256, BN=256, TM=16, TN=16, BK=64, is_atrans=0, block_mapping=8,
                                           shared_prefetch=1, reg_prefetch=1)),
    ("bf16-odd-8191x8189x8195", (8191, 8189, 8195), dict(dtype=3, dtype_c=4, BM=256, BN=256, TM=16, TN=16, BK=32, is_atrans=0,
                                                         block_mapping=8, shared_prefetch=1, reg_prefetch=1)),
    ("fp32-odd-8190x8191x8193-at1", (8190, 8191, 8193), dict(BM=256, BN=256, TM=16, TN=8, BK=32, is_atrans=1,
                                                             block_mapping=4, shared_prefetch=1, reg_prefetch=1)),
)

CONFIG4_KERNELS = ((MFMA, dict(BM=128, BN=128, TM=8, TN=8, BK=16, shared_prefetch=1, is_atrans=0)),
                   (MFMA, dict(BM=64, BN=64, BK=32, is_atrans=1)),
                   # direct staging with a partial last K tile (1000 = 62*16 + 8)
                   (MFMA, dict(BM=128, BN=64, TM=8, TN=4, BK=16, shared_prefetch=1, reg_prefetch=1, is_atrans=0)),
                   (SIMT, dict(BM=64, BN=64, BK=8, is_atrans=0)))
CONFIG5_KERNELS = (dict(BM=128, BN=128, TM=8, TN=8, BK=32, shared_prefetch=1, reg_prefetch=1),
                   dict(BM=64, BN=64, BK=32))


def test_config1_fp32_1024_uniform(oracle):
    """BASELINE config 1: fp32 1024^3, BM=BN=64, BK=16, TM=TN=4, row-major A[M,K], uniform[-1,1)."""
    M = N = K = 1024
    a = SI.uniform((M, K), SI.STREAM_A)
    b = SI.uniform((K, N), SI.STREAM_B)
    want = oracle.matmul(a, b, a_trans=False)
    tol = fp32_tolerance(K, a, b)
    for kind in (SIMT, MFMA):
        for at in (0, 1):
            cfg = make_config(M, N, K, BM=64, BN=64, BK=16, TM=4, TN=4, is_atrans=at)
            print(f"[case] config1 kind={kind} atrans={at}", flush=True)
            got, _ = run_gemm(cfg, a, b, kind)
            err = float(np.abs(got - want).max())
            print(f"        max|err|={err:.3e} tol={tol:.3e}", flush=True)
            assert err <= tol
            assert err <= 2e-4   # far inside the contract: fp32 accumulation of 1024 terms in [-1,1]


def test_config4_fp32_edge_tiles_normal(oracle):
    """BASELINE config 4: M=4096, N=1536, K=1000, normal(0,1); a 96-row panel is checked in full
    against the oracle, plus a column-sum identity over the whole output."""
    M, N, K = 4096, 1536, 1000
    a = SI.normal((M, K), SI.STREAM_A)
    b = SI.normal((K, N), SI.STREAM_B)
    rows = (2000, 2096)
    want = oracle.matmul(a, b, a_trans=False, rows=rows)
    tol = fp32_tolerance(K, a, b)
    for kind, kw in CONFIG4_KERNELS:
        cfg = make_config(M, N, K, **kw)
        print(f"[case] config4 kind={kind} {kw}", flush=True)
        got, _ = run_gemm(cfg, a, b, kind)
        assert not np.isnan(got).any()
        err = float(np.abs(got[rows[0]:rows[1]] - want).max())
        print(f"        panel max|err|={err:.3e} tol={tol:.3e}", flush=True)
        assert err <= tol
        # size-independent property: 1^T (A B) == (1^T A) B, evaluated in float64
        lhs = got.astype(np.float64).sum(axis=0)
        rhs = a.astype(np.float64).sum(axis=0) @ b.astype(np.float64)
        assert np.abs(lhs - rhs).max() <= tol * np.sqrt(M)


def test_config5_fp16_4096(oracle):
    """BASELINE config 5: fp16 inputs, fp32 accumulate/output, 4096^3, normal(0,0.5) rounded to fp16;
    the oracle runs on the upcast values.  Bar: <= 2e-2 relative (to the RMS magnitude of C)."""
    M = N = K = 4096
    a = quantize(SI.normal((M, K), SI.STREAM_A, std=0.5), 2)
    b = quantize(SI.normal((K, N), SI.STREAM_B, std=0.5), 2)
    rows = (1024, 1088)
    want = oracle.matmul(a, b, a_trans=False, rows=rows)
    scale = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    cfgs = [("tuned", dict(_tuned("gemm_4096_fp16.json")))]        # the kernel bench.py launches
    cfgs += [(str(kw), make_config(M, N, K, dtype=2, dtype_c=4, is_atrans=0, **kw)) for kw in CONFIG5_KERNELS]
    for kw, cfg in cfgs:
        print(f"[case] config5 {kw}", flush=True)
        got, _ = run_gemm(cfg, a, b, MFMA)
        assert not np.isnan(got).any()
        err = float(np.abs(got[rows[0]:rows[1]] - want).max())
        print(f"        panel max|err|={err:.3e} scale={scale:.3e} rel={err / scale:.3e}", flush=True)
        assert err / scale <= 2e-2
        lhs = got.astype(np.float64).sum(axis=0)
        rhs = a.astype(np.float64).sum(axis=0) @ b.astype(np.float64)
        assert np.abs(lhs - rhs).max() <= 2e-2 * scale * np.sqrt(M)


def test_config5_bf16_4096(oracle):
    """The config-5 workload with bfloat16 inputs (DATATYPE 3): normal(0, 0.5) rounded to bf16, fp32
    accumulate/output, the tuned kernel bench.py launches; the oracle runs on the upcast values.
    Bar: <= 2e-2 relative (to the RMS magnitude of C), plus the column-sum identity over the whole output."""
    M = N = K = 4096
    a = quantize(SI.normal((M, K), SI.STREAM_A, std=0.5), 3)
    b = quantize(SI.normal((K, N), SI.STREAM_B, std=0.5), 3)
    rows = (2048, 2112)
    want = oracle.matmul(a, b, a_trans=False, rows=rows)
    scale = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    cfg = dict(_tuned("gemm_4096_fp16.json"))
    cfg["DATATYPE_A"] = cfg["DATATYPE_B"] = 3
    print("[case] config5 with bf16 inputs, tuned kernel", flush=True)
    got, info = run_gemm(cfg, a, b, MFMA)
    assert info["lds_bytes"] == 0          # the direct-staging kernel
    assert not np.isnan(got).any()
    err = float(np.abs(got[rows[0]:rows[1]] - want).max())
    print(f"        panel max|err|={err:.3e} scale={scale:.3e} rel={err / scale:.3e}", flush=True)
    assert err / scale <= 2e-2
    lhs = got.astype(np.float64).sum(axis=0)
    rhs = a.astype(np.float64).sum(axis=0) @ b.astype(np.float64)
    assert np.abs(lhs - rhs).max() <= 2e-2 * scale * np.sqrt(M)


def _tuned(name):
    import json
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(os.path.join(root, "codegendemo_amd", "TunedConfigs", name)) as f:
        return json.load(f)["cfgs"][0]


@pytest.mark.parametrize("which", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("hiprtc", hiprtc_params())
def test_tuned_4096_kernels_are_bit_exact_on_integers(oracle, which, hiprtc):
    """The kernels bench.py launches (all 256 CUs busy, every stage of the K loop under real memory
    latency), on integers in [-2, 2]: sums of 4096 products (<= 16384) are exact in fp32, so the whole
    4096 x 4096 result must equal the oracle bit for bit whatever the summation order."""
    cfg = dict(_tuned("gemm_4096_fp32.json" if which == "fp32" else "gemm_4096_fp16.json"))
    if which == "bf16":
        cfg["DATATYPE_A"] = cfg["DATATYPE_B"] = 3
    M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
    a = SI.small_ints((M, K), SI.STREAM_A, lim=2)
    b = SI.small_ints((K, N), SI.STREAM_B, lim=2)
    print(f"[case] tuned {which} {M}x{N}x{K} hiprtc={hiprtc}", flush=True)
    got, info = run_gemm(cfg, a, b, hiprtc=hiprtc)
    assert info["lds_bytes"] == 0          # the direct-staging kernel
    want = oracle.matmul(a, b, a_trans=False)
    assert not np.isnan(got).any()
    bad = np.argwhere(got != want)
    assert bad.size == 0, f"tuned {which}: {len(bad)} mismatches, first at {bad[:5].tolist()}"


def test_config3_fp32_4096_uniform(oracle):
    """BASELINE config 3: fp32 4096^3, row-major A[M,K], uniform[-1,1), the tuned kernel bench.py launches:
    a 64-row panel in full against the oracle, plus the column-sum identity over the whole output."""
    cfg = dict(_tuned("gemm_4096_fp32.json"))
    M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
    a = SI.uniform((M, K), SI.STREAM_A)
    b = SI.uniform((K, N), SI.STREAM_B)
    rows = (3000, 3064)
    want = oracle.matmul(a, b, a_trans=False, rows=rows)
    tol = fp32_tolerance(K, a, b)
    print("[case] config3 tuned fp32 4096^3", flush=True)
    got, _ = run_gemm(cfg, a, b)
    assert not np.isnan(got).any()
    err = float(np.abs(got[rows[0]:rows[1]] - want).max())
    print(f"        panel max|err|={err:.3e} tol={tol:.3e}", flush=True)
    assert err <= tol
    assert err <= 1e-3                       # far inside the contract
    lhs = got.astype(np.float64).sum(axis=0)
    rhs = a.astype(np.float64).sum(axis=0) @ b.astype(np.float64)
    assert np.abs(lhs - rhs).max() <= tol * np.sqrt(M)


@pytest.mark.parametrize("index", range(5))
@pytest.mark.parametrize("hiprtc", hiprtc_params())
def test_tuned_edge_shape_kernels_are_bit_exact_on_integers(oracle, index, hiprtc):
    """The five best configs of the 4096 x 1536 x 1000 sweep (768 or more blocks, two of them resident per
    compute unit, a partial last K tile): integers in [-2, 2] give sums that are exact in fp32, so the whole
    result must equal the oracle bit for bit."""
    import json
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(os.path.join(root, "codegendemo_amd", "TunedConfigs", "gemm_4096x1536x1000_fp32.json")) as f:
        cfg = json.load(f)["cfgs"][index]
    M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
    a = SI.small_ints((M, K), SI.STREAM_A, lim=2)
    b = SI.small_ints((K, N), SI.STREAM_B, lim=2)
    print(f"[case] tuned edge shape #{index} {M}x{N}x{K} hiprtc={hiprtc}", flush=True)
    got, _ = run_gemm(cfg, a, b, hiprtc=hiprtc)
    want = oracle.matmul(a, b, a_trans=False)
    assert not np.isnan(got).any()
    bad = np.argwhere(got != want)
    assert bad.size == 0, f"tuned edge config {index}: {len(bad)} mismatches, first at {bad[:5].tolist()}"


def spilling_fp64_twins():
    """The config whose -O3 build returned wrong sums, and its neighbours (other extents in M, N and K: with or
    without edge tiles, with or without a partial last K tile).  The neighbours were right at -O3; all of them run
    out of registers, so all of them are handed out as -O1 rebuilds, and must be right."""
    out = [("M8-N208-K592", SPILLING_FP64_CONFIG)]
    for tag, (m, n, k) in (("M64-N192-K592", (64, 192, 592)), ("M8-N208-K640", (8, 208, 640)), ("M40-N144-K200", (40, 144, 200))):
        out.append((tag, dict(SPILLING_FP64_CONFIG, M_SIZE=m, N_SIZE=n, K_SIZE=k)))
    return out


@pytest.mark.parametrize("hiprtc", hiprtc_params())
def test_kernel_that_needs_scratch_memory_is_exact(oracle, hiprtc):
    """A register-staged kernel whose first build runs out of registers is built again at a lower optimisation
    level by the engine; the kernel it hands out says so (build flag), is bit-exact on integers and still reports
    its scratch use.  The cause of the wrong -O3 build is unknown: this test guards the workaround, under both
    compilers, on the failing config and its neighbours."""
    from tests.gemm_helpers import build_kernel
    for tag, cfg in spilling_fp64_twins():
        kpm, ui, kernel, info = build_kernel(cfg, MFMA, hiprtc=hiprtc)
        assert info["kind"] == MFMA and info["lds_bytes"] > 0          # register staging: fp64 has no direct-staging form
        assert info["low_opt"] and info["build_flags"] & _native.BUILD_LOW_OPT and ui.m_buildFlags & _native.BUILD_LOW_OPT
        assert kernel.n_spills > 0 and info["scratch_bytes"] == 4 * kernel.n_spills
        kernel.unload()
        M, N, K = cfg["M_SIZE"], cfg["N_SIZE"], cfg["K_SIZE"]
        a = SI.small_ints((M, K), SI.STREAM_A, lim=2)
        b = SI.small_ints((K, N), SI.STREAM_B, lim=2)
        print(f"[case] spilling fp64 {tag} hiprtc={hiprtc}", flush=True)
        got, _ = run_gemm(cfg, a, b, MFMA, hiprtc=hiprtc)
        want = a.astype(np.float64) @ b.astype(np.float64)
        assert np.array_equal(got, want), f"{tag}: {int((got != want).sum())} wrong elements"
        assert np.array_equal(want[:8].astype(np.float32), oracle.matmul(a, b, a_trans=False, rows=(0, 8)))


@pytest.mark.parametrize("tag,shape,kw", LARGE_CASES, ids=[c[0] for c in LARGE_CASES])
def test_large_problems_are_exact_on_integers(oracle, tag, shape, kw):
    """Problems of eight times the BASELINE work through the direct-staging kernel (row and tile offsets beyond
    2^25 elements, 16 times the blocks of the tuned launch).  Operands are integers in [-2, 2] drawn on the device, so
    every sum is exact in fp32 whatever the order: the whole result must equal the exact product bit for bit — taken
    from an fp64 product on the device, which is exact as well (an independent route: the vendor library) — and a
    row panel of it the CPU oracle's."""
    import torch
    from tests.gemm_helpers import build_kernel
    M, N, K = shape
    cfg = make_config(M, N, K, **kw)
    kpm, ui, kernel, info = build_kernel(cfg, MFMA)
    assert info["lds_bytes"] == 0, "expected the direct-staging kernel"
    g = torch.Generator(device="cuda:0").manual_seed(20251127)
    ta = kpm.dtypeTorch('A')
    a = torch.randint(-2, 3, (M, K), device="cuda:0", generator=g).to(ta)
    b = torch.randint(-2, 3, (K, N), device="cuda:0", generator=g).to(ta)
    a_op = a.t().contiguous() if kpm.isATranspose else a
    c = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda:0")
    print(f"[case] large {tag} {M}x{N}x{K}", flush=True)
    kernel.run(a_op, b, c)
    torch.cuda.synchronize()
    want = torch.matmul(a.to(torch.float64), b.to(torch.float64))
    bad = int((c.to(torch.float64) != want).sum().item())          # NaN (never written) counts as different
    assert bad == 0, f"{tag}: {bad} elements differ from the exact product"
    rows = [0, 1, M // 2, M - 2, M - 1]
    panel = oracle.matmul(a[rows].to(torch.float32).cpu().numpy(), b.to(torch.float32).cpu().numpy(), a_trans=False)
    assert np.array_equal(c[rows].cpu().numpy(), panel)
    kernel.unload()
