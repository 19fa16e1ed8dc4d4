"""Tuning-space generation: {KEY: [values…]} file -> validated {"cfgs": [...]} combinations -> sub-JSONs.

Counterpart of Runtime/python/kcg/ConfigGenerator.py.  The reference's `config_gen` (:94-126) calls
`get_cfgs`, `read_params` and `getTempJsonFileName`, none of which exist in that snapshot; their
behaviour here follows the README (cartesian product of the per-key value lists, pruned by the
TuningSpaceChecker_Matmul predicates) and the file names the reference's debug comments show
(`tmp_json_<start>_<end>.json`, testGetKernels.py:17).  Pruning happens while enumerating, and the
engine's own validity predicate is part of it, so every emitted point compiles.
"""
import itertools
import json
import os

from .Operators.matmul import TuningSpaceChecker_Matmul
from .Utils import ConfigKeywords, PathManager


def read_params(path: str) -> dict:
    with open(path, "r") as f:
        return json.load(f)


def save_to_json(obj, output_file="config_combinations.json"):
    with open(output_file, "w") as f:
        json.dump(obj, f, indent=4)


def getTempJsonFileName(startIndex: int, endIndex: int, outDir: str) -> str:
    return f"{outDir}/tmp_json_{startIndex}_{endIndex}.json"


def _expand_dtype(config: dict) -> dict:
    kw = ConfigKeywords
    c = dict(config)
    if kw.KEY_DTYPE_C in c:
        c.setdefault(kw.KEY_DTYPE_A, c[kw.KEY_DTYPE_C])
        c.setdefault(kw.KEY_DTYPE_B, c[kw.KEY_DTYPE_C])
    return c


def iter_cfgs(param_options: dict, engine_check: bool = True, stats: dict = None):
    """Yield every valid combination of a tuning-space description."""
    keys = list(param_options.keys())
    values = [v if isinstance(v, (list, tuple)) else [v] for v in param_options.values()]
    chk = TuningSpaceChecker_Matmul
    n_total = n_ok = 0
    for combo in itertools.product(*values):
        n_total += 1
        cfg = _expand_dtype(dict(zip(keys, combo)))
        if not (chk.check_warp(cfg) and chk.check_size(cfg) and chk.check_shm_size(cfg)):
            continue
        if engine_check and not chk.check_engine(cfg):
            continue
        n_ok += 1
        yield cfg
    if stats is not None:
        stats["enumerated"] = n_total
        stats["valid"] = n_ok


def get_cfgs(tuning_cfg_file: str, engine_check: bool = True) -> list:
    return list(iter_cfgs(read_params(tuning_cfg_file), engine_check))


def sample_cfgs(param_options: dict, n: int, seed: int, max_draws: int = 2000000):
    """A seeded sample of what get_cfgs returns for a tuning space too large to enumerate (the reference's
    GEMM_configs_1024.json spans some 10^8 raw points): points are drawn uniformly from the cartesian product
    and pass through the same predicates as iter_cfgs.  Returns (valid, rejected): `valid` holds n points that
    pass everything (each of them compiles); `rejected` the first n raw points that did not (the reference's
    checker or the engine's predicate said no: the engine answers those with KCG_ERR_INVALID_CONFIG)."""
    import random
    rng = random.Random(seed)
    keys = list(param_options.keys())
    values = [v if isinstance(v, (list, tuple)) else [v] for v in param_options.values()]
    chk = TuningSpaceChecker_Matmul
    valid, rejected, seen = [], [], set()
    for _ in range(max_draws):
        if len(valid) >= n:
            break
        combo = tuple(rng.choice(v) for v in values)
        if combo in seen:
            continue
        seen.add(combo)
        cfg = _expand_dtype(dict(zip(keys, combo)))
        if chk.check_warp(cfg) and chk.check_size(cfg) and chk.check_shm_size(cfg) and chk.check_engine(cfg):
            valid.append(cfg)
        elif len(rejected) < n:
            rejected.append(cfg)
    return valid, rejected


def split_bigjson_to_temp(bigcfgs: dict, startIndex: int, endIndex: int, outDir: str) -> str:
    outDir = outDir.rstrip("/")
    part = {"cfgs": bigcfgs["cfgs"][startIndex:endIndex]}
    filename = getTempJsonFileName(startIndex, endIndex, outDir)
    save_to_json(part, filename)
    return filename


def config_gen(tuning_cfg_file: str, preGeneratedJson: str, singleLength: int, cacheTuningSPaceFile: str,
               splitBigJson=True):
    """-> (list of sub-JSON paths, number of configs); same contract as ConfigGenerator.py:94-126."""
    if preGeneratedJson:
        combs = read_params(preGeneratedJson)
    else:
        combs = {"cfgs": get_cfgs(tuning_cfg_file)}
        if cacheTuningSPaceFile:
            with open(cacheTuningSPaceFile, "w") as f:
                json.dump(combs, f)
    items = combs["cfgs"]
    names = []
    if splitBigJson:
        os.makedirs(PathManager.tmp_dir(), exist_ok=True)
        for i in range(0, len(items), singleLength):
            names.append(split_bigjson_to_temp(combs, i, i + singleLength, PathManager.tmp_dir()))
    return names, len(items)


def make_config(M, N, K, BM=64, BN=64, BK=16, TM=4, TN=4, dtype=4, dtype_c=None, is_atrans=1,
                warp_layout=(8, 8), lsu=1, glw=None, shared_prefetch=0, reg_prefetch=0,
                load_continuous=1, reduce_c_continuous=1, block_mapping=8, scatter=None, gsw=None, unroll=4):
    """One complete config dict from the handful of parameters people actually choose; the layout
    fields are derived (BLOCK_LAYOUT = BLOCK_SIZE / (THREAD_SIZE * WARP_LAYOUT)).  Raises ValueError
    when the tile cannot be laid out with the given warp layout."""
    kw = ConfigKeywords
    wlm, wln = warp_layout
    if BM % (TM * wlm) or BN % (TN * wln):
        raise ValueError(f"tile {BM}x{BN} is not a multiple of thread tile x warp layout ({TM * wlm}x{TN * wln})")
    esz = {2: 2, 3: 2, 4: 4, 8: 8}[dtype]
    if glw is None:
        glw = min(16 // esz, 4 if esz >= 4 else 8)
    sa = scatter if scatter is not None else min(TM, 4)
    sb = scatter if scatter is not None else min(TN, 4)
    return {
        kw.KEY_BLOCK_SIZE_M: BM, kw.KEY_BLOCK_SIZE_N: BN, kw.KEY_BLOCK_SIZE_K: BK,
        kw.KEY_THREAD_SIZE_M: TM, kw.KEY_THREAD_SIZE_N: TN, kw.KEY_WARP_SIZE: 64,
        kw.KEY_BLOCK_LAYOUT_M: BM // (TM * wlm), kw.KEY_BLOCK_LAYOUT_N: BN // (TN * wln),
        kw.KEY_WARP_LAYOUT_M: wlm, kw.KEY_WARP_LAYOUT_N: wln,
        kw.KEY_DTYPE_A: dtype, kw.KEY_DTYPE_B: dtype, kw.KEY_DTYPE_C: dtype if dtype_c is None else dtype_c,
        kw.KEY_M: M, kw.KEY_N: N, kw.KEY_K: K, kw.KEY_IS_A_TRANSPOSE: int(is_atrans),
        kw.KEY_GLOB_LOAD_WIDTH_A: glw, kw.KEY_GLOB_LOAD_WIDTH_B: glw,
        kw.KEY_WARP_SCATTER_WIDTH_A: sa, kw.KEY_WARP_SCATTER_WIDTH_B: sb,
        kw.KEY_THREAD_SCATTER_WIDTH_A: sa, kw.KEY_THREAD_SCATTER_WIDTH_B: sb,
        kw.KEY_LOCAL_SPLIT_U: lsu, kw.KEY_BLOCK_MAPPING: block_mapping,
        kw.KEY_GLOB_STORE_WIDTH: gsw if gsw is not None else min(4, 16 // esz),
        kw.KEY_UNROLL_NUM: unroll, kw.KEY_REG_PREFETCH: int(reg_prefetch), kw.KEY_SHARED_PREFETCH: int(shared_prefetch),
        kw.KEY_LOAD_CONTINUOUS: int(load_continuous), kw.KEY_REDUCE_C_CONTINUOUS: int(reduce_c_continuous),
    }


def sweep_grid_points(param_options: dict):
    """One config per point of the (BM, BN, BK, TM, TN, SHARED_PREFETCH, REG_PREFETCH) grid of a
    tuning space: the first block/warp layout (in file order) that the engine accepts.  Returns
    (configs, skipped) where skipped lists the grid points no layout can realise (e.g. a 32x32 tile
    with 8x8 thread tiles has 16 threads, less than one wave) — skipped, not failed."""
    kw = ConfigKeywords
    grid_keys = [kw.KEY_BLOCK_SIZE_M, kw.KEY_BLOCK_SIZE_N, kw.KEY_BLOCK_SIZE_K, kw.KEY_THREAD_SIZE_M,
                 kw.KEY_THREAD_SIZE_N, kw.KEY_SHARED_PREFETCH, kw.KEY_REG_PREFETCH]
    seen, skipped = {}, []
    opts = {k: (v if isinstance(v, (list, tuple)) else [v]) for k, v in param_options.items()}
    for point in itertools.product(*[opts[k] for k in grid_keys]):
        fixed = dict(opts)
        for k, v in zip(grid_keys, point):
            fixed[k] = [v]
        first = next(iter_cfgs(fixed), None)
        if first is None:
            skipped.append(dict(zip(grid_keys, point)))
        else:
            seen[point] = first
    return list(seen.values()), skipped
