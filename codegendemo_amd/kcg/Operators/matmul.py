"""Python operator API of the GEMM: the tuning-config record and the tuning-space predicates.

Counterpart of Runtime/python/kcg/Operators/matmul.py in the reference: KernelArgMatmul (:75-246),
getMatmulSignature (:61-72) and TuningSpaceChecker_Matmul (:249-313).  The 31 fields, their JSON keys
and the predicates are the reference's; the field list itself is driven by the native keyword table
so the ABI order (src/main.cc:64-96) exists in one place.
"""
from ..Utils import ConfigKeywords, EnumKernelDType, ToTorchType, get_dtype_from_int, sizeof
from ... import _native

# keyword -> attribute name on KernelArgMatmul (everything else: attribute == keyword)
_FIELD_OF = {"M_SIZE": "M", "N_SIZE": "N", "K_SIZE": "K", "IS_ATRANS": "isATranspose",
             "DATATYPE_A": "_dtA", "DATATYPE_B": "_dtB", "DATATYPE_C": "_dtC"}

_DEFAULTS = {
    "BLOCK_SIZE_M": 64, "BLOCK_SIZE_N": 64, "BLOCK_SIZE_K": 16, "THREAD_SIZE_M": 4, "THREAD_SIZE_N": 4,
    "WARP_SIZE": 64, "BLOCK_LAYOUT_M": 4, "BLOCK_LAYOUT_N": 1, "WARP_LAYOUT_M": 16, "WARP_LAYOUT_N": 4,
    "IS_ATRANS": 1, "UNROLL_NUM": 1,
}  # every other tuning field defaults to 0, as in the reference constructor (matmul.py:77-108)


def getMatmulSignature(dtypeA, dtypeB, dtypeC) -> dict:
    """Kernel signature {arg index: '*<type>'}: three global pointers (Kernel.py:152-188,228-238).
    Depends on the dtypes only; unlike the reference no device tensors are allocated to find out."""
    import torch
    names = {torch.float16: "fp16", torch.bfloat16: "bf16", torch.float32: "fp32", torch.float64: "fp64"}
    return {i: "*" + names[t] for i, t in enumerate((dtypeA, dtypeB, dtypeC))}


class KernelArgMatmul:
    def __init__(self, m, n, k, typeA, typeB, typeC):
        for kw in ConfigKeywords.ORDER:
            setattr(self, _FIELD_OF.get(kw, kw), _DEFAULTS.get(kw, 0))
        self._dtA, self._dtB, self._dtC = int(typeA), int(typeB), int(typeC)
        self.M, self.N, self.K = m, n, k

    # ---- JSON round trip (matmul.py:110-177) --------------------------------------------------
    def jsonfy(self):
        return {kw: int(getattr(self, _FIELD_OF.get(kw, kw))) for kw in _json_order()}

    def assignWithJson(self, jsonObj):
        for kw in ConfigKeywords.ORDER:
            v = jsonObj[kw]
            if kw == "IS_ATRANS":
                v = int(v > 0)
            setattr(self, _FIELD_OF.get(kw, kw), int(v))

    # ---- the ABI view --------------------------------------------------------------------------
    def values(self):
        """The 31 integers in compile_kernel_matmul order."""
        return [int(getattr(self, _FIELD_OF.get(kw, kw))) for kw in ConfigKeywords.ORDER]

    def check(self):
        """Config validity.  The reference asserts tile/layout consistency and an LDS bound
        (matmul.py:180-194); here the native predicate decides (which also covers the divisibility
        rules the reference schedule assumes silently), raising InvalidConfigError with the reason.
        Problem sizes need not be multiples of the block tile."""
        _native.check_config(self.values())

    def dtype(self, index: str):
        return {"A": self._dtA, "B": self._dtB, "C": self._dtC}[index]

    def dtypeTorch(self, index: str):
        return ToTorchType(self.dtype(index))

    def __str__(self):
        body = " ,\n".join(f' "{k}" :  {v}' for k, v in self.jsonfy().items())
        return "{\n" + body + " \n}"

    def __eq__(self, other):
        return isinstance(other, KernelArgMatmul) and self.values() == other.values()

    def __hash__(self):
        return hash(tuple(self.values()))


def _json_order():
    """Key order of jsonfy() in the reference (matmul.py:111-143): dtypes, sizes and IS_ATRANS sit
    after the warp layout, ahead of the load widths."""
    o = list(ConfigKeywords.ORDER)
    tail = [k for k in o if k in ("DATATYPE_A", "DATATYPE_B", "DATATYPE_C", "M_SIZE", "N_SIZE", "K_SIZE", "IS_ATRANS")]
    head = [k for k in o if k not in tail]
    at = head.index("WARP_LAYOUT_N") + 1
    return head[:at] + tail + head[at:]


def kernelArgFromConfig(config: dict) -> KernelArgMatmul:
    """One entry of a {"cfgs": [...]} file -> KernelArgMatmul (KCGTask.py:381-422)."""
    kw = ConfigKeywords
    arg = KernelArgMatmul(config[kw.KEY_M], config[kw.KEY_N], config[kw.KEY_K],
                          config[kw.KEY_DTYPE_A], config[kw.KEY_DTYPE_B], config[kw.KEY_DTYPE_C])
    arg.assignWithJson(config)
    return arg


# gfx950: 160 KiB of LDS per CU and a workgroup may use all of it.  The reference pruned at 16 KiB
# (`< 16384`, matmul.py:258), which rejects even its own 64x64 fp32 tiles.
LDS_LIMIT_BYTES = 160 * 1024


class TuningSpaceChecker_Matmul:
    @staticmethod
    def check_shm_size(config: dict) -> bool:
        """LDS bound of a tuning-space point; on success the single DATATYPE_C entry is expanded to
        DATATYPE_A/B/C like the reference does (matmul.py:251-265)."""
        kw = ConfigKeywords
        dtypeC = config[kw.KEY_DTYPE_C]
        nbytes = sizeof(get_dtype_from_int(config.get(kw.KEY_DTYPE_A, dtypeC)))   # operands live in LDS
        bm, bn, bk = config[kw.KEY_BLOCK_SIZE_M], config[kw.KEY_BLOCK_SIZE_N], config[kw.KEY_BLOCK_SIZE_K]
        lsu = config[kw.KEY_LOCAL_SPLIT_U]
        stages = 2 if config.get(kw.KEY_SHARED_PREFETCH, 0) else 1
        operands = (bm + bn) * bk * nbytes * stages
        partials = bm * bn * 4 * lsu if lsu > 1 else 0
        if max(operands, partials) <= LDS_LIMIT_BYTES:
            config.setdefault(kw.KEY_DTYPE_A, dtypeC)
            config.setdefault(kw.KEY_DTYPE_B, dtypeC)
            return True
        return False

    @staticmethod
    def check_warp(config: dict) -> bool:
        kw = ConfigKeywords
        return config[kw.KEY_WARP_LAYOUT_M] * config[kw.KEY_WARP_LAYOUT_N] == config[kw.KEY_WARP_SIZE]

    @staticmethod
    def check_size(config: dict, allow_edge_tiles: bool = True) -> bool:
        """Tile/layout consistency and scatter widths (matmul.py:277-313).  The reference also
        requires M%BM == N%BN == K%BK == 0; this engine predicates edge tiles, so that part is
        applied only with allow_edge_tiles=False."""
        kw = ConfigKeywords
        bm, bn, bk = config[kw.KEY_BLOCK_SIZE_M], config[kw.KEY_BLOCK_SIZE_N], config[kw.KEY_BLOCK_SIZE_K]
        if not allow_edge_tiles:
            if config[kw.KEY_M] % bm or config[kw.KEY_N] % bn or config[kw.KEY_K] % bk:
                return False
        if config[kw.KEY_BLOCK_LAYOUT_M] * config[kw.KEY_WARP_LAYOUT_M] * config[kw.KEY_THREAD_SIZE_M] != bm:
            return False
        if config[kw.KEY_BLOCK_LAYOUT_N] * config[kw.KEY_WARP_LAYOUT_N] * config[kw.KEY_THREAD_SIZE_N] != bn:
            return False
        wa, wb = config[kw.KEY_WARP_SCATTER_WIDTH_A], config[kw.KEY_WARP_SCATTER_WIDTH_B]
        ta, tb = config[kw.KEY_THREAD_SCATTER_WIDTH_A], config[kw.KEY_THREAD_SCATTER_WIDTH_B]
        if wa < ta or wb < tb:
            return False
        if wa % ta or wb % tb:
            return False
        return True

    @staticmethod
    def check_engine(config: dict) -> bool:
        """Everything the kernel templates need (native predicate); a point that passes compiles."""
        values = [int(config[k]) for k in ConfigKeywords.ORDER]
        return _native.is_valid_config(values)
