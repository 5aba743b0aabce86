"""`--kv-cache-dtype` names of the TurboQuant cache formats (the reference documents them at
README.md:94-110 and selects the mode through AITHER_TQ_MODE / AITHER_TQ_BITS)."""
from typing import NamedTuple, Optional


class CacheFormat(NamedTuple):
    kind: str             # "uniform" or "hybrid"
    bits: Optional[int]   # uniform: 4 / 3 / 2
    mode: Optional[str]   # hybrid: "tq35" or "tq25"
    packed_bytes_d128: int
    norms_in_row: bool


KV_CACHE_DTYPES = {
    "tq-t4nc": CacheFormat("uniform", 4, None, 64, False),
    "tq-t3nc": CacheFormat("uniform", 3, None, 48, False),
    "tq-t2nc": CacheFormat("uniform", 2, None, 32, False),
    "tq-t35nc": CacheFormat("hybrid", None, "tq35", 64, True),
    "tq35": CacheFormat("hybrid", None, "tq35", 64, True),
    "tq25": CacheFormat("hybrid", None, "tq25", 44, True),
}


def resolve_kv_cache_dtype(name: str) -> CacheFormat:
    try:
        return KV_CACHE_DTYPES[name.lower()]
    except KeyError:
        raise ValueError(f"unknown TurboQuant kv-cache dtype {name!r}; known: {sorted(KV_CACHE_DTYPES)}")


def tq_dim_for_head(head_size: int, fmt: CacheFormat) -> int:
    """Bytes per (token, head) row of the serving cache tensor: uniform formats reserve 4 spare
    bytes after the codes (the norms live in separate float32 tensors), hybrid rows carry their
    norms (reference: aither_kvcache/vllm/engine.py:125-133)."""
    if fmt.kind == "hybrid":
        from ..hybrid_quantizer import HybridTurboQuant
        return HybridTurboQuant.packed_dim_for_mode(head_size, fmt.mode)
    from ..packing import packed_size
    return packed_size(head_size, fmt.bits) + 4
