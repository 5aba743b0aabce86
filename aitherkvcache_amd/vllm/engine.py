"""Cache-tensor arithmetic of the serving integration: page size, row width, page alignment and
the PRIMARY uint8 layout, as the reference's engine patches compute them
(aither_kvcache/vllm/engine.py:110-154 and :223-392).  Pure functions over sizes and one raw
byte buffer; nothing here imports vLLM or patches it.
"""
from typing import Tuple

import torch

from .kv_cache_dtype import CacheFormat, tq_dim_for_head


def tq_page_size_bytes(block_size: int, num_kv_heads: int, head_size: int, fmt: CacheFormat) -> int:
    """Bytes of one cache page (K and V of block_size tokens); uniform rows are codes + 4 reserved
    bytes, hybrid rows carry their norms (reference: engine.py:110-122)."""
    return 2 * block_size * num_kv_heads * tq_dim_for_head(head_size, fmt)


def align_page_size(raw_bytes: int) -> int:
    """Next power of two >= raw_bytes (unchanged when <= 0): page sizes of layers with different
    head sizes then divide one another (reference: engine.py:136-154)."""
    if raw_bytes <= 0:
        return raw_bytes
    return 1 << (raw_bytes - 1).bit_length()


def reshape_primary(raw: torch.Tensor, num_blocks: int, block_size: int, num_kv_heads: int,
                    head_size: int, fmt: CacheFormat) -> torch.Tensor:
    """View a layer's raw cache bytes as uint8 [num_blocks, 2, block_size, num_kv_heads, tq_dim]
    (reference: engine.py:340-375).  Raises ValueError when the buffer is too small; bytes beyond
    the layout (page padding at the end of the buffer) are left out of the view."""
    tq_dim = tq_dim_for_head(head_size, fmt)
    need = num_blocks * 2 * block_size * num_kv_heads * tq_dim
    flat = raw.reshape(-1).view(torch.uint8)
    if flat.numel() < need:
        raise ValueError(f"raw cache tensor holds {flat.numel()} bytes, the layout needs {need} "
                         f"({num_blocks} blocks x 2 x {block_size} x {num_kv_heads} heads x {tq_dim})")
    return flat[:need].view(num_blocks, 2, block_size, num_kv_heads, tq_dim)


def primary_views(kv_cache: torch.Tensor, head_size: int, fmt: CacheFormat) -> Tuple[torch.Tensor, torch.Tensor]:
    """(k_rows, v_rows): strided uint8 views [num_blocks, block_size, num_kv_heads, packed] of a
    PRIMARY cache tensor, the form the encode and attention entry points take (they honour the
    strides; the 4 reserved bytes of a uniform row are skipped by the row pitch)."""
    if kv_cache.dim() != 5 or kv_cache.shape[1] != 2 or kv_cache.dtype != torch.uint8:
        raise ValueError("kv_cache must be uint8 [num_blocks, 2, block_size, num_kv_heads, tq_dim]")
    tq_dim = tq_dim_for_head(head_size, fmt)
    if kv_cache.shape[-1] != tq_dim:
        raise ValueError(f"kv_cache rows are {kv_cache.shape[-1]} bytes, {tq_dim} expected for this format")
    packed = tq_dim if fmt.kind == "hybrid" else tq_dim - 4
    return kv_cache[:, 0, :, :, :packed], kv_cache[:, 1, :, :, :packed]
