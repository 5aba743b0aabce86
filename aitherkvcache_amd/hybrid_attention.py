"""Encode-on-write and paged decode attention for the hybrid (tq35 / tq25) cache.

The reference has no fused path for hybrid data: its tq::hybrid_decode_step
(aither_kvcache/vllm/hooks.py:240-345) encodes the new token, decompresses every block the
batch addresses with HybridTurboQuant.decode and runs dense SDPA.  Here the same attention
(softmax(q K^T * scale) V over the decoded rows) is computed directly on the packed rows (64 bytes
for tq35, 44 for tq25) by one kernel sequence, and the new token is written by one scatter kernel.
Cache tensors are uint8 [num_blocks, block_size, num_kv_heads, >= packed_dim] (norms are inside the
rows); strided views with 4-byte aligned rows are accepted.
"""
from typing import Optional

import torch

from . import _lib


def hybrid_encode_and_store(htq, x: torch.Tensor, slot_mapping: torch.Tensor, cache: torch.Tensor,
                            block_size: int = 16, max_blocks: int = 0) -> None:
    """Write x [num_tokens, num_kv_heads, 128] into cache[blk, pos, head, :packed_dim] for
    slot = blk * block_size + pos; negative slots and blocks >= max_blocks are skipped."""
    if max_blocks == 0:
        max_blocks = cache.shape[0]
    num_tokens, num_kv_heads, head_dim = x.shape
    if num_tokens == 0:
        return
    table = htq.kernel_table
    dev = _lib.require_gpu(x, slot_mapping, cache, table)
    if cache.dtype != torch.uint8 or cache.stride(-1) != 1 or cache.shape[-1] < htq.packed_dim:
        raise ValueError(f"cache must be uint8 with contiguous rows of >= {htq.packed_dim} bytes")
    if head_dim != htq.head_dim:
        raise ValueError(f"head_dim {head_dim} != {htq.head_dim}")
    if x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        x = x.float()
    x = htq.to_group_order(x, head_axis=1)        # (a variance-ranked split: coordinates into group order first)
    if x.stride(-1) != 1:
        x = x.contiguous()
    slots = slot_mapping if slot_mapping.is_contiguous() else slot_mapping.contiguous()
    _lib.check(getattr(_lib.lib(), htq._abi + "_encode_paged")(
        x.data_ptr(), _lib.dtype_code(x), num_tokens, num_kv_heads, x.stride(0), x.stride(1),
        slots.data_ptr(), _lib.itype_code(slots), table.data_ptr(),
        cache.data_ptr(), cache.stride(0), cache.stride(1), cache.stride(2),
        block_size, max_blocks, _lib.stream_ptr(dev)))


def hybrid_encode_and_store_pair(htq, key: torch.Tensor, value: torch.Tensor, slot_mapping: torch.Tensor,
                                 k_cache: torch.Tensor, v_cache: torch.Tensor, block_size: int = 16,
                                 max_blocks: int = 0) -> None:
    """K and V of a step (the two encodes of tq::hybrid_decode_step, reference vllm/hooks.py:271-284) in one call:
    one launch while the step is small.  Tensors or caches that differ in dtype, shape or strides go through
    hybrid_encode_and_store one after the other."""
    same = (key.shape == value.shape and key.dtype == value.dtype and key.stride() == value.stride()
            and key.dim() == 3 and key.stride(-1) == 1 and key.dtype in (torch.float16, torch.bfloat16, torch.float32)
            and k_cache.shape == v_cache.shape and k_cache.stride() == v_cache.stride()
            and k_cache.dtype == torch.uint8 and v_cache.dtype == torch.uint8 and k_cache.stride(-1) == 1
            and k_cache.shape[-1] >= htq.packed_dim and htq.group_order is None
            and slot_mapping.is_contiguous() and key.shape[-1] == htq.head_dim)
    if not same:
        hybrid_encode_and_store(htq, key, slot_mapping, k_cache, block_size, max_blocks)
        hybrid_encode_and_store(htq, value, slot_mapping, v_cache, block_size, max_blocks)
        return
    num_tokens, num_kv_heads, _ = key.shape
    if num_tokens == 0:
        return
    if max_blocks == 0:
        max_blocks = k_cache.shape[0]
    table = htq.kernel_table
    dev = _lib.require_gpu(key, value, slot_mapping, k_cache, v_cache, table)
    _lib.check(getattr(_lib.lib(), htq._abi + "_encode_paged_kv")(
        key.data_ptr(), value.data_ptr(), _lib.dtype_code(key), num_tokens, num_kv_heads, key.stride(0), key.stride(1),
        slot_mapping.data_ptr(), _lib.itype_code(slot_mapping), table.data_ptr(),
        k_cache.data_ptr(), v_cache.data_ptr(), k_cache.stride(0), k_cache.stride(1), k_cache.stride(2),
        block_size, max_blocks, _lib.stream_ptr(dev)))


class HybridPagedAttention:
    """attn = HybridPagedAttention(htq, num_query_heads=32)
    out = attn.forward(query, k_cache, v_cache, block_tables, context_lens, scale=...)"""

    def __init__(self, htq, num_query_heads: int):
        self._htq = htq
        self.num_query_heads = num_query_heads
        self.head_dim = htq.head_dim
        self._workspace: Optional[torch.Tensor] = None

    def forward(self, query, k_cache, v_cache, block_tables, context_lens, block_size: int = 16,
                num_kv_heads: Optional[int] = None, scale: Optional[float] = None) -> torch.Tensor:
        if num_kv_heads is None:
            num_kv_heads = k_cache.shape[2]
        if scale is None:
            scale = 1.0 / (self.head_dim ** 0.5)
        table = self._htq.kernel_table
        dev = _lib.require_gpu(query, k_cache, v_cache, block_tables, context_lens, table)
        num_seqs, num_q_heads, head_dim = query.shape
        if head_dim != self.head_dim or num_q_heads != self.num_query_heads:
            raise ValueError(f"query shape {tuple(query.shape)} does not match heads="
                             f"{self.num_query_heads}, head_dim={self.head_dim}")
        q = query
        if q.dtype not in (torch.float16, torch.bfloat16, torch.float32):
            q = q.float()
        # A variance-ranked split stores every kv head's rows in that head's group order: the query heads of the
        # kv head are moved into the same order (the dot products do not change), the outputs are moved back.
        ranked = self._htq.group_order is not None
        if ranked:
            q = self._htq.to_group_order(q.reshape(num_seqs, num_kv_heads, -1, head_dim), head_axis=1) \
                .reshape(num_seqs, num_q_heads, head_dim)
        if q.stride(-1) != 1:
            q = q.contiguous()
        out = torch.empty((num_seqs, num_q_heads, head_dim), dtype=q.dtype, device=dev)
        if num_seqs == 0:
            return out
        for name, t in (("k_cache", k_cache), ("v_cache", v_cache)):
            if t.dtype != torch.uint8 or t.stride(-1) != 1 or t.shape[-1] < self._htq.packed_dim:
                raise ValueError(f"{name} must be uint8 with contiguous rows of >= {self._htq.packed_dim} bytes")
        bt = block_tables if block_tables.stride(-1) == 1 else block_tables.contiguous()
        cl = context_lens if context_lens.is_contiguous() else context_lens.contiguous()
        L = _lib.lib()
        need = L.akv_hybrid_paged_attn_workspace_bytes(num_seqs, num_q_heads)
        if self._workspace is None or self._workspace.numel() < need or self._workspace.device != dev:
            self._workspace = torch.empty(need, dtype=torch.uint8, device=dev)
        ws = self._workspace
        _lib.check(getattr(L, self._htq._abi + "_paged_attn")(
            q.data_ptr(), _lib.dtype_code(q), q.stride(0), q.stride(1),
            k_cache.data_ptr(), k_cache.stride(0), k_cache.stride(1), k_cache.stride(2),
            v_cache.data_ptr(), v_cache.stride(0), v_cache.stride(1), v_cache.stride(2),
            bt.data_ptr(), _lib.itype_code(bt), bt.stride(0), cl.data_ptr(), _lib.itype_code(cl),
            table.data_ptr(),
            out.data_ptr(), _lib.dtype_code(out), out.stride(0), out.stride(1),
            num_seqs, num_q_heads, num_kv_heads, block_size, min(k_cache.shape[0], v_cache.shape[0]),
            bt.shape[1], float(scale),
            ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev)))
        if ranked:
            out = self._htq.from_group_order(out.reshape(num_seqs, num_kv_heads, -1, head_dim), head_axis=1) \
                .reshape(num_seqs, num_q_heads, head_dim)
        return out if out.dtype == query.dtype else out.to(query.dtype)

    def last_call_status(self) -> int:
        """0 when the most recent forward() ran clean; bit 0 set when a bounded hand-off wait inside
        its main kernel gave up (the outputs of that call are NaN).  Synchronises the stream."""
        return _lib.attn_status(self._workspace)
