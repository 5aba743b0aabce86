"""torch custom ops for one decode step over a TurboQuant cache, with the signatures of the
reference's aither_kvcache/vllm/hooks.py:129-213 (tq::decode_step) and :240-363
(tq::hybrid_decode_step): encode the step's new K/V tokens into the paged cache, then attend.

Each op is one C-ABI call for the write (K and V in one launch) and one for the attention; nothing in the body
synchronises with the host or allocates after the first call for a given batch shape, so the
ops can be recorded into a HIP graph after a warm-up call.

Differences from the reference, both on purpose: tokens whose slot is negative are skipped
(the reference indexes with them, which wraps to the end of the cache), and the hybrid op
attends directly on the packed rows in float32 instead of decompressing every block and running
bf16 SDPA.
"""
import logging
from typing import Dict, Optional

import torch

from ..fused_attention import TQPagedAttention
from ..fused_kv_update import fused_kv_update_pair
from ..hybrid_attention import HybridPagedAttention, hybrid_encode_and_store_pair
from ..hybrid_quantizer import HybridTurboQuant
from ..quantizer import TurboQuant

logger = logging.getLogger("turboquant.hooks")

_tq_quantizers: Dict[int, object] = {}       # head_size -> TurboQuant | HybridTurboQuant
_tq_fused_attn: Dict[tuple, object] = {}     # (layer_idx, head_size) -> attention object
_USE_CUSTOM_OP = False
_USE_HYBRID_CUSTOM_OP = False


def init_quantizer(head_size: int, bits: Optional[int] = 4, mode: Optional[str] = None,
                   device: str = "cuda", num_kv_heads: int = 1):
    """Create (once) the quantizer the ops use for heads of `head_size`."""
    q = _tq_quantizers.get(head_size)
    if q is None:
        if mode is not None:
            q = HybridTurboQuant(head_dim=head_size, mode=mode, device=device)
            q.calibrate_uniform(num_kv_heads=num_kv_heads)
        else:
            q = TurboQuant(head_dim=head_size, bits=bits, device=device)
        _tq_quantizers[head_size] = q
    return q


def reset_state() -> None:
    _tq_quantizers.clear()
    _tq_fused_attn.clear()


def decode_step(query, key, value, kv_cache, output, k_norms, v_norms, slot_mapping, block_table,
                seq_lens, layer_idx: int, num_heads: int, num_kv_heads: int, head_size: int,
                scale: float, num_actual: int) -> torch.Tensor:
    """Body of tq::decode_step.  kv_cache uint8 [blocks, 2, block_size, kv_heads, tq_dim];
    k_norms / v_norms float32 [layers, blocks, block_size, kv_heads]; mutates kv_cache, output,
    k_norms, v_norms; returns output.clone()."""
    tq = _tq_quantizers[head_size]
    key_cache, value_cache = kv_cache[:, 0], kv_cache[:, 1]
    block_size = key_cache.shape[1]
    n = key.shape[0]
    prep = tq.prepared_rotation()
    fused_kv_update_pair(key, value, slot_mapping[:n], key_cache, k_norms[layer_idx], value_cache,
                         v_norms[layer_idx], tq.rotation, tq.boundaries_inner, tq.bits,
                         block_size=block_size, prepared=prep)
    attn = _tq_fused_attn.get((layer_idx, head_size))
    if attn is None:
        attn = TQPagedAttention(tq, num_heads)
        _tq_fused_attn[(layer_idx, head_size)] = attn
    out = attn.forward(query[:num_actual], key_cache, k_norms[layer_idx], value_cache,
                       v_norms[layer_idx], block_table, seq_lens, block_size=block_size,
                       num_kv_heads=num_kv_heads)
    output[:num_actual] = out.to(output.dtype)
    return output.clone()


def hybrid_decode_step(query, key, value, kv_cache, output, slot_mapping, block_table, seq_lens,
                       layer_idx: int, num_heads: int, num_kv_heads: int, head_size: int,
                       scale: float, num_actual: int) -> torch.Tensor:
    """Body of tq::hybrid_decode_step; kv_cache uint8 [blocks, 2, block_size, kv_heads, packed_dim] (64 bytes for tq35, 44 for tq25)."""
    htq = _tq_quantizers[head_size]
    key_cache, value_cache = kv_cache[:, 0], kv_cache[:, 1]
    block_size = key_cache.shape[1]
    n = key.shape[0]
    hybrid_encode_and_store_pair(htq, key, value, slot_mapping[:n], key_cache, value_cache, block_size=block_size)
    attn = _tq_fused_attn.get((layer_idx, head_size))
    if attn is None:
        attn = HybridPagedAttention(htq, num_heads)
        _tq_fused_attn[(layer_idx, head_size)] = attn
    out = attn.forward(query[:num_actual], key_cache, value_cache, block_table, seq_lens,
                       block_size=block_size, num_kv_heads=num_kv_heads, scale=scale)
    output[:num_actual] = out.to(output.dtype)
    return output.clone()


def register_custom_ops() -> bool:
    """Register tq::decode_step and tq::hybrid_decode_step (idempotent).  Returns True when the
    ops are available under torch.ops.tq."""
    global _USE_CUSTOM_OP, _USE_HYBRID_CUSTOM_OP
    if _USE_CUSTOM_OP and _USE_HYBRID_CUSTOM_OP:
        return True
    if not hasattr(torch.library, "custom_op"):
        logger.info("torch.library.custom_op unavailable; call decode_step() directly")
        return False

    @torch.library.custom_op("tq::decode_step",
                             mutates_args=("kv_cache", "output", "k_norms", "v_norms"))
    def _decode_step_op(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                        kv_cache: torch.Tensor, output: torch.Tensor, k_norms: torch.Tensor,
                        v_norms: torch.Tensor, slot_mapping: torch.Tensor,
                        block_table: torch.Tensor, seq_lens: torch.Tensor, layer_idx: int,
                        num_heads: int, num_kv_heads: int, head_size: int, scale: float,
                        num_actual: int) -> torch.Tensor:
        return decode_step(query, key, value, kv_cache, output, k_norms, v_norms, slot_mapping,
                           block_table, seq_lens, layer_idx, num_heads, num_kv_heads, head_size,
                           scale, num_actual)

    @_decode_step_op.register_fake
    def _(query, key, value, kv_cache, output, k_norms, v_norms, slot_mapping, block_table,
          seq_lens, layer_idx, num_heads, num_kv_heads, head_size, scale, num_actual):
        return output.clone()

    @torch.library.custom_op("tq::hybrid_decode_step", mutates_args=("kv_cache", "output"))
    def _hybrid_decode_step_op(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                               kv_cache: torch.Tensor, output: torch.Tensor,
                               slot_mapping: torch.Tensor, block_table: torch.Tensor,
                               seq_lens: torch.Tensor, layer_idx: int, num_heads: int,
                               num_kv_heads: int, head_size: int, scale: float,
                               num_actual: int) -> torch.Tensor:
        return hybrid_decode_step(query, key, value, kv_cache, output, slot_mapping, block_table,
                                  seq_lens, layer_idx, num_heads, num_kv_heads, head_size, scale,
                                  num_actual)

    @_hybrid_decode_step_op.register_fake
    def _(query, key, value, kv_cache, output, slot_mapping, block_table, seq_lens, layer_idx,
          num_heads, num_kv_heads, head_size, scale, num_actual):
        return output.clone()

    _USE_CUSTOM_OP = _USE_HYBRID_CUSTOM_OP = True
    return True
