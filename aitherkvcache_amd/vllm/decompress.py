"""Decode of the cache blocks a batch touches into a float16 / bfloat16 / float32 block buffer:
the job of TurboQuantImpl._batch_decompress_active_blocks (aither_kvcache/vllm/backend.py:
1040-1091), which the reference's prefill and non-fused decode paths run before dense attention.

The reference gathers the unique active blocks, decodes them as one flat batch and scatters the
result back.  Here the block table goes to the kernel as it is: every listed block inside the
cache is decoded from where it lies to where it belongs, K and V in one call each, with no
intermediate tensors.  A block that several sequences share is decoded once per listing, to the
same values.
"""
import torch

from .. import _lib


def decode_blocks(cache: torch.Tensor, norms: torch.Tensor, buf: torch.Tensor, tq,
                  block_ids: torch.Tensor, num_blocks: int) -> None:
    """cache uint8 [blocks, block_size, kv_heads, >= packed_dim], norms float32 [blocks, block_size,
    kv_heads], buf [blocks, block_size, kv_heads, head_dim]; block_ids any integer tensor (flattened
    here); ids outside [0, num_blocks) are skipped."""
    dev = _lib.require_gpu(cache, norms, buf, block_ids)
    if cache.dtype != torch.uint8 or norms.dtype != torch.float32:
        raise TypeError("cache must be uint8 and norms float32")
    if cache.dim() != 4 or norms.dim() != 3 or buf.dim() != 4:
        raise ValueError("expected cache [B, bs, H, bytes], norms [B, bs, H], buf [B, bs, H, d]")
    if cache.stride(3) != 1 or buf.stride(3) != 1:
        raise ValueError("last dimension of cache and buf must be contiguous")
    if tuple(cache.shape[:3]) != tuple(norms.shape) or tuple(buf.shape[:3]) != tuple(norms.shape):
        raise ValueError("cache, norms and buf disagree on [blocks, block_size, kv_heads]")
    if buf.shape[3] != tq.head_dim or cache.shape[3] < tq._packed_dim:
        raise ValueError("row sizes do not match the quantizer")
    if num_blocks > cache.shape[0]:
        raise ValueError("num_blocks exceeds the cache")
    ids = block_ids.reshape(-1)
    if ids.dtype not in (torch.int32, torch.int64):
        ids = ids.to(torch.int64)
    if not ids.is_contiguous():
        ids = ids.contiguous()
    if ids.numel() == 0 or num_blocks == 0:
        return
    _lib.check(_lib.lib().akv_decode_blocks(
        cache.data_ptr(), cache.stride(0), cache.stride(1), cache.stride(2),
        norms.data_ptr(), norms.stride(0), norms.stride(1), norms.stride(2),
        ids.data_ptr(), _lib.itype_code(ids), ids.numel(), num_blocks,
        cache.shape[1], cache.shape[2], tq.head_dim,
        tq.prepared_rotation().ptr, tq.centroids.data_ptr(), tq.bits,
        buf.data_ptr(), _lib.dtype_code(buf), buf.stride(0), buf.stride(1), buf.stride(2),
        _lib.stream_ptr(dev)))


def batch_decompress_active_blocks(key_cache, value_cache, k_buf, v_buf, tq, packed_dim, block_table,
                                   num_blocks, k_norms, v_norms) -> None:
    """Argument order of the reference method (backend.py:1040-1043); the per-layer norm tensors,
    which the reference reads from class state (:1073-1075), are passed in."""
    if packed_dim != tq._packed_dim:
        raise ValueError(f"packed_dim {packed_dim} does not match the quantizer ({tq._packed_dim})")
    decode_blocks(key_cache, k_norms, k_buf, tq, block_table, num_blocks)
    decode_blocks(value_cache, v_norms, v_buf, tq, block_table, num_blocks)
