"""Paged storage of spectral K/V encodings (reference: aither_kvcache/triattention/cache.py:37-232).

Same tensors, methods and block layout as the reference's SpectralKVCache: per physical block
k/v_indices and k/v_packed [block_size, kv_heads, F] uint8 and k/v_scales [block_size, kv_heads]
float16.  Storing, copying and clearing blocks are tensor assignments (bookkeeping, not the hot
path); reading a sequence back for attention does not go through `fetch_sequence` at all --
`TriAttention.decode_step_paged` hands the block pool and the block tables to the decode kernel.
The fill counters live on the host (the reference reads them back with .item() on every store).
"""
import math
from typing import Optional, Tuple

import torch

from .. import _lib
from .config import TriAttentionConfig
from .encoder import SpectralEncoding


class SpectralKVCache:
    def __init__(self, config: TriAttentionConfig, max_blocks: int = 1024, device: str = "cpu"):
        if config.coeff_bits != 4:
            raise NotImplementedError("the paged spectral cache stores int4 coefficients")
        self.config = config
        self.max_blocks = max_blocks
        self.block_size = config.block_size
        self.num_kv_heads = config.num_kv_heads
        self.num_freqs = config.num_freqs
        self.device = device
        F, KVH, BS = config.num_freqs, config.num_kv_heads, config.block_size

        def u8():
            return torch.zeros(max_blocks, BS, KVH, F, dtype=torch.uint8, device=device)

        def f16():
            return torch.zeros(max_blocks, BS, KVH, dtype=torch.float16, device=device)

        self.k_indices, self.k_packed, self.k_scales = u8(), u8(), f16()
        self.v_indices, self.v_packed, self.v_scales = u8(), u8(), f16()
        self._block_fill = [0] * max_blocks

    def _arrays(self):
        return (self.k_indices, self.k_packed, self.k_scales, self.v_indices, self.v_packed, self.v_scales)

    @property
    def bytes_allocated(self) -> int:
        return sum(t.element_size() * t.numel() for t in self._arrays())

    @property
    def bytes_per_token(self) -> int:
        """Bytes of one token's K row plus V row of one kv head (reference: cache.py:100-103)."""
        return self.config.bytes_per_kv_token * 2

    def store_token(self, block_idx: int, slot_idx: int, k_enc: SpectralEncoding, v_enc: SpectralEncoding) -> None:
        """k_enc / v_enc of one token: indices, packed [kv_heads, F], scales [kv_heads]."""
        for dst, src in zip(self._arrays(), tuple(k_enc) + tuple(v_enc)):
            dst[block_idx, slot_idx] = src
        self._block_fill[block_idx] = max(self._block_fill[block_idx], slot_idx + 1)

    def encode_and_store(self, keys: torch.Tensor, values: torch.Tensor, slot_mapping: torch.Tensor) -> None:
        """Encode-on-write of a step: keys / values [num_tokens, kv_heads, head_dim] (keys before RoPE) are encoded
        (SpectralKVEncoder.encode, reference encoder.py:73-149) and written into the block pool at
        slot = block * block_size + position per token, one launch per tensor -- what the reference does with
        encode followed by store_token per token (cache.py:106-140).  Negative slots and slots past the cache are
        skipped.  No counterpart in the reference."""
        T, KVH, D = keys.shape
        if KVH != self.num_kv_heads or D != self.config.head_dim or values.shape != keys.shape:
            raise ValueError(f"keys / values {tuple(keys.shape)} / {tuple(values.shape)} do not fit kv_heads="
                             f"{self.num_kv_heads}, head_dim={self.config.head_dim}")
        if slot_mapping.numel() != T:
            raise ValueError("slot_mapping must hold one slot per token")
        if T == 0:
            return
        dev = _lib.require_gpu(keys, values, self.k_indices)
        sm = slot_mapping if slot_mapping.dtype in (torch.int32, torch.int64) else slot_mapping.long()
        host_slots = None if sm.is_cuda else sm.tolist()
        sm = sm.to(dev).contiguous()
        L = _lib.lib()
        for x, (idx, cf, sc) in ((keys, (self.k_indices, self.k_packed, self.k_scales)),
                                 (values, (self.v_indices, self.v_packed, self.v_scales))):
            if x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
                x = x.float()
            if x.stride(-1) != 1:
                x = x.contiguous()
            _lib.check(L.akv_tri_encode_paged(
                x.data_ptr(), _lib.dtype_code(x), T, KVH, D, x.stride(0), x.stride(1), self.num_freqs,
                sm.data_ptr(), _lib.itype_code(sm), self.max_blocks * self.block_size,
                idx.data_ptr(), cf.data_ptr(), sc.data_ptr(), _lib.stream_ptr(dev)))
        # (the fill counters serve memory_stats alone: they follow slots given as host data, and are not read back
        # from the device for slots that live there)
        if host_slots is not None:
            for s_ in host_slots:
                if 0 <= s_ < self.max_blocks * self.block_size:
                    b, p_ = divmod(s_, self.block_size)
                    self._block_fill[b] = max(self._block_fill[b], p_ + 1)

    def store_block(self, block_idx: int, k_enc: SpectralEncoding, v_enc: SpectralEncoding,
                    num_tokens: Optional[int] = None) -> None:
        """k_enc / v_enc of up to block_size tokens: [num_tokens, kv_heads, F] etc."""
        if num_tokens is None:
            num_tokens = k_enc.indices.shape[0]
        n = min(num_tokens, self.block_size)
        for dst, src in zip(self._arrays(), tuple(k_enc) + tuple(v_enc)):
            dst[block_idx, :n] = src[:n]
        self._block_fill[block_idx] = n

    def store_sequence(self, block_table: torch.Tensor, k_enc: SpectralEncoding, v_enc: SpectralEncoding) -> None:
        """Write a whole sequence ([S, kv_heads, F] etc.) through its block table in one indexed
        assignment per tensor (no counterpart in the reference, which stores block by block)."""
        S = k_enc.indices.shape[0]
        nb = math.ceil(S / self.block_size)
        bt = block_table[:nb].to(device=self.k_indices.device, dtype=torch.long)
        tok = torch.arange(S, device=bt.device)
        blk, pos = bt[tok // self.block_size], tok % self.block_size
        for dst, src in zip(self._arrays(), tuple(k_enc) + tuple(v_enc)):
            dst[blk, pos] = src.to(dst.device)
        for j, b in enumerate(bt.tolist()):
            self._block_fill[b] = min(self.block_size, S - j * self.block_size)

    def fetch_sequence(self, block_table: torch.Tensor, context_len: int) -> Tuple[SpectralEncoding, SpectralEncoding]:
        """(k_enc, v_enc) with [context_len, kv_heads, F] / [context_len, kv_heads] tensors, gathered
        through the block table (reference: cache.py:163-198)."""
        nb = math.ceil(context_len / self.block_size)
        phys = block_table[:nb].to(device=self.k_indices.device, dtype=torch.long)
        got = [t[phys].reshape(-1, *t.shape[2:])[:context_len] for t in self._arrays()]
        return SpectralEncoding(*got[:3]), SpectralEncoding(*got[3:])

    def copy_block(self, src_block: int, dst_block: int) -> None:
        for t in self._arrays():
            t[dst_block] = t[src_block]
        self._block_fill[dst_block] = self._block_fill[src_block]

    def clear_block(self, block_idx: int) -> None:
        for t in self._arrays():
            t[block_idx].zero_()
        self._block_fill[block_idx] = 0

    def memory_stats(self) -> dict:
        total_tokens = sum(self._block_fill)
        return {
            "max_blocks": self.max_blocks,
            "used_blocks": sum(1 for f in self._block_fill if f > 0),
            "total_tokens": total_tokens,
            "bytes_allocated": self.bytes_allocated,
            "bytes_per_token": self.bytes_per_token,
            "compression_ratio": self.config.kv_compression_ratio,
            "equivalent_fp16_bytes": total_tokens * self.config.head_dim * 2 * 2,
        }
