"""The compressed KV cache object of the serving integration: per-layer packed codes and float32
norms in HBM, with a pinned-host cold tier that blocks can be spilled to and warmed from
(reference: aither_kvcache/vllm/cache.py:22-173, class TQGPUCache).

Same constructor, tensors, per-layer views and methods as the reference.  What differs underneath:
`encode_and_store` is the fused encode-on-write kernel (one launch for K, one for V; negative slots
skipped on the device, no boolean-mask gather and no host synchronisation), and spill / warm move
the selected blocks through one pinned staging buffer per tensor, so the copy to the device is a
real asynchronous copy on the current stream (advanced indexing of a pinned tensor yields pageable
memory, which makes the reference's `non_blocking=True` a synchronous copy).  The reference's
second class, ColdTierCache (a background thread that encodes on the CPU), is not built: this
package has no CPU encode path.
"""
import logging
from typing import List, Set

import torch

from ..fused_kv_update import fused_encode_and_store
from ..packing import packed_size
from ..quantizer import TurboQuant

logger = logging.getLogger("turboquant.vllm.cache")


class TQGPUCache:
    def __init__(self, num_layers: int, max_blocks: int, block_size: int, num_kv_heads: int,
                 head_dim: int, bits: int = 4, device: str = "cuda"):
        self.tq = TurboQuant(head_dim=head_dim, bits=bits, device=device)
        self.num_layers = num_layers
        self.max_blocks = max_blocks
        self.block_size = block_size
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.packed_dim = packed_size(head_dim, bits)
        code_shape = (num_layers, max_blocks, block_size, num_kv_heads, self.packed_dim)
        norm_shape = code_shape[:-1]
        # HBM: one contiguous tensor per kind, [layer, block, position, head(, byte)]
        self._k_packed = torch.zeros(code_shape, dtype=torch.uint8, device=device)
        self._k_norms = torch.zeros(norm_shape, dtype=torch.float32, device=device)
        self._v_packed = torch.zeros(code_shape, dtype=torch.uint8, device=device)
        self._v_norms = torch.zeros(norm_shape, dtype=torch.float32, device=device)
        # per-layer views (no copy): what the encode and attention entry points take
        self.k_packed = [self._k_packed[li] for li in range(num_layers)]
        self.k_norms = [self._k_norms[li] for li in range(num_layers)]
        self.v_packed = [self._v_packed[li] for li in range(num_layers)]
        self.v_norms = [self._v_norms[li] for li in range(num_layers)]
        # cold tier in pinned host memory (allocated pinned; existing memory is never registered)
        pin = torch.cuda.is_available()
        self._cold_k_packed = torch.zeros(code_shape, dtype=torch.uint8, pin_memory=pin)
        self._cold_k_norms = torch.zeros(norm_shape, dtype=torch.float32, pin_memory=pin)
        self._cold_v_packed = torch.zeros(code_shape, dtype=torch.uint8, pin_memory=pin)
        self._cold_v_norms = torch.zeros(norm_shape, dtype=torch.float32, pin_memory=pin)
        self._cold_valid = torch.zeros(max_blocks, dtype=torch.bool)
        self._spilled_set: Set[int] = set()
        self._stage: List[torch.Tensor] = []        # pinned staging, grown on demand
        mb = num_layers * 2 * max_blocks * block_size * num_kv_heads * (self.packed_dim + 4) / (1024 ** 2)
        logger.info("TQGPUCache: %d layers x %d blocks @ TQ%d, %.0f MB HBM + %.0f MB host",
                    num_layers, max_blocks, bits, mb, mb)

    def _pairs(self):
        return ((self._k_packed, self._cold_k_packed), (self._k_norms, self._cold_k_norms),
                (self._v_packed, self._cold_v_packed), (self._v_norms, self._cold_v_norms))

    def _staging(self, n: int) -> List[torch.Tensor]:
        """Pinned buffers [block, layer, ...]: the first n blocks are one contiguous run of bytes."""
        if not self._stage or self._stage[0].shape[0] < n:
            pin = torch.cuda.is_available()
            self._stage = [torch.empty((n, c.shape[0]) + tuple(c.shape[2:]), dtype=c.dtype, pin_memory=pin)
                           for _, c in self._pairs()]
        return self._stage

    def encode_and_store(self, layer_idx: int, key: torch.Tensor, value: torch.Tensor,
                         slot_mapping: torch.Tensor) -> None:
        """Encode the new K and V tokens ([T, kv_heads, head_dim]) into the layer's blocks; tokens
        with a negative slot are skipped (reference: cache.py:100-122)."""
        fused_encode_and_store(self, layer_idx, key, value, slot_mapping)

    def spill_blocks(self, block_indices: torch.Tensor) -> None:
        """Copy blocks (all layers) from HBM to the cold tier (reference: cache.py:124-134)."""
        if block_indices.numel() == 0:
            return
        bi_dev = block_indices.to(device=self._k_packed.device, dtype=torch.long)
        bi = block_indices.detach().to("cpu", torch.long)
        n = bi.numel()
        stage = self._staging(n)
        for (hot, _), st in zip(self._pairs(), stage):
            st[:n].copy_(hot.index_select(1, bi_dev).transpose(0, 1).contiguous(), non_blocking=True)
        torch.cuda.current_stream(self._k_packed.device).synchronize()
        for (_, cold), st in zip(self._pairs(), stage):
            cold[:, bi] = st[:n].transpose(0, 1)
        self._cold_valid[bi] = True
        self._spilled_set.update(bi.tolist())

    def warm_blocks(self, block_indices: torch.Tensor) -> None:
        """Copy blocks that have been spilled back into HBM; others are left alone
        (reference: cache.py:136-153).  The device copies are queued on the current stream."""
        if block_indices.numel() == 0:
            return
        bi = block_indices.detach().to("cpu", torch.long)
        bi = bi[self._cold_valid[bi]]
        n = bi.numel()
        if n == 0:
            return
        dev = self._k_packed.device
        # the staging buffers may still feed the copies of an earlier call
        torch.cuda.current_stream(dev).synchronize()
        stage = self._staging(n)
        bi_dev = bi.to(dev)
        for (hot, cold), st in zip(self._pairs(), stage):
            st[:n].copy_(cold.index_select(1, bi).transpose(0, 1))
            hot.index_copy_(1, bi_dev, st[:n].to(dev, non_blocking=True).transpose(0, 1))

    def cold_tier_stats(self) -> dict:
        valid_blocks = int(self._cold_valid.sum().item())
        per_block = 2 * self.block_size * self.num_kv_heads * (self.packed_dim + 4) * self.num_layers
        return {"cold_blocks": valid_blocks, "cold_tokens": valid_blocks * self.block_size,
                "cold_mb": valid_blocks * per_block / (1024 ** 2), "max_blocks": self.max_blocks}

    def has_spilled(self, block_idx: int) -> bool:
        return block_idx in self._spilled_set

    def clear_spilled(self, block_indices: list) -> None:
        self._spilled_set.difference_update(block_indices)
