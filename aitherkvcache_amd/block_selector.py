"""Block selection for sparse decode attention over a 4-bit TurboQuant cache.

Same classes, functions and arguments as the reference's aither_kvcache/block_selector.py:
`BlockRepresentativeCache` (norm-weighted mean of the rotated-domain key codes per block and kv
head, kept from the packed codes), `score_blocks`, `select_blocks` and the orchestrating
`BlockSelector`.  The attention kernel is unchanged: it is handed the filtered block table and
context lengths.  Every step is one HIP kernel launch behind the C ABI (akv_block_*).

Differences from the reference, on purpose: the token counts are int32 (int16 there); among table
columns of exactly equal score the lower column is selected (torch.topk leaves that open); block
ids outside [0, max_blocks) in an update are skipped.
"""
import math
from typing import Optional, Tuple

import torch

from . import _lib


def _index_tensor(t: torch.Tensor) -> torch.Tensor:
    if t.dtype not in (torch.int32, torch.int64):
        t = t.to(torch.int64)
    return t if t.is_contiguous() else t.contiguous()


class BlockRepresentativeCache:
    """Per-block key representatives in the even / odd (high / low nibble) split of the packed row
    (reference: block_selector.py:29-126).  Memory: 4 x max_blocks x kv_heads x half_d floats."""

    def __init__(self, max_blocks: int, num_kv_heads: int, half_d: int, device, centroids: torch.Tensor):
        self.max_blocks = max_blocks
        self.num_kv_heads = num_kv_heads
        self.half_d = half_d
        self.centroids = centroids.to(device=device, dtype=torch.float32).contiguous()
        shape = (max_blocks, num_kv_heads, half_d)
        self._acc_even = torch.zeros(shape, dtype=torch.float32, device=device)
        self._acc_odd = torch.zeros_like(self._acc_even)
        self._counts = torch.zeros(max_blocks, num_kv_heads, dtype=torch.int32, device=device)
        self.rep_even = torch.zeros_like(self._acc_even)
        self.rep_odd = torch.zeros_like(self._acc_even)

    def _update(self, block_indices, k_packed, k_norms, finalize: bool) -> None:
        dev = _lib.require_gpu(block_indices, k_packed, k_norms, self._acc_even)
        n, h, pd = k_packed.shape
        if h != self.num_kv_heads or pd != self.half_d:
            raise ValueError(f"k_packed shape {tuple(k_packed.shape)} does not match kv_heads={self.num_kv_heads}, "
                             f"packed_dim={self.half_d}")
        if k_packed.dtype != torch.uint8 or k_packed.stride(2) != 1:
            raise TypeError("k_packed must be uint8 with a contiguous last dimension")
        if tuple(k_norms.shape) != (n, h):
            raise ValueError("k_norms must be [N, num_kv_heads]")
        kn = k_norms if k_norms.dtype == torch.float32 else k_norms.float()
        bi = _index_tensor(block_indices.reshape(-1))
        if bi.numel() != n:
            raise ValueError("one block index per token expected")
        _lib.check(_lib.lib().akv_block_rep_update(
            bi.data_ptr(), _lib.itype_code(bi), n, k_packed.data_ptr(), k_packed.stride(0), k_packed.stride(1),
            kn.data_ptr(), kn.stride(0), kn.stride(1), self.centroids.data_ptr(),
            self._acc_even.data_ptr(), self._acc_odd.data_ptr(), self._counts.data_ptr(),
            self.rep_even.data_ptr() if finalize else None, self.rep_odd.data_ptr() if finalize else None,
            self.max_blocks, self.num_kv_heads, self.half_d, _lib.stream_ptr(dev)))

    def update(self, block_indices: torch.Tensor, positions: torch.Tensor, k_packed: torch.Tensor,
               k_norms: torch.Tensor) -> None:
        """block_indices [N] physical block of each new token, positions [N] (not needed for the mean),
        k_packed [N, kv_heads, packed_dim] uint8, k_norms [N, kv_heads] float32."""
        self._update(block_indices, k_packed, k_norms, finalize=False)

    def finalize(self, block_indices: Optional[torch.Tensor] = None) -> None:
        """rep = acc / max(count, 1) for the given blocks, or for all of them."""
        dev = self._acc_even.device
        _lib.require_gpu(self._acc_even)
        if block_indices is None:
            ptr, code, n = None, 0, 0
        else:
            bi = _index_tensor(block_indices.reshape(-1))
            ptr, code, n = bi.data_ptr(), _lib.itype_code(bi), bi.numel()
        _lib.check(_lib.lib().akv_block_rep_finalize(
            ptr, code, n, self._acc_even.data_ptr(), self._acc_odd.data_ptr(), self._counts.data_ptr(),
            self.rep_even.data_ptr(), self.rep_odd.data_ptr(), self.max_blocks, self.num_kv_heads, self.half_d,
            _lib.stream_ptr(dev)))

    def clear_blocks(self, block_indices: torch.Tensor) -> None:
        """Zero the accumulators, counts and representatives of freed blocks."""
        bi = block_indices.reshape(-1).long()
        for t in (self._acc_even, self._acc_odd, self._counts, self.rep_even, self.rep_odd):
            t[bi] = 0


def score_blocks(q_even: torch.Tensor, q_odd: torch.Tensor, rep_even: torch.Tensor, rep_odd: torch.Tensor,
                 block_tables: torch.Tensor, context_lens: torch.Tensor, gqa_ratio: int,
                 block_size: int) -> torch.Tensor:
    """[num_seqs, max_blocks_per_seq] float32 relevance of every table column to the query
    (reference: block_selector.py:129-179); columns past the context are -inf."""
    dev = _lib.require_gpu(q_even, q_odd, rep_even, rep_odd, block_tables, context_lens)
    num_seqs, num_q_heads, half_d = q_even.shape
    if num_q_heads % gqa_ratio != 0:
        raise ValueError("num_q_heads must be a multiple of gqa_ratio")
    qe = q_even.float().contiguous()
    qo = q_odd.float().contiguous()
    if not (rep_even.is_contiguous() and rep_odd.is_contiguous()) or rep_even.dtype != torch.float32:
        raise TypeError("representatives must be contiguous float32")
    bt = block_tables if block_tables.dtype in (torch.int32, torch.int64) else block_tables.long()
    if bt.stride(1) != 1:
        bt = bt.contiguous()
    cl = _index_tensor(context_lens)
    scores = torch.empty(num_seqs, bt.shape[1], dtype=torch.float32, device=dev)
    _lib.check(_lib.lib().akv_block_scores(
        qe.data_ptr(), qo.data_ptr(), rep_even.data_ptr(), rep_odd.data_ptr(),
        bt.data_ptr(), _lib.itype_code(bt), bt.stride(0), cl.data_ptr(), _lib.itype_code(cl),
        num_seqs, num_q_heads, num_q_heads // gqa_ratio, half_d, bt.shape[1], block_size, rep_even.shape[0],
        scores.data_ptr(), _lib.stream_ptr(dev)))
    return scores


def select_blocks(scores: torch.Tensor, block_tables: torch.Tensor, context_lens: torch.Tensor, block_size: int,
                  max_selected: int, num_sink_blocks: int = 2,
                  num_recent_blocks: int = 2) -> Tuple[torch.Tensor, torch.Tensor]:
    """(filtered_block_tables [num_seqs, max_selected], filtered_context_lens [num_seqs]); the shapes do
    not depend on the data (reference: block_selector.py:182-236)."""
    dev = _lib.require_gpu(scores, block_tables, context_lens)
    num_seqs, max_bps = scores.shape
    sc = scores if scores.dtype == torch.float32 and scores.is_contiguous() else scores.float().contiguous()
    bt = block_tables if block_tables.dtype in (torch.int32, torch.int64) else block_tables.long()
    if bt.stride(1) != 1:
        bt = bt.contiguous()
    cl = _index_tensor(context_lens)
    fbt = torch.empty(num_seqs, max_selected, dtype=bt.dtype, device=dev)
    fcl = torch.empty(num_seqs, dtype=cl.dtype, device=dev)
    if max_bps == 0:
        return fbt.zero_(), torch.minimum(cl, torch.zeros_like(cl))
    _lib.check(_lib.lib().akv_block_select(
        sc.data_ptr(), bt.data_ptr(), _lib.itype_code(bt), bt.stride(0), cl.data_ptr(), _lib.itype_code(cl),
        num_seqs, max_bps, block_size, max_selected, num_sink_blocks, num_recent_blocks,
        fbt.data_ptr(), fcl.data_ptr(), _lib.stream_ptr(dev)))
    return fbt, fcl


class BlockSelector:
    """Scores and selects blocks when select_ratio < 1; does nothing otherwise
    (reference: block_selector.py:239-337)."""

    def __init__(self, max_blocks: int, num_kv_heads: int, half_d: int, device, centroids: torch.Tensor,
                 select_ratio: float = 1.0, num_sink_blocks: int = 2, num_recent_blocks: int = 2,
                 min_blocks_for_selection: int = 64):
        self.select_ratio = select_ratio
        self.num_sink_blocks = num_sink_blocks
        self.num_recent_blocks = num_recent_blocks
        self.min_blocks = min_blocks_for_selection
        self.enabled = select_ratio < 1.0
        if self.enabled:
            self._rep_cache = BlockRepresentativeCache(max_blocks, num_kv_heads, half_d, device, centroids)
            self._max_selected = max(num_sink_blocks + num_recent_blocks + 1, math.ceil(max_blocks * select_ratio))
        else:
            self._rep_cache = None
            self._max_selected = 0

    @property
    def max_selected(self) -> int:
        return self._max_selected

    def update_reps(self, block_indices, positions, k_packed, k_norms) -> None:
        """Fold newly written tokens into their blocks' representatives (update + finalize of the
        touched blocks, one launch each)."""
        if self._rep_cache is not None:
            self._rep_cache._update(block_indices, k_packed, k_norms, finalize=True)

    def clear_blocks(self, block_indices) -> None:
        if self._rep_cache is not None:
            self._rep_cache.clear_blocks(block_indices)

    def select(self, q_even, q_odd, block_tables, context_lens, gqa_ratio: int,
               block_size: int = 16) -> Tuple[torch.Tensor, torch.Tensor]:
        if not self.enabled or block_tables.shape[1] < self.min_blocks:
            return block_tables, context_lens
        scores = score_blocks(q_even, q_odd, self._rep_cache.rep_even, self._rep_cache.rep_odd, block_tables,
                              context_lens, gqa_ratio, block_size)
        return select_blocks(scores, block_tables, context_lens, block_size, self._max_selected,
                             self.num_sink_blocks, self.num_recent_blocks)
