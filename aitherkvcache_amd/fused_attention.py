"""Paged decode attention straight from the TurboQuant-compressed cache, in the rotated
domain: q' = Pi q once, score_t = |k_t| <q', c[codes_t]> / sqrt(d), out = Pi^T (sum_t w_t |v_t|
c[codes_t]) -- the computation of the reference's TQPagedAttentionRef
(aither_kvcache/fused_attention.py:91-185) behind the interface of its TQPagedAttention
(:538-748).  Pre-rotation, the stream-K split over long contexts, the merge and the inverse
rotation all run on the GPU through one C-ABI call; 2-, 3- and 4-bit caches are handled by
kernels (the reference runs a Python loop for 2/3-bit).
"""
import math
import os
from typing import Optional

import torch

from . import _lib

HAS_HIP = _lib.available()
HAS_TRITON = HAS_HIP


class TQPagedAttention:
    """attn = TQPagedAttention(tq, num_query_heads=32)
    out = attn.forward(query, k_packed, k_norms, v_packed, v_norms, block_tables, context_lens)
    """

    # Kept for call compatibility (fused_attention.py:632-633).  The split over the context is
    # decided on the device from context_lens, so these two no longer steer anything.
    SPLITK_THRESHOLD = int(os.environ.get("AITHER_TQ_SPLITK_THRESHOLD", "64"))
    SPLITK_NUM_SPLITS = int(os.environ.get("AITHER_TQ_SPLITK_SPLITS", "16"))

    def __init__(self, tq, num_query_heads: int, block_selector=None):
        self._tq = tq
        self.rotation = tq.rotation
        self.centroids = tq.centroids
        self.scale = 1.0 / math.sqrt(tq.head_dim)   # always 1/sqrt(d), as the reference (:563)
        self.head_dim = tq.head_dim
        self.num_levels = tq.num_levels
        self.bits = tq.bits
        self.packed_dim = tq._packed_dim
        self.num_query_heads = num_query_heads
        self._block_selector = block_selector
        self._workspace: Optional[torch.Tensor] = None
        self._use_hip = True
        self._use_triton = False

    def _get_workspace(self, num_seqs: int, device) -> torch.Tensor:
        need = _lib.lib().akv_paged_attn_workspace_bytes(num_seqs, self.num_query_heads, self.head_dim)
        ws = self._workspace
        if ws is None or ws.numel() < need or ws.device != device:
            ws = torch.empty(need, dtype=torch.uint8, device=device)
            self._workspace = ws
        return ws

    def forward_no_alloc(self, query, k_packed, k_norms, v_packed, v_norms, block_tables, context_lens,
                         out: torch.Tensor, block_size: int = 16, num_kv_heads: Optional[int] = None) -> torch.Tensor:
        """forward() for callers that may not allocate (under graph capture, in a loop that forbids
        it): the result goes into `out` (same shape as `query`, float16 / bfloat16 / float32) and the
        library works in a fixed scratch array of its own instead of a workspace tensor.  Inputs must
        already be in the form the kernels take (float query with contiguous rows, float32 norms,
        contiguous table rows); batches too large for the built-in array raise.  No block selector."""
        if self._block_selector is not None:
            raise ValueError("forward_no_alloc does not run the block selector (it allocates)")
        return self.forward(query, k_packed, k_norms, v_packed, v_norms, block_tables, context_lens,
                            block_size, num_kv_heads, _static_out=out)

    def forward(self, query, k_packed, k_norms, v_packed, v_norms, block_tables, context_lens,
                block_size: int = 16, num_kv_heads: Optional[int] = None, _static_out=None) -> torch.Tensor:
        """query [num_seqs, num_query_heads, head_dim] -> same shape and dtype.

        k/v_packed [num_blocks, block_size, num_kv_heads, >= packed_dim] uint8 (may be strided
        views with 4-byte aligned rows), k/v_norms [num_blocks, block_size, num_kv_heads] float32,
        block_tables [num_seqs, max_blocks_per_seq] int32/int64, context_lens [num_seqs]."""
        if num_kv_heads is None:
            num_kv_heads = k_packed.shape[2]
        tq = self._tq
        if tq.rotation is not self.rotation:     # the quantizer's matrix was reassigned: follow it
            self.rotation = tq.rotation
        if self._block_selector is not None:
            # as in the reference (:659-668): even / odd coordinates of the rotated query score the blocks,
            # the kernel then walks the filtered table
            q_rot = torch.matmul(query.float(), self.rotation.T)
            block_tables, context_lens = self._block_selector.select(
                q_rot[..., 0::2].contiguous(), q_rot[..., 1::2].contiguous(), block_tables, context_lens,
                query.shape[1] // num_kv_heads, block_size)
        dev = _lib.require_gpu(query, k_packed, k_norms, v_packed, v_norms, block_tables, context_lens)
        num_seqs, num_q_heads, head_dim = query.shape
        if head_dim != self.head_dim or num_q_heads != self.num_query_heads:
            raise ValueError(f"query shape {tuple(query.shape)} does not match heads="
                             f"{self.num_query_heads}, head_dim={self.head_dim}")
        q = query
        if q.dtype not in (torch.float16, torch.bfloat16, torch.float32):
            q = q.float()
        if q.stride(-1) != 1:
            q = q.contiguous()
        if _static_out is not None:
            out = _static_out
            if out.shape != query.shape or out.stride(-1) != 1 or not out.is_cuda:
                raise ValueError("out must be a device tensor of the query's shape with contiguous rows")
        else:
            out = torch.empty((num_seqs, num_q_heads, head_dim), dtype=q.dtype, device=dev)
        if num_seqs == 0:
            return out if _static_out is not None else out.to(query.dtype)
        for name, t in (("k_packed", k_packed), ("v_packed", v_packed)):
            if t.dtype != torch.uint8 or t.stride(-1) != 1 or t.shape[-1] < self.packed_dim:
                raise ValueError(f"{name} must be uint8 with contiguous rows of >= {self.packed_dim} bytes")
        if _static_out is not None and (k_norms.dtype != torch.float32 or v_norms.dtype != torch.float32):
            raise ValueError("forward_no_alloc needs float32 norms (a conversion would allocate)")
        k_norms = k_norms if k_norms.dtype == torch.float32 else k_norms.float()
        v_norms = v_norms if v_norms.dtype == torch.float32 else v_norms.float()
        bt = block_tables if block_tables.stride(-1) == 1 else block_tables.contiguous()
        cl = context_lens if context_lens.is_contiguous() else context_lens.contiguous()
        num_blocks = min(k_packed.shape[0], k_norms.shape[0], v_packed.shape[0], v_norms.shape[0])
        if _static_out is not None:
            if q is not query or bt is not block_tables or cl is not context_lens:
                raise ValueError("forward_no_alloc needs inputs that take no conversion")
            _lib.check(_lib.lib().akv_paged_attn_static(
                q.data_ptr(), _lib.dtype_code(q), q.stride(0), q.stride(1),
                k_packed.data_ptr(), k_packed.stride(0), k_packed.stride(1), k_packed.stride(2),
                k_norms.data_ptr(), k_norms.stride(0), k_norms.stride(1), k_norms.stride(2),
                v_packed.data_ptr(), v_packed.stride(0), v_packed.stride(1), v_packed.stride(2),
                v_norms.data_ptr(), v_norms.stride(0), v_norms.stride(1), v_norms.stride(2),
                bt.data_ptr(), _lib.itype_code(bt), bt.stride(0), cl.data_ptr(), _lib.itype_code(cl),
                self._tq.prepared_rotation().ptr, self.centroids.data_ptr(), self.bits,
                out.data_ptr(), _lib.dtype_code(out), out.stride(0), out.stride(1),
                num_seqs, num_q_heads, num_kv_heads, head_dim, block_size, num_blocks, bt.shape[1], self.scale,
                _lib.stream_ptr(dev)))
            self._last_static = dev
            return out
        self._last_static = None
        ws = self._get_workspace(num_seqs, dev)
        _lib.check(_lib.lib().akv_paged_attn(
            q.data_ptr(), _lib.dtype_code(q), q.stride(0), q.stride(1),
            k_packed.data_ptr(), k_packed.stride(0), k_packed.stride(1), k_packed.stride(2),
            k_norms.data_ptr(), k_norms.stride(0), k_norms.stride(1), k_norms.stride(2),
            v_packed.data_ptr(), v_packed.stride(0), v_packed.stride(1), v_packed.stride(2),
            v_norms.data_ptr(), v_norms.stride(0), v_norms.stride(1), v_norms.stride(2),
            bt.data_ptr(), _lib.itype_code(bt), bt.stride(0), cl.data_ptr(), _lib.itype_code(cl),
            tq.prepared_rotation().ptr, self.centroids.data_ptr(), self.bits,
            out.data_ptr(), _lib.dtype_code(out), out.stride(0), out.stride(1),
            num_seqs, num_q_heads, num_kv_heads, head_dim, block_size, num_blocks, bt.shape[1], self.scale,
            ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev)))
        return out if out.dtype == query.dtype else out.to(query.dtype)

    def last_call_status(self) -> int:
        """0 when the most recent forward() / forward_no_alloc() ran clean; bit 0 set when a bounded hand-off
        wait inside its main kernel gave up (the outputs of that call are NaN).  Synchronises the stream."""
        if getattr(self, "_last_static", None) is not None:
            return _lib.attn_status_static(self._last_static)       # the library's built-in scratch array
        return _lib.attn_status(self._workspace)


class _RotationHolder:
    """What TQPagedAttention reads from a quantizer, for callers that bring the rotation and the codebook
    themselves."""

    def __init__(self, rotation: torch.Tensor, centroids: torch.Tensor, head_dim: int, bits: int):
        from .packing import packed_size
        self.rotation = rotation
        self.centroids = centroids.to(torch.float32).contiguous()
        self.head_dim = head_dim
        self.bits = bits
        self.num_levels = 1 << bits
        self._packed_dim = packed_size(head_dim, bits)

    def prepared_rotation(self):
        from .quantizer import prepared_rotation_for
        return prepared_rotation_for(self.rotation)


class TQPagedAttentionRef:
    """Constructor and forward() of the reference's pure-PyTorch class (fused_attention.py:53-185): rotation
    [head_dim, head_dim], centroids [2**bits], an explicit score scale, fixed head counts and block size.
    Here it runs the same HIP kernels as TQPagedAttention (there is no CPU path: tensors must live on the GPU);
    the results are those the golden vectors of the reference's class are checked against."""

    def __init__(self, rotation: torch.Tensor, centroids: torch.Tensor, scale: float, num_kv_heads: int,
                 num_query_heads: int, head_dim: int, block_size: int, bits: int = 4):
        self.rotation = rotation
        self.centroids = centroids
        self.scale = scale
        self.num_kv_heads = num_kv_heads
        self.num_query_heads = num_query_heads
        self.gqa_ratio = num_query_heads // num_kv_heads
        self.head_dim = head_dim
        self.block_size = block_size
        self.bits = bits
        self._impl = TQPagedAttention(_RotationHolder(rotation, centroids, head_dim, bits), num_query_heads)
        self._impl.scale = float(scale)

    def forward(self, query, k_packed, k_norms, v_packed, v_norms, block_tables, context_lens) -> torch.Tensor:
        """query [num_seqs, num_query_heads, head_dim] -> same shape and dtype."""
        return self._impl.forward(query, k_packed, k_norms, v_packed, v_norms, block_tables, context_lens,
                                  block_size=self.block_size, num_kv_heads=self.num_kv_heads)

