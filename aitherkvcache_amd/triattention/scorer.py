"""Trigonometric-series scores on MI355X (reference: aither_kvcache/triattention/scorer.py:43-226).

`score` returns the pre-softmax logits [B, QH, S]: for callers that add a mask or look at the scores.  The decode
step itself never materialises them (TriAttention.decode_step is one kernel over the spectral cache)."""
import math
from typing import Optional, Tuple

import torch

from .. import _lib
from .config import TriAttentionConfig
from .encoder import SpectralEncoding, packed_shape, unpack_coefficients
from .spectral import rope_frequencies


class TrigSeriesScorer:
    def __init__(self, config: TriAttentionConfig, device: str = "cpu"):
        self.config = config
        self.head_dim = config.head_dim
        self.num_pairs = config.num_pairs
        self.num_freqs = config.num_freqs
        self.coeff_bits = config.coeff_bits
        self.pre_rope = config.pre_rope
        self.scale = 1.0 / math.sqrt(config.head_dim)
        self.gqa_ratio = config.gqa_ratio
        # float32 table evaluated on the host exactly as the reference does, then moved
        self._theta = rope_frequencies(config.head_dim, config.rope_base, device="cpu").to(device)

    def to(self, device: str) -> "TrigSeriesScorer":
        self._theta = self._theta.to(device)
        return self

    def _unpack_coefficients(self, enc: SpectralEncoding) -> Tuple[torch.Tensor, torch.Tensor]:
        """(even, odd) float32 components [..., F] of an encoding (torch ops)."""
        return unpack_coefficients(enc.packed, enc.scales, self.coeff_bits)

    def score(self, query: torch.Tensor, k_enc: SpectralEncoding, query_pos: Optional[torch.Tensor] = None,
              key_positions: Optional[torch.Tensor] = None) -> torch.Tensor:
        """query [B, QH, D]; k_enc with indices [B, S, KVH, F]; query_pos [B] (default S); key_positions [B, S]
        (default 0..S-1) -> float32 logits [B, QH, S]."""
        dev = _lib.require_gpu(query, k_enc.indices, k_enc.packed, k_enc.scales, query_pos, key_positions)
        if self._theta.device != dev:
            self._theta = self._theta.to(dev)
        B, QH, D = query.shape
        _, S, KVH, F = k_enc.indices.shape
        if D != self.head_dim or QH % KVH != 0:
            raise ValueError(f"bad shapes: query {tuple(query.shape)}, encoding {tuple(k_enc.indices.shape)}")
        cshape, cdtype = packed_shape([B, S, KVH], F, self.coeff_bits)
        if k_enc.indices.dtype != torch.uint8 or k_enc.packed.dtype != cdtype or list(k_enc.packed.shape) != cshape:
            raise ValueError(f"encoding does not fit coeff_bits={self.coeff_bits}: packed {k_enc.packed.dtype} "
                             f"{list(k_enc.packed.shape)}, expected {cdtype} {cshape}")
        q = query if query.dtype in (torch.float16, torch.bfloat16, torch.float32) else query.float()
        q = q.contiguous()
        ki, kc = k_enc.indices.contiguous(), k_enc.packed.contiguous()
        ks = k_enc.scales.to(torch.float16).contiguous()

        def pos(t, shape):
            if t is None:
                return None
            if t.dtype not in (torch.int32, torch.int64):
                t = t.long()
            return t.expand(shape).contiguous()

        qp, kp = pos(query_pos, (B,)), pos(key_positions, (B, S))
        out = torch.empty(B, QH, S, dtype=torch.float32, device=dev)
        _lib.check(_lib.lib().akv_tri_scores(
            q.data_ptr(), _lib.dtype_code(q), ki.data_ptr(), kc.data_ptr(), ks.data_ptr(), self._theta.data_ptr(),
            _lib.ptr(qp), _lib.itype_code(qp) if qp is not None else 0,
            _lib.ptr(kp), _lib.itype_code(kp) if kp is not None else 0,
            out.data_ptr(), B, S, QH, KVH, D, F, self.coeff_bits, 1 if self.pre_rope else 0, _lib.stream_ptr(dev)))
        return out

    def score_single(self, query: torch.Tensor, k_enc: SpectralEncoding, query_pos: int,
                     key_positions: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One query [1, QH, D] at an integer position against all keys -> [1, QH, S]."""
        return self.score(query, k_enc, torch.tensor([query_pos], device=query.device), key_positions)
