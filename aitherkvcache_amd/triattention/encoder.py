"""Spectral KV encoding (write side of TriAttention).

Keeps the F RoPE pairs (dims 2i, 2i+1) of largest energy per token, ascending by index, and
quantises their 2F values to 4 bits against the token's max-abs scale (reference:
aither_kvcache/triattention/encoder.py:73-133).  On an MI355X tensor with head_dim <= 128 this is one
HIP kernel (akv_tri_encode); host tensors and wider heads take the same steps as torch ops.
"""
from typing import NamedTuple, Optional

import torch

from .. import _lib
from .config import TriAttentionConfig


class SpectralEncoding(NamedTuple):
    indices: torch.Tensor   # [..., F] uint8   retained pair indices, ascending
    packed: torch.Tensor    # [..., F] uint8   code(even) << 4 | code(odd)
    scales: torch.Tensor    # [...]    float16 max |coefficient| of the token


class SpectralKVEncoder:
    def __init__(self, config: TriAttentionConfig):
        if config.coeff_bits != 4:
            raise NotImplementedError("only int4 coefficients (coeff_bits=4) are built")
        self.config = config
        self.head_dim = config.head_dim
        self.num_pairs = config.num_pairs
        self.num_freqs = config.num_freqs
        self.coeff_bits = config.coeff_bits

    def encode(self, x: torch.Tensor, num_freqs: Optional[int] = None) -> SpectralEncoding:
        F = num_freqs or self.num_freqs
        if x.is_cuda and self.head_dim <= 128 and x.dtype in (torch.float16, torch.bfloat16, torch.float32):
            batch = list(x.shape[:-1])
            xf = x.reshape(-1, self.head_dim)
            if xf.stride(-1) != 1:
                xf = xf.contiguous()
            n = xf.shape[0]
            idx = torch.empty(n, F, dtype=torch.uint8, device=x.device)
            cf = torch.empty(n, F, dtype=torch.uint8, device=x.device)
            sc = torch.empty(n, dtype=torch.float16, device=x.device)
            _lib.check(_lib.lib().akv_tri_encode(
                xf.data_ptr(), _lib.dtype_code(xf), n, self.head_dim, xf.stride(0) if n else self.head_dim, F,
                idx.data_ptr(), cf.data_ptr(), sc.data_ptr(), _lib.stream_ptr(x.device)))
            return SpectralEncoding(idx.reshape(batch + [F]), cf.reshape(batch + [F]), sc.reshape(batch))
        pairs = x.reshape(*x.shape[:-1], self.num_pairs, 2).float()
        energy = pairs.pow(2).sum(-1)
        keep = energy.topk(F, dim=-1).indices.sort(dim=-1).values
        vals = torch.gather(pairs, -2, keep.unsqueeze(-1).expand(*keep.shape, 2))
        scales = vals.abs().flatten(-2).amax(-1).clamp(min=1e-8)
        codes = ((vals / scales[..., None, None] + 1) * 7.5).round().clamp(0, 15).to(torch.uint8)
        return SpectralEncoding(keep.to(torch.uint8), (codes[..., 0] << 4) | codes[..., 1],
                                scales.to(torch.float16))

    def decode(self, enc: SpectralEncoding) -> torch.Tensor:
        """Dense [..., head_dim] float32 reconstruction (zeros at the discarded pairs)."""
        s = enc.scales.float().unsqueeze(-1)
        v0 = ((enc.packed >> 4).float() / 7.5 - 1.0) * s
        v1 = ((enc.packed & 0x0F).float() / 7.5 - 1.0) * s
        idx = enc.indices.long()
        out = torch.zeros(*idx.shape[:-1], self.head_dim, dtype=torch.float32, device=idx.device)
        out.scatter_(-1, idx * 2, v0)
        out.scatter_(-1, idx * 2 + 1, v1)
        return out
