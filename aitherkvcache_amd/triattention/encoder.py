"""Spectral KV encoding (write side of TriAttention).

Keeps the F RoPE pairs (dims 2i, 2i+1) of largest energy per token, ascending by index, and
quantises their 2F values against the token's max-abs scale to 4 bits (a byte per pair) or 8 bits (two
bytes per pair), or keeps them as float16 (coeff_bits 16) (reference:
aither_kvcache/triattention/encoder.py:73-149).  On an MI355X tensor with head_dim <= 128 this is one
HIP kernel (akv_tri_encode); host tensors and wider heads take the same steps as torch ops.
"""
from typing import NamedTuple, Optional

import torch

from .. import _lib
from .config import TriAttentionConfig


class SpectralEncoding(NamedTuple):
    indices: torch.Tensor   # [..., F] uint8   retained pair indices, ascending
    packed: torch.Tensor    # coeff_bits 4: [..., F] uint8, code(even) << 4 | code(odd); 8: [..., 2F] uint8,
                            # code(even), code(odd) per pair; 16: [..., F, 2] float16, the components
    scales: torch.Tensor    # [...]    float16 max |coefficient| of the token (ones for coeff_bits 16)


def packed_shape(batch, num_freqs: int, coeff_bits: int):
    """Shape and dtype of SpectralEncoding.packed for a batch shape (encoder.py:107-147 of the reference)."""
    batch = list(batch)
    if coeff_bits == 4:
        return batch + [num_freqs], torch.uint8
    if coeff_bits == 8:
        return batch + [2 * num_freqs], torch.uint8
    if coeff_bits == 16:
        return batch + [num_freqs, 2], torch.float16
    raise ValueError(f"Unsupported coeff_bits: {coeff_bits}")


def unpack_coefficients(packed: torch.Tensor, scales: torch.Tensor, coeff_bits: int):
    """(even, odd) float32 components [..., F] of an encoding, with the reference's arithmetic
    (scorer.py:84-113): (code / half - 1) * scale for 4 and 8 bits, the float16 values for 16."""
    if coeff_bits == 16:
        return packed[..., 0].float(), packed[..., 1].float()
    s = scales.float().unsqueeze(-1)
    if coeff_bits == 4:
        return ((packed >> 4).float() / 7.5 - 1.0) * s, ((packed & 0x0F).float() / 7.5 - 1.0) * s
    if coeff_bits == 8:
        raw = packed.float().reshape(*packed.shape[:-1], packed.shape[-1] // 2, 2)
        return (raw[..., 0] / 127.5 - 1.0) * s, (raw[..., 1] / 127.5 - 1.0) * s
    raise ValueError(f"Unsupported coeff_bits: {coeff_bits}")


class SpectralKVEncoder:
    def __init__(self, config: TriAttentionConfig):
        if config.coeff_bits not in (4, 8, 16):
            raise ValueError(f"Unsupported coeff_bits: {config.coeff_bits}")
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
            cshape, cdtype = packed_shape([n], F, self.coeff_bits)
            cf = torch.empty(cshape, dtype=cdtype, device=x.device)
            sc = torch.empty(n, dtype=torch.float16, device=x.device)
            _lib.check(_lib.lib().akv_tri_encode(
                xf.data_ptr(), _lib.dtype_code(xf), n, self.head_dim, xf.stride(0) if n else self.head_dim, F,
                self.coeff_bits, idx.data_ptr(), cf.data_ptr(), sc.data_ptr(), _lib.stream_ptr(x.device)))
            return SpectralEncoding(idx.reshape(batch + [F]), cf.reshape(batch + cshape[1:]), sc.reshape(batch))
        pairs = x.reshape(*x.shape[:-1], self.num_pairs, 2).float()
        energy = pairs.pow(2).sum(-1)
        keep = energy.topk(F, dim=-1).indices.sort(dim=-1).values
        vals = torch.gather(pairs, -2, keep.unsqueeze(-1).expand(*keep.shape, 2))
        if self.coeff_bits == 16:
            return SpectralEncoding(keep.to(torch.uint8), vals.to(torch.float16),
                                    torch.ones(x.shape[:-1], dtype=torch.float16, device=x.device))
        scales = vals.abs().flatten(-2).amax(-1).clamp(min=1e-8)
        half, top = (7.5, 15) if self.coeff_bits == 4 else (127.5, 255)
        codes = ((vals / scales[..., None, None] + 1) * half).round().clamp(0, top).to(torch.uint8)
        packed = (codes[..., 0] << 4) | codes[..., 1] if self.coeff_bits == 4 else codes.flatten(-2)
        return SpectralEncoding(keep.to(torch.uint8), packed, scales.to(torch.float16))

    def decode(self, enc: SpectralEncoding) -> torch.Tensor:
        """Dense [..., head_dim] float32 reconstruction (zeros at the discarded pairs)."""
        v0, v1 = unpack_coefficients(enc.packed, enc.scales, self.coeff_bits)
        idx = enc.indices.long()
        out = torch.zeros(*idx.shape[:-1], self.head_dim, dtype=torch.float32, device=idx.device)
        out.scatter_(-1, idx * 2, v0)
        out.scatter_(-1, idx * 2 + 1, v1)
        return out

    def encode_adaptive(self, x: torch.Tensor, min_energy_ratio: Optional[float] = None,
                        max_freqs: Optional[int] = None):
        """Encode with as many pairs as the most demanding vector of the batch needs to reach
        `min_energy_ratio` of its pair energy, between num_freqs and max_freqs (reference: encoder.py:205-241).
        Returns (encoding, pairs needed per vector)."""
        from .spectral import pair_energy_profile
        if min_energy_ratio is None:
            min_energy_ratio = self.config.min_energy_ratio
        if max_freqs is None:
            max_freqs = self.num_pairs
        prof = pair_energy_profile(x.float())
        share = prof.cumsum(-1) / (prof.sum(-1, keepdim=True) + 1e-12)
        needed = ((share >= min_energy_ratio).float().argmax(dim=-1) + 1).clamp(self.num_freqs, max_freqs)
        return self.encode(x, num_freqs=int(needed.max().item())), needed

    def compression_stats(self, x: torch.Tensor) -> dict:
        """Compression ratio, retained energy, reconstruction error of `x` (reference: encoder.py:243-270)."""
        from .spectral import spectral_concentration
        dec = self.decode(self.encode(x)).float()
        xf = x.float().to(dec.device)
        return {
            "num_freqs": self.num_freqs,
            "coeff_bits": self.coeff_bits,
            "bytes_per_token": self.config.bytes_per_kv_token,
            "compression_ratio": self.config.compression_ratio,
            "mse": (xf - dec).square().mean().item(),
            "energy_ratio": spectral_concentration(xf, self.num_freqs).mean().item(),
            "cosine_similarity": torch.nn.functional.cosine_similarity(
                xf.reshape(-1, self.head_dim), dec.reshape(-1, self.head_dim), dim=-1).mean().item(),
        }
