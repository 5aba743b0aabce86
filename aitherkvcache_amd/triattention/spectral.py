"""RoPE frequency table and pair-energy helpers (reference: aither_kvcache/triattention/spectral.py:34-140).
The helpers are analysis tools (torch ops on whatever device the tensor lives on); the hot path does not call them."""
from typing import Optional, Tuple

import torch


def rope_frequencies(head_dim: int, base: float = 1_000_000.0, device: str = "cpu",
                     dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """theta_i = base ** (-2 i / head_dim), i = 0 .. head_dim/2 - 1, evaluated in `dtype`."""
    i = torch.arange(head_dim // 2, device=device, dtype=dtype)
    return base ** (-2.0 * i / head_dim)


def pair_energies(x: torch.Tensor) -> torch.Tensor:
    """E_i = x[2i]^2 + x[2i+1]^2 -> [..., head_dim / 2]."""
    return x.reshape(*x.shape[:-1], x.shape[-1] // 2, 2).square().sum(-1)


def topk_pairs(x: torch.Tensor, k: int, return_values: bool = True) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Indices (uint8, ascending) of the k pairs of largest energy and, optionally, their values [..., k, 2]."""
    keep = pair_energies(x).topk(k, dim=-1).indices.sort(dim=-1).values
    if not return_values:
        return keep.to(torch.uint8), None
    pairs = x.reshape(*x.shape[:-1], x.shape[-1] // 2, 2)
    return keep.to(torch.uint8), torch.gather(pairs, -2, keep.unsqueeze(-1).expand(*keep.shape, 2))


def spectral_concentration(x: torch.Tensor, k: int) -> torch.Tensor:
    """Share of the pair energy held by the k strongest pairs, per vector."""
    e = pair_energies(x)
    return e.topk(k, dim=-1).values.sum(-1) / (e.sum(-1) + 1e-12)


def pair_energy_profile(x: torch.Tensor) -> torch.Tensor:
    """Pair energies in descending order."""
    return pair_energies(x).sort(dim=-1, descending=True).values
