"""RoPE frequency table, pair-energy helpers, the pairwise form of the score and an orthonormal DCT
(reference: aither_kvcache/triattention/spectral.py:34-269).  The helpers are analysis tools (torch ops on
whatever device the tensor lives on); the hot path does not call them."""
import math
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


def trig_series_coefficients(q: torch.Tensor, k: torch.Tensor,
                             freq_indices: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per RoPE pair, the dot product c_i = q_e k_e + q_o k_o and the cross product s_i = q_o k_e - q_e k_o of the
    (even, odd) halves of q and k [..., head_dim]: the score of a key at distance Delta is
    sum_i c_i cos(Delta theta_i) + s_i sin(Delta theta_i).  `freq_indices` [..., F] restricts the pairs."""
    qp = q.reshape(*q.shape[:-1], q.shape[-1] // 2, 2)
    kp = k.reshape(*k.shape[:-1], k.shape[-1] // 2, 2)
    if freq_indices is not None:
        sel = freq_indices.long().unsqueeze(-1)
        qp = torch.gather(qp, -2, sel.expand(*sel.shape[:-1], 2))
        kp = torch.gather(kp, -2, sel.expand(*sel.shape[:-1], 2))
    c = (qp * kp).sum(-1)
    s = qp[..., 1] * kp[..., 0] - qp[..., 0] * kp[..., 1]
    return c, s


def rope_phase_matrix(positions_q: torch.Tensor, positions_k: torch.Tensor,
                      theta: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos and sin of (positions_k - positions_q) * theta: positions_q [B] or [B, 1], positions_k [B, S],
    theta [F] -> two tensors [B, S, F]."""
    delta = positions_k - positions_q.reshape(positions_q.shape[0], 1)
    ph = delta[..., None] * theta
    return torch.cos(ph), torch.sin(ph)


def dct_matrix(N: int, device: str = "cpu", dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Orthonormal DCT-II matrix: D[k, n] = w_k sqrt(2/N) cos(pi (2n + 1) k / (2N)), w_0 = 1/sqrt(2), else 1."""
    n = torch.arange(N, device=device, dtype=dtype)
    D = torch.cos(math.pi / (2 * N) * torch.outer(n, 2 * n + 1)) * math.sqrt(2.0 / N)
    D[0] = D[0] / math.sqrt(2.0)
    return D


def dct(x: torch.Tensor, D: Optional[torch.Tensor] = None) -> torch.Tensor:
    """DCT-II of the last axis (orthonormal); `D` may hold a precomputed dct_matrix."""
    if D is None:
        D = dct_matrix(x.shape[-1], device=x.device, dtype=x.dtype)
    return x @ D.T


def idct(x: torch.Tensor, D: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Inverse of dct (the matrix is orthogonal, so its transpose inverts it)."""
    if D is None:
        D = dct_matrix(x.shape[-1], device=x.device, dtype=x.dtype)
    return x @ D
