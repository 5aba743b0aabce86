"""Rotation matrices for TurboQuant (init-time host code; the kernels consume the result).

Mirrors aither_kvcache/rotation.py of the reference: the same torch calls in the same
order, so that the same seed yields the same matrix on the same torch / LAPACK build.
"""
import math

import torch


def random_orthogonal(d: int, seed: int = 42, device: str = "cuda",
                      dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Haar-distributed orthogonal matrix: QR of a seeded CPU Gaussian, columns re-signed by
    sign(diag(R)) with 0 -> +1 (reference: rotation.py:20-35)."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    gauss = torch.randn(d, d, generator=g, dtype=dtype)
    q, r = torch.linalg.qr(gauss)
    s = torch.sign(torch.diagonal(r))
    s = torch.where(s == 0, torch.ones_like(s), s)
    return (q * s[None, :]).to(device=device)


def hadamard_matrix(d: int, dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Normalised Walsh-Hadamard matrix (Sylvester construction), H H^T = I
    (reference: rotation.py:38-50)."""
    if d <= 0 or d & (d - 1):
        raise AssertionError(f"d must be power of 2, got {d}")
    h = torch.ones(1, 1, dtype=dtype)
    while h.shape[0] < d:
        h = torch.cat([torch.cat([h, h], 1), torch.cat([h, -h], 1)], 0)
    return h / math.sqrt(d)


def random_signs(d: int, seed: int = 42, device: str = "cuda") -> torch.Tensor:
    """Seeded Rademacher vector (reference: rotation.py:53-57)."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return (2 * torch.randint(0, 2, (d,), generator=g, dtype=torch.float32) - 1).to(device)


def randomized_hadamard_matrix(d: int, seed: int = 42, device: str = "cuda",
                               dtype: torch.dtype = torch.float32,
                               num_rounds: int = 3) -> torch.Tensor:
    """Dense (H D_k) ... (H D_1) with seeds seed, seed+1, ... (reference: rotation.py:60-80).
    The quantizer treats the result like any other dense rotation."""
    h = hadamard_matrix(d, dtype=dtype).to(device)
    m = torch.eye(d, dtype=dtype, device=device)
    for r in range(num_rounds):
        m = h @ torch.diag(random_signs(d, seed=seed + r, device=device).to(dtype)) @ m
    return m


def fast_hadamard_transform(x: torch.Tensor) -> torch.Tensor:
    """Unnormalised Walsh-Hadamard transform of the last axis by butterflies
    (reference: rotation.py:83-108).  Init/diagnostic helper; not used on the hot path."""
    d = x.shape[-1]
    if d <= 0 or d & (d - 1):
        raise AssertionError(f"last dim must be power of 2, got {d}")
    y = x.clone()
    h = 1
    while h < d:
        v = y.reshape(*y.shape[:-1], d // (2 * h), 2, h)
        y = torch.stack([v[..., 0, :] + v[..., 1, :], v[..., 0, :] - v[..., 1, :]], dim=-2)
        y = y.reshape(*x.shape[:-1], d)
        h *= 2
    return y
