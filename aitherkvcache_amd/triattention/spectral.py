"""RoPE frequency table (reference: aither_kvcache/triattention/spectral.py:34-51)."""
import torch


def rope_frequencies(head_dim: int, base: float = 1_000_000.0, device: str = "cpu",
                     dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """theta_i = base ** (-2 i / head_dim), i = 0 .. head_dim/2 - 1, evaluated in `dtype`."""
    i = torch.arange(head_dim // 2, device=device, dtype=dtype)
    return base ** (-2.0 * i / head_dim)
