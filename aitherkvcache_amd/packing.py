"""Packed-code layouts and sizes (reference: aither_kvcache/packing.py:13-131).

All three bit widths are ONE MSB-first bit stream with `bits` bits per index:

  4-bit  byte k = idx[2k] << 4 | idx[2k+1]
  2-bit  byte k = idx[4k] << 6 | idx[4k+1] << 4 | idx[4k+2] << 2 | idx[4k+3]
  3-bit  8 indices -> one 24-bit big-endian word, index i in bits 23-3i .. 21-3i

The hot path never calls these helpers -- the HIP kernels pack while they encode and unpack while
they attend or decode.  They are the reference's public host-side utilities (plain torch integer
ops on whatever device the tensor lives on), kept so that callers which import them keep working;
one generic routine per direction serves the three widths.
"""
import torch

# bits -> (indices per group, bytes per group): the smallest run of indices that fills whole bytes
_GROUP = {4: (2, 1), 3: (8, 3), 2: (4, 1)}


def _pack_stream(indices: torch.Tensor, bits: int) -> torch.Tensor:
    per, nbytes = _GROUP[bits]
    d = indices.shape[-1]
    assert d % per == 0, f"Dimension must be divisible by {per} for {bits}-bit packing, got {d}"
    grp = (indices.to(torch.int32) & ((1 << bits) - 1)).reshape(*indices.shape[:-1], d // per, per)
    shifts = torch.arange(per - 1, -1, -1, dtype=torch.int32, device=indices.device) * bits
    word = (grp << shifts).sum(dim=-1, dtype=torch.int32)                   # disjoint bit fields: sum == or
    byte_shifts = torch.arange(nbytes - 1, -1, -1, dtype=torch.int32, device=indices.device) * 8
    out = ((word.unsqueeze(-1) >> byte_shifts) & 0xFF).to(torch.uint8)
    return out.reshape(*indices.shape[:-1], (d // per) * nbytes)


def _unpack_stream(packed: torch.Tensor, dim: int, bits: int) -> torch.Tensor:
    per, nbytes = _GROUP[bits]
    groups = dim // per
    raw = packed[..., :groups * nbytes].to(torch.int32).reshape(*packed.shape[:-1], groups, nbytes)
    byte_shifts = torch.arange(nbytes - 1, -1, -1, dtype=torch.int32, device=packed.device) * 8
    word = (raw << byte_shifts).sum(dim=-1, dtype=torch.int32)
    shifts = torch.arange(per - 1, -1, -1, dtype=torch.int32, device=packed.device) * bits
    out = ((word.unsqueeze(-1) >> shifts) & ((1 << bits) - 1)).to(torch.uint8)
    return out.reshape(*packed.shape[:-1], groups * per)


def pack_4bit(indices: torch.Tensor) -> torch.Tensor:
    """[..., D] values in [0, 15] -> [..., D // 2] uint8 (reference: packing.py:13-23)."""
    return _pack_stream(indices, 4)


def unpack_4bit(packed: torch.Tensor, dim: int) -> torch.Tensor:
    """[..., D // 2] uint8 -> [..., D] uint8 in [0, 15] (reference: packing.py:26-37)."""
    return _unpack_stream(packed, dim, 4)


def pack_2bit(indices: torch.Tensor) -> torch.Tensor:
    """[..., D] values in [0, 3] -> [..., D // 4] uint8 (reference: packing.py:40-52)."""
    return _pack_stream(indices, 2)


def unpack_2bit(packed: torch.Tensor, dim: int) -> torch.Tensor:
    """[..., D // 4] uint8 -> [..., D] uint8 in [0, 3] (reference: packing.py:55-70)."""
    return _unpack_stream(packed, dim, 2)


def pack_3bit(indices: torch.Tensor) -> torch.Tensor:
    """[..., D] values in [0, 7] -> [..., D * 3 // 8] uint8 (reference: packing.py:73-98)."""
    return _pack_stream(indices, 3)


def unpack_3bit(packed: torch.Tensor, dim: int) -> torch.Tensor:
    """[..., D * 3 // 8] uint8 -> [..., D] uint8 in [0, 7] (reference: packing.py:101-118)."""
    return _unpack_stream(packed, dim, 3)


def packed_size(dim: int, bits: int) -> int:
    """Bytes that hold `dim` indices of `bits` bits (reference: packing.py:121-131)."""
    if bits == 4:
        return dim // 2
    if bits == 3:
        assert dim % 8 == 0
        return dim * 3 // 8
    if bits == 2:
        return dim // 4
    raise ValueError(f"Unsupported bit-width: {bits}")
