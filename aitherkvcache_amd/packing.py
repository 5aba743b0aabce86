"""Packed-code sizes.  The bit layouts themselves (reference: aither_kvcache/packing.py:13-118)
are produced and consumed inside the HIP kernels:

  4-bit  byte k = idx[2k] << 4 | idx[2k+1]
  2-bit  byte k = idx[4k] << 6 | idx[4k+1] << 4 | idx[4k+2] << 2 | idx[4k+3]
  3-bit  8 indices -> one 24-bit big-endian word, index i in bits 23-3i .. 21-3i

i.e. all three are one MSB-first bit stream with `bits` bits per index.
"""


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
