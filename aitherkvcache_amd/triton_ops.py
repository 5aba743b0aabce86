"""Quantize+pack / unpack+lookup entry points with the names the reference exports from
aither_kvcache/triton_ops.py:220-259.  They launch HIP kernels (no Triton involved); the
module and function names are kept so that callers of the reference keep working.

Two differences, both deliberate: exact ties (y equal to a boundary) go to the LOWER bin like
the reference's torch path (quantizer.py:203-207) rather than the upper one like its Triton
kernels, and 3-bit is implemented (the reference's 3-bit kernel is an empty stub).
"""
import torch

from . import _lib
from .packing import packed_size

HAS_HIP = _lib.available()
HAS_TRITON = HAS_HIP  # the flag callers gate on (quantizer.py:113-120 of the reference)


def hip_quantize(y: torch.Tensor, boundaries: torch.Tensor, bits: int) -> torch.Tensor:
    """y [N, D] float32 -> packed [N, packed_size(D, bits)] uint8."""
    assert y.is_cuda, "HIP kernels require device tensors"
    dev = _lib.require_gpu(y, boundaries)
    y = y.float()
    if y.stride(-1) != 1:
        y = y.contiguous()
    n, d = y.shape
    out = torch.empty(n, packed_size(d, bits), dtype=torch.uint8, device=dev)
    b = boundaries.float().contiguous()
    _lib.check(_lib.lib().akv_quantize_pack(y.data_ptr(), n, d, y.stride(0) if n else d, b.data_ptr(),
                                            bits, out.data_ptr(), out.shape[1], _lib.stream_ptr(dev)))
    return out


def hip_dequantize(packed: torch.Tensor, centroids: torch.Tensor, D: int, bits: int) -> torch.Tensor:
    """packed [N, packed_size(D, bits)] uint8 -> centroids[idx] [N, D] float32."""
    assert packed.is_cuda, "HIP kernels require device tensors"
    dev = _lib.require_gpu(packed, centroids)
    if packed.stride(-1) != 1:
        packed = packed.contiguous()
    n = packed.shape[0]
    out = torch.empty(n, D, dtype=torch.float32, device=dev)
    c = centroids.float().contiguous()
    _lib.check(_lib.lib().akv_unpack_lookup(packed.data_ptr(), n, D, packed.stride(0) if n else 1,
                                            c.data_ptr(), bits, out.data_ptr(), D, _lib.stream_ptr(dev)))
    return out


def triton_quantize_4bit(y, boundaries):
    return hip_quantize(y, boundaries, 4)


def triton_dequantize_4bit(packed, centroids, D):
    return hip_dequantize(packed, centroids, D, 4)


def triton_quantize_2bit(y, boundaries):
    return hip_quantize(y, boundaries, 2)


def triton_dequantize_2bit(packed, centroids, D):
    return hip_dequantize(packed, centroids, D, 2)


def triton_quantize_3bit(y, boundaries):
    return hip_quantize(y, boundaries, 3)


def triton_dequantize_3bit(packed, centroids, D):
    return hip_dequantize(packed, centroids, D, 3)
