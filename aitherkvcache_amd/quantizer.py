"""TurboQuant quantizer on MI355X: same interface as the reference's
aither_kvcache/quantizer.py (TurboQuantConfig, TurboQuant.encode/decode/validate/benchmark/...),
with encode and decode each running as one HIP kernel through the C ABI.

encode:  norm -> x/(norm+1e-10) -> rotation -> codebook search -> bit packing   (quantizer.py:122-166)
decode:  unpack -> centroid lookup -> inverse rotation -> * norm -> cast        (quantizer.py:168-197)

Tensors must live on a HIP device; there is no CPU implementation.
"""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _lib
from .codebook import get_codebook, get_theory_bounds
from .packing import packed_size
from .rotation import random_orthogonal, randomized_hadamard_matrix

_KERNEL_HEAD_DIMS = (64, 128, 256, 512)


@dataclass
class TurboQuantConfig:
    """Same fields and defaults as the reference (quantizer.py:36-47).  `use_triton` is kept
    for call compatibility; the HIP kernels are always used."""
    head_dim: int = 128
    bits: int = 4
    seed: int = 42
    use_hadamard: bool = False
    hadamard_rounds: int = 3
    device: str = "cuda"
    dtype: torch.dtype = torch.float16
    use_triton: bool = True


def _rotation_key(rotation: torch.Tensor):
    """What tells one matrix from another without reading it: where it lies, how it is laid out there (a
    transposed view shares address and version with its base) and how often it has been written."""
    return (rotation.data_ptr(), rotation._version, rotation.stride(), rotation.dtype, str(rotation.device))


class PreparedRotation:
    """Device buffer with the layouts of the rotation the kernels read (Pi, Pi^T and the MFMA
    operand tiles), produced by akv_rotation_prepare."""

    def __init__(self, rotation: torch.Tensor):
        _lib.require_gpu(rotation)
        d = rotation.shape[0]
        if rotation.shape != (d, d):
            raise ValueError(f"rotation must be square, got {tuple(rotation.shape)}")
        self.head_dim = d
        # (the tensor the key below is taken from stays referenced: while this object lives, e.g. in the cache of
        # prepared_rotation_for, its address cannot be handed to another tensor that would then match the key)
        self._origin = rotation
        self.source = rotation.detach().to(torch.float32).contiguous()
        L = _lib.lib()
        nbytes = L.akv_rotation_prepared_bytes(d)
        self.buffer = torch.empty(nbytes, dtype=torch.uint8, device=rotation.device)
        _lib.check(L.akv_rotation_prepare(self.source.data_ptr(), d, self.buffer.data_ptr(), nbytes,
                                          _lib.stream_ptr(rotation.device)))
        self._key = _rotation_key(rotation)

    def matches(self, rotation: torch.Tensor) -> bool:
        return self._key == _rotation_key(rotation)

    @property
    def ptr(self) -> int:
        return self.buffer.data_ptr()


_PREPARED_CACHE: dict = {}


def prepared_rotation_for(rotation: torch.Tensor) -> PreparedRotation:
    """Prepared form of an arbitrary rotation tensor, cached per storage address, layout and version
    (used by the entry points that receive `rotation` as an argument, like
    fused_tq4_kv_update)."""
    key = _rotation_key(rotation)
    hit = _PREPARED_CACHE.get(key)
    if hit is None:
        if len(_PREPARED_CACHE) > 64:
            _PREPARED_CACHE.clear()
        hit = PreparedRotation(rotation)
        _PREPARED_CACHE[key] = hit
    return hit


class TurboQuant:
    """TurboQuant KV-cache quantizer (2, 3 or 4 bits per coordinate).

    tq = TurboQuant(head_dim=128, bits=4)
    packed, norms = tq.encode(kv)          # uint8 [..., packed_dim], float32 [...]
    kv_hat = tq.decode(packed, norms)      # [..., head_dim] in tq.dtype
    """

    def __init__(self, config: Optional[TurboQuantConfig] = None, **kwargs):
        if config is None:
            config = TurboQuantConfig(**kwargs)
        self.config = config
        self.head_dim = config.head_dim
        self.bits = config.bits
        self.num_levels = 1 << config.bits
        self.device = config.device
        self.dtype = config.dtype

        if config.bits not in (2, 3, 4):
            raise ValueError(f"Supported bit-widths: 2, 3, 4. Got {config.bits}")
        if config.head_dim <= 0 or (config.head_dim & (config.head_dim - 1)) != 0:
            raise ValueError(f"head_dim must be power of 2, got {config.head_dim}")

        if config.use_hadamard:
            rot = randomized_hadamard_matrix(config.head_dim, seed=config.seed, device="cpu",
                                             num_rounds=config.hadamard_rounds)
        else:
            rot = random_orthogonal(config.head_dim, seed=config.seed, device="cpu")
        self._rotation = rot.to(config.device)
        self._prepared: Optional[PreparedRotation] = None

        centroids, boundaries, mse_total = get_codebook(config.head_dim, config.bits)
        self.centroids = torch.tensor(centroids, dtype=torch.float32, device=config.device)
        self.boundaries_inner = torch.tensor(boundaries, dtype=torch.float32, device=config.device)
        self.mse_total = mse_total
        self.theory_lower, self.theory_upper = get_theory_bounds(config.bits)
        self._packed_dim = packed_size(config.head_dim, config.bits)
        # The reference reports whether its Triton kernels are active; here the HIP kernels
        # are the only engine.
        self._use_triton = False
        self._use_hip = True

    # -- rotation (assignable, like the reference's plain attribute) --------------------
    @property
    def rotation(self) -> torch.Tensor:
        return self._rotation

    @rotation.setter
    def rotation(self, value: torch.Tensor) -> None:
        self._rotation = value
        self._prepared = None

    def prepared_rotation(self) -> PreparedRotation:
        if self._prepared is None or not self._prepared.matches(self._rotation):
            self._prepared = PreparedRotation(self._rotation)
        return self._prepared

    def _check_kernel_dim(self) -> None:
        if self.head_dim not in _KERNEL_HEAD_DIMS:
            raise NotImplementedError(
                f"HIP kernels are built for head_dim in {_KERNEL_HEAD_DIMS}, got {self.head_dim}")

    # -- encode / decode ------------------------------------------------------------------
    def encode(self, x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """[..., head_dim] float16/bfloat16/float32 -> (uint8 [..., packed_dim], float32 [...])."""
        assert x.shape[-1] == self.head_dim, f"Expected last dim {self.head_dim}, got {x.shape[-1]}"
        self._check_kernel_dim()
        dev = _lib.require_gpu(x, self._rotation)
        batch = list(x.shape[:-1])
        if x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
            x = x.float()
        xf = x.reshape(-1, self.head_dim)
        if xf.stride(-1) != 1:
            xf = xf.contiguous()
        n = xf.shape[0]
        packed = torch.empty(n, self._packed_dim, dtype=torch.uint8, device=dev)
        norms = torch.empty(n, dtype=torch.float32, device=dev)
        _lib.check(_lib.lib().akv_encode(
            xf.data_ptr(), _lib.dtype_code(xf), n, self.head_dim, xf.stride(0) if n else self.head_dim,
            self.prepared_rotation().ptr, self.boundaries_inner.data_ptr(), self.bits,
            packed.data_ptr(), self._packed_dim, norms.data_ptr(), _lib.stream_ptr(dev)))
        return packed.reshape(batch + [self._packed_dim]), norms.reshape(batch)

    def decode(self, packed: torch.Tensor, norms: torch.Tensor) -> torch.Tensor:
        """(uint8 [..., packed_dim], norms [...]) -> [..., head_dim] in self.dtype."""
        self._check_kernel_dim()
        dev = _lib.require_gpu(packed, norms, self._rotation)
        batch = list(norms.shape)
        pf = packed.reshape(-1, packed.shape[-1])
        if pf.stride(-1) != 1:
            pf = pf.contiguous()
        nf = norms.reshape(-1).float().contiguous()
        n = nf.shape[0]
        out_dtype = self.dtype if self.dtype in (torch.float16, torch.bfloat16, torch.float32) else torch.float32
        out = torch.empty(n, self.head_dim, dtype=out_dtype, device=dev)
        _lib.check(_lib.lib().akv_decode(
            pf.data_ptr(), pf.stride(0) if n else self._packed_dim, nf.data_ptr(), n, self.head_dim,
            self.prepared_rotation().ptr, self.centroids.data_ptr(), self.bits,
            out.data_ptr(), _lib.dtype_code(out), self.head_dim, _lib.stream_ptr(dev)))
        return out.reshape(batch + [self.head_dim]).to(self.dtype)

    # -- analysis (same figures as the reference, quantizer.py:236-370) -----------------------
    def compression_ratio(self) -> float:
        return (self.head_dim * 2) / (self._packed_dim + 4)

    def compression_ratio_vs_fp8(self) -> float:
        return self.head_dim / (self._packed_dim + 4)

    def memory_report(self, seq_len: int, num_layers: int = 32, num_kv_heads: int = 8) -> dict:
        vectors = seq_len * num_layers * num_kv_heads * 2
        fp16 = vectors * self.head_dim * 2
        fp8 = vectors * self.head_dim
        tq = vectors * (self._packed_dim + 4)
        return {
            "config": f"TQ{self.bits} d={self.head_dim} seq={seq_len} L={num_layers} H={num_kv_heads}",
            "fp16_mb": fp16 / 2 ** 20,
            "fp8_mb": fp8 / 2 ** 20,
            f"tq{self.bits}_mb": tq / 2 ** 20,
            "ratio_vs_fp16": fp16 / tq,
            "ratio_vs_fp8": fp8 / tq,
        }

    def validate(self, num_vectors: int = 10000, device: Optional[str] = None) -> dict:
        """Round trip of random unit vectors: MSE, inner-product error, theory bounds."""
        dev = device or self.device
        x = torch.randn(num_vectors, self.head_dim, device=dev, dtype=torch.float32)
        x = x / x.norm(dim=-1, keepdim=True)
        packed, norms = self.encode(x)
        x_hat = self.decode(packed, norms).float()
        mse = (x - x_hat).pow(2).sum(-1).mean().item()
        n = min(num_vectors, 5000)
        ia = torch.randint(0, num_vectors, (n,), device=dev)
        ib = torch.randint(0, num_vectors, (n,), device=dev)
        true_ip = (x[ia] * x[ib]).sum(-1)
        est_ip = (x_hat[ia] * x[ib]).sum(-1)
        return {
            "bits": self.bits,
            "head_dim": self.head_dim,
            "num_vectors": num_vectors,
            "mse": mse,
            "mse_theory_lower": self.theory_lower,
            "mse_theory_upper": self.theory_upper,
            "mse_ratio_to_lower": mse / self.theory_lower if self.theory_lower > 0 else float("inf"),
            "ip_mse": (true_ip - est_ip).pow(2).mean().item(),
            "ip_bias": (est_ip - true_ip).mean().item(),
            "max_abs_error": (x - x_hat).abs().max().item(),
            "compression_vs_fp16": self.compression_ratio(),
            "compression_vs_fp8": self.compression_ratio_vs_fp8(),
            "triton_active": self._use_triton,
            "hip_active": self._use_hip,
        }

    def benchmark(self, num_vectors: int = 32768, warmup: int = 10, iters: int = 100,
                  device: Optional[str] = None) -> dict:
        """Wall-clock encode/decode throughput the way the reference measures it
        (quantizer.py:317-362): warm-up, then `iters` calls bracketed by a device sync."""
        dev = device or self.device
        x = torch.randn(num_vectors, self.head_dim, device=dev, dtype=torch.float16)
        for _ in range(warmup):
            p, n = self.encode(x)
            self.decode(p, n)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            p, n = self.encode(x)
        torch.cuda.synchronize()
        encode_us = (time.perf_counter() - t0) / iters * 1e6
        t0 = time.perf_counter()
        for _ in range(iters):
            self.decode(p, n)
        torch.cuda.synchronize()
        decode_us = (time.perf_counter() - t0) / iters * 1e6
        return {
            "bits": self.bits,
            "num_vectors": num_vectors,
            "encode_us": encode_us,
            "decode_us": decode_us,
            "encode_throughput_mvec_s": num_vectors / encode_us,
            "decode_throughput_mvec_s": num_vectors / decode_us,
            "triton_active": self._use_triton,
            "hip_active": self._use_hip,
            "device": dev,
        }

    def __repr__(self) -> str:
        return (f"TurboQuant(d={self.head_dim}, bits={self.bits}, "
                f"compress={self.compression_ratio():.1f}x, mse={self.mse_total:.4f}, engine=HIP)")
