"""Hybrid bit-width quantizer (tq35, tq25) on MI355X, with the interface of the reference's
aither_kvcache/hybrid_quantizer.py (HybridTurboQuant.encode/decode/calibrate_uniform, layouts).

tq35: a 128-d vector is split into dims [0,64) and [64,128).  Each half is L2-normalised, rotated
by a sign-flipped 64-point Walsh-Hadamard transform, scalar-quantised (3-bit / 2-bit
Lloyd-Max codebook of the sphere-coordinate Beta law), and the residual is sketched with one
sign bit per coordinate after a second sign-flipped Hadamard transform (QJL).  The two norms
of a half travel as fp16 inside the 64-byte row (hybrid_quantizer.py:92-123,706-779).
tq25: dims [0,32) at 2 bits and [32,128) at 1 bit, 44-byte rows; the 96 coordinates of the second
group are transformed as a 64-point and a 32-point block and divided by sqrt(96), as the reference's
fwht_general does (hybrid_quantizer.py:154-193) -- not a unitary transform, and kept that way.

encode / decode are HIP kernels (one wavefront per vector, butterflies across lanes); the
codebooks and sign vectors are built on the host at construction, as in the reference.
`calibrate_uniform()` is the configuration the kernels are written for; `calibrate(sample)` runs the
same kernels on coordinates permuted into group order.  head_dim is 128.
"""
from __future__ import annotations

import functools
import math
from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import numpy as np
import torch

from . import _lib

__all__ = ["HybridTurboQuant", "HybridLayout", "GroupLayout", "MODE_CONFIGS"]

# (outlier share of dims, (total bits group 0, total bits group 1)); one bit of each total is
# the QJL sign, the rest index the MSE codebook (reference: hybrid_quantizer.py:52-65).
MODE_CONFIGS: Dict[str, dict] = {
    "tq35": {"outlier_ratio": 0.50, "group_bits": (4, 3)},
    "tq25": {"outlier_ratio": 0.25, "group_bits": (3, 2)},
}


@dataclass(frozen=True)
class GroupLayout:
    dim: int
    mse_bits: int
    mse_packed_bytes: int
    qjl_packed_bytes: int
    norm_bytes: int
    residual_norm_bytes: int
    total_bytes: int


@dataclass(frozen=True)
class HybridLayout:
    group0: GroupLayout
    group1: GroupLayout
    packed_dim: int


def _group_layout(dim: int, mse_bits: int) -> GroupLayout:
    mse = -(-dim * mse_bits // 8)
    qjl = -(-dim // 8)
    return GroupLayout(dim, mse_bits, mse, qjl, 2, 2, mse + qjl + 4)


def _make_hybrid_layout(head_dim: int, mode: str) -> HybridLayout:
    """Byte layout of a packed vector (reference: hybrid_quantizer.py:92-123)."""
    cfg = MODE_CONFIGS[mode]
    b0, b1 = cfg["group_bits"]
    d0 = round(head_dim * cfg["outlier_ratio"])
    g0 = _group_layout(d0, b0 - 1)
    g1 = _group_layout(head_dim - d0, b1 - 1)
    return HybridLayout(g0, g1, g0.total_bytes + g1.total_bytes)


# Codebooks of the tq35 / head_dim 128 case as the reference's float64 grid iteration leaves
# them (float32).  The middle boundary of a symmetric codebook is exactly 0 in theory; what the
# iteration leaves there is summation noise (0.0 for the 3-bit book, -2**-58 for the 2-bit
# book), and it decides which code an all-zero group receives -- so the literal values are
# kept.  Decoded values do not depend on it (such a group has norm 0).
# (tq25: the one-bit book's only boundary is such noise, -2**-57)
_TQ25_BOOKS = {
    (32, 2): (np.array([-0.26338478922843933, -0.07983556389808655, 0.07983556389808655,
                        0.26338478922843933], dtype=np.float32),
              np.array([-0.17161017656326294, 0.0, 0.17161017656326294], dtype=np.float32)),
    (96, 1): (np.array([-0.08164610713720322, 0.08164610713720322], dtype=np.float32),
              np.array([-6.938893903907228e-18], dtype=np.float32)),
}
_TQ35_D64 = {
    3: (np.array([-0.264565646648407, -0.16685186326503754, -0.09433808922767639,
                  -0.03065413422882557, 0.03065413422882557, 0.09433808922767639,
                  0.16685186326503754, 0.264565646648407], dtype=np.float32),
        np.array([-0.21570874750614166, -0.13059496879577637, -0.062496110796928406, 0.0,
                  0.062496110796928406, 0.13059496879577637, 0.21570874750614166],
                 dtype=np.float32)),
    2: (np.array([-0.187562957406044, -0.0565478578209877, 0.0565478578209877,
                  0.187562957406044], dtype=np.float32),
        np.array([-0.12205541133880615, -3.469446951953614e-18, 0.12205541133880615],
                 dtype=np.float32)),
}


# ---- host-side helpers of the reference's module (hybrid_quantizer.py:130-234,310-396): torch ops on whatever
# device the tensor lives on.  The kernels do these steps in registers; callers that import the helpers keep working.
def fwht_pow2(x: torch.Tensor) -> torch.Tensor:
    """Unnormalised Walsh-Hadamard transform of the last axis (a power of two), written back into `x`."""
    from .rotation import fast_hadamard_transform
    x.copy_(fast_hadamard_transform(x))
    return x


def fwht_general(x: torch.Tensor) -> torch.Tensor:
    """The same for any length: the axis is cut into descending powers of two (96 = 64 + 32) and each piece is
    transformed on its own.  Returns a new tensor."""
    from .rotation import fast_hadamard_transform
    n, at, out = x.shape[-1], 0, []
    while n > 0:
        piece = 1 << (n.bit_length() - 1)
        out.append(fast_hadamard_transform(x[..., at:at + piece]))
        at, n = at + piece, n - piece
    return torch.cat(out, dim=-1) if out else x.clone()


def structured_hadamard(x: torch.Tensor, signs: torch.Tensor, normalized: bool = True,
                        inverse: bool = False) -> torch.Tensor:
    """H diag(signs) x (forward) or diag(signs) H x (inverse), divided by sqrt(dim) when `normalized`."""
    y = fwht_general(x) * signs if inverse else fwht_general(x * signs)
    return y / math.sqrt(x.shape[-1]) if normalized else y


def pack_multibit(indices: torch.Tensor, bits: int) -> torch.Tensor:
    """[..., dim] indices of `bits` bits (1..8) -> [..., ceil(dim bits / 8)] uint8, one MSB-first bit stream."""
    dim = indices.shape[-1]
    nbytes = -(-dim * bits // 8)
    shifts = torch.arange(bits - 1, -1, -1, device=indices.device)
    stream = ((indices.long().unsqueeze(-1) >> shifts) & 1).reshape(*indices.shape[:-1], dim * bits)
    stream = torch.nn.functional.pad(stream, (0, nbytes * 8 - dim * bits))
    weights = 1 << torch.arange(7, -1, -1, device=indices.device)
    return (stream.reshape(*indices.shape[:-1], nbytes, 8) * weights).sum(-1).to(torch.uint8)


def unpack_multibit(packed: torch.Tensor, dim: int, bits: int) -> torch.Tensor:
    """Inverse of pack_multibit -> [..., dim] uint8."""
    shifts = torch.arange(7, -1, -1, device=packed.device)
    stream = ((packed.long().unsqueeze(-1) >> shifts) & 1).reshape(*packed.shape[:-1], packed.shape[-1] * 8)
    weights = 1 << torch.arange(bits - 1, -1, -1, device=packed.device)
    return (stream[..., :dim * bits].reshape(*packed.shape[:-1], dim, bits) * weights).sum(-1).to(torch.uint8)


@functools.lru_cache(maxsize=None)
def _lloyd_on_grid(dim: int, bits: int) -> Tuple[np.ndarray, np.ndarray]:
    """Lloyd iteration on a 10,000-point grid over (-0.999, 0.999) weighted by the marginal
    density of a coordinate of a uniform point on S^{dim-1}, (1-x^2)^((dim-3)/2); at most 200
    sweeps, stop when the centroids move less than 1e-10 (reference:
    hybrid_quantizer.py:241-303).  float64 throughout, float32 results."""
    levels = 1 << bits
    grid = np.linspace(-0.999, 0.999, 10000, dtype=np.float64)
    expo = (dim - 3) / 2.0
    base = 1.0 - grid * grid
    w = base ** expo if expo >= 0 else np.maximum(base, 1e-30) ** expo
    w /= w.sum()
    cen = np.linspace(grid[0], grid[-1], levels, dtype=np.float64)
    for _ in range(200):
        owner = np.clip(np.searchsorted((cen[:-1] + cen[1:]) / 2.0, grid, side="left"), 0, levels - 1)
        mass = np.bincount(owner, weights=w, minlength=levels)
        moment = np.bincount(owner, weights=w * grid, minlength=levels)
        new = np.where(mass > 1e-30, moment / np.where(mass > 1e-30, mass, 1.0), cen)
        moved = np.abs(new - cen).max()
        cen = new
        if moved < 1e-10:
            break
    return cen.astype(np.float32), ((cen[:-1] + cen[1:]) / 2.0).astype(np.float32)


def dimension_aware_codebook(dim: int, bits: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """(centroids [2^bits], inner boundaries [2^bits - 1]) float32 CPU tensors."""
    if dim == 64 and bits in _TQ35_D64:
        c, b = _TQ35_D64[bits]
    elif (dim, bits) in _TQ25_BOOKS:
        c, b = _TQ25_BOOKS[(dim, bits)]
    else:
        c, b = _lloyd_on_grid(dim, bits)
    return torch.from_numpy(c.copy()), torch.from_numpy(b.copy())


class HybridTurboQuant:
    """htq = HybridTurboQuant(head_dim=128, mode="tq35"); htq.calibrate_uniform()
    packed = htq.encode(kv)        # uint8 [..., 64] (tq25: [..., 44])
    kv_hat = htq.decode(packed)    # float32 [..., 128]
    """

    def __init__(self, head_dim: int = 128, mode: str = "tq35", seed: int = 42,
                 device: str = "cuda") -> None:
        if mode not in MODE_CONFIGS:
            raise ValueError(f"Unsupported mode {mode!r}. Choose from {list(MODE_CONFIGS.keys())}.")
        self.head_dim = head_dim
        self.mode = mode
        self.seed = seed
        self.device = device
        self.layout: HybridLayout = _make_hybrid_layout(head_dim, mode)
        b0, b1 = MODE_CONFIGS[mode]["group_bits"]
        self._g0_mse_bits, self._g1_mse_bits = b0 - 1, b1 - 1
        self._g0_dim, self._g1_dim = self.layout.group0.dim, self.layout.group1.dim

        # Four Rademacher vectors drawn in this order from ONE generator seeded with `seed`:
        # group-0 Hadamard, group-1 Hadamard, group-0 QJL, group-1 QJL
        # (reference: hybrid_quantizer.py:514-523).
        gen = torch.Generator(device="cpu")
        gen.manual_seed(seed)

        def draw(n: int) -> torch.Tensor:
            return 2 * torch.randint(0, 2, (n,), generator=gen, dtype=torch.float32) - 1

        signs = [draw(self._g0_dim), draw(self._g1_dim), draw(self._g0_dim), draw(self._g1_dim)]
        self._g0_had_signs, self._g1_had_signs, self._g0_qjl_signs, self._g1_qjl_signs = \
            [s.to(device) for s in signs]
        c0, bnd0 = dimension_aware_codebook(self._g0_dim, self._g0_mse_bits)
        c1, bnd1 = dimension_aware_codebook(self._g1_dim, self._g1_mse_bits)
        self._g0_centroids, self._g0_boundaries = c0.to(device), bnd0.to(device)
        self._g1_centroids, self._g1_boundaries = c1.to(device), bnd1.to(device)
        self._g0_qjl_scale = math.sqrt(math.pi / 2.0) / self._g0_dim
        self._g1_qjl_scale = math.sqrt(math.pi / 2.0) / self._g1_dim

        self._group0_indices: Optional[torch.Tensor] = None
        self._group1_indices: Optional[torch.Tensor] = None
        self._num_kv_heads = 0
        self._calibrated = False
        self._uniform_split = False

        # One float32 table for the kernels (layout fixed by include/aitherkv.h).
        self._table: Optional[torch.Tensor] = None
        if mode == "tq35" and head_dim == 128:
            tab = torch.zeros(_lib.HYB_TABLE_FLOATS, dtype=torch.float32)
            tab[0:64], tab[64:128], tab[128:192], tab[192:256] = signs
            tab[256:264], tab[264:268] = c0, c1
            tab[268:275], tab[275:278] = bnd0, bnd1
            self._table = tab.to(device)
        elif mode == "tq25" and head_dim == 128:
            tab = torch.zeros(_lib.HYB_TABLE_FLOATS, dtype=torch.float32)
            tab[0:32], tab[32:128], tab[128:160], tab[160:256] = signs
            tab[256:260], tab[260:262] = c0, c1
            tab[262:265], tab[265:266] = bnd0, bnd1
            self._table = tab.to(device)
        # entry points of the mode (include/aitherkv.h)
        self._abi = "akv_hybrid25" if mode == "tq25" else "akv_hybrid"

    # -- calibration ----------------------------------------------------------------------
    def calibrate_uniform(self, num_kv_heads: int = 1) -> None:
        """First g0_dim dims form group 0, the rest group 1, for every head
        (reference: hybrid_quantizer.py:590-603)."""
        self._num_kv_heads = num_kv_heads
        g0 = torch.arange(self._g0_dim, device=self.device)
        g1 = torch.arange(self._g0_dim, self.head_dim, device=self.device)
        self._group0_indices = g0.unsqueeze(0).expand(num_kv_heads, -1).contiguous()
        self._group1_indices = g1.unsqueeze(0).expand(num_kv_heads, -1).contiguous()
        self._calibrated = True
        self._uniform_split = True

    def calibrate(self, sample_vectors: torch.Tensor) -> None:
        """Variance-ranked per-head groups (reference: hybrid_quantizer.py:553-588): per kv head the g0_dim
        coordinates of largest mean square over the sample form group 0 (in descending order of that score), the
        others group 1.  sample_vectors [num_samples, num_kv_heads, head_dim].
        The kernels work on the uniform split; a ranked split is the same codec on permuted coordinates, so the
        vectors are gathered into group order before they are encoded (`to_group_order`) and scattered back after
        they are decoded -- one extra pass of torch ops per call that the uniform split does not pay."""
        if sample_vectors.dim() != 3:
            raise ValueError(f"Expected [num_samples, num_kv_heads, head_dim], got shape {list(sample_vectors.shape)}")
        _, num_kv_heads, hdim = sample_vectors.shape
        if hdim != self.head_dim:
            raise ValueError(f"head_dim mismatch: expected {self.head_dim}, got {hdim}")
        self._num_kv_heads = num_kv_heads
        order = sample_vectors.float().square().mean(dim=0).sort(dim=-1, descending=True).indices.to(self.device)
        self._group0_indices = order[:, :self._g0_dim].contiguous()
        self._group1_indices = order[:, self._g0_dim:].contiguous()
        self._calibrated = True
        self._uniform_split = False

    @property
    def group_order(self) -> Optional[torch.Tensor]:
        """[num_kv_heads, head_dim] coordinate order (group 0, then group 1) of a ranked split; None for the
        uniform split, where the order is the identity."""
        if not self._calibrated or self._uniform_split:
            return None
        return torch.cat([self._group0_indices, self._group1_indices], dim=-1)

    def to_group_order(self, x: torch.Tensor, head_axis: Optional[int] = None) -> torch.Tensor:
        """x [..., head_dim] with coordinates moved into group order.  head_axis names the axis that runs over the
        kv heads; without one the flattened vectors cycle over the heads when their number is a multiple of
        num_kv_heads and use head 0's order otherwise (the reference's rule, hybrid_quantizer.py:640-662)."""
        return self._reorder(x, head_axis, inverse=False)

    def from_group_order(self, x: torch.Tensor, head_axis: Optional[int] = None) -> torch.Tensor:
        """Inverse of to_group_order."""
        return self._reorder(x, head_axis, inverse=True)

    def _reorder(self, x: torch.Tensor, head_axis: Optional[int], inverse: bool) -> torch.Tensor:
        order = self.group_order
        if order is None:
            return x
        order = order.to(x.device)
        H, D = order.shape
        if head_axis is not None:
            xm = x.movedim(head_axis, -2)
            if xm.shape[-2] != H:
                raise ValueError(f"axis {head_axis} has {xm.shape[-2]} entries, calibrated for {H} kv heads")
            idx = order.expand(xm.shape)
        else:
            flat = x.reshape(-1, D)
            xm = flat.reshape(-1, H, D) if (H > 1 and flat.shape[0] % H == 0) else flat
            idx = order.expand(xm.shape) if xm.dim() == 3 else order[0].expand(xm.shape)
        out = torch.empty_like(xm).scatter_(-1, idx, xm) if inverse else torch.gather(xm, -1, idx)
        return out.movedim(-2, head_axis) if head_axis is not None else out.reshape(x.shape)

    def _ensure_ready(self) -> None:
        if not self._calibrated:
            raise RuntimeError("HybridTurboQuant: must call calibrate() or calibrate_uniform() "
                               "before encode/decode.")
        if self._table is None:
            raise NotImplementedError(
                f"HIP kernels exist for head_dim 128 only (got mode {self.mode!r}, head_dim {self.head_dim})")

    @property
    def kernel_table(self) -> torch.Tensor:
        self._ensure_ready()
        return self._table

    # -- encode / decode --------------------------------------------------------------------
    def encode(self, x: torch.Tensor) -> torch.Tensor:
        """[..., 128] float -> uint8 [..., packed_dim] (64 for tq35, 44 for tq25)."""
        self._ensure_ready()
        assert x.shape[-1] == self.head_dim, f"Expected last dim {self.head_dim}, got {x.shape[-1]}"
        dev = _lib.require_gpu(x, self._table)
        batch = list(x.shape[:-1])
        if x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
            x = x.float()
        xf = self.to_group_order(x).reshape(-1, self.head_dim)
        if xf.stride(-1) != 1:
            xf = xf.contiguous()
        n = xf.shape[0]
        out = torch.empty(n, self.layout.packed_dim, dtype=torch.uint8, device=dev)
        _lib.check(getattr(_lib.lib(), self._abi + "_encode")(
            xf.data_ptr(), _lib.dtype_code(xf), n, xf.stride(0) if n else self.head_dim,
            self._table.data_ptr(), out.data_ptr(), self.layout.packed_dim, _lib.stream_ptr(dev)))
        return out.reshape(batch + [self.layout.packed_dim])

    def decode(self, packed: torch.Tensor) -> torch.Tensor:
        """uint8 [..., packed_dim] -> float32 [..., 128]."""
        self._ensure_ready()
        assert packed.shape[-1] == self.layout.packed_dim, \
            f"Expected last dim {self.layout.packed_dim}, got {packed.shape[-1]}"
        dev = _lib.require_gpu(packed, self._table)
        batch = list(packed.shape[:-1])
        pf = packed.reshape(-1, self.layout.packed_dim)
        if pf.stride(-1) != 1:
            pf = pf.contiguous()
        n = pf.shape[0]
        out = torch.empty(n, self.head_dim, dtype=torch.float32, device=dev)
        _lib.check(getattr(_lib.lib(), self._abi + "_decode")(
            pf.data_ptr(), pf.stride(0) if n else self.layout.packed_dim, n, self._table.data_ptr(),
            out.data_ptr(), self.head_dim, _lib.stream_ptr(dev)))
        return self.from_group_order(out).reshape(batch + [self.head_dim])

    # -- analysis -----------------------------------------------------------------------------
    def validate(self, num_vectors: int = 10000) -> dict:
        """Round trip on random vectors whose first group has twice the scale
        (reference: hybrid_quantizer.py:939-1001)."""
        if not self._calibrated:
            self.calibrate_uniform(num_kv_heads=1)
        x = torch.randn(num_vectors, self.head_dim, device=self.device, dtype=torch.float32)
        x[:, :self._g0_dim] *= 2.0
        x_hat = self.decode(self.encode(x))
        mse = (x - x_hat).pow(2).sum(-1).mean().item()
        energy = x.pow(2).sum(-1).mean().item()
        return {
            "mode": self.mode,
            "head_dim": self.head_dim,
            "num_vectors": num_vectors,
            "packed_dim_bytes": self.layout.packed_dim,
            "mse": mse,
            "relative_mse": mse / energy if energy > 0 else float("inf"),
            "cosine_similarity": torch.nn.functional.cosine_similarity(x, x_hat, dim=-1).mean().item(),
            "max_abs_error": (x - x_hat).abs().max().item(),
            "compression_vs_fp16": self.head_dim * 2 / self.layout.packed_dim,
            "compression_vs_fp8": self.head_dim / self.layout.packed_dim,
            "group0": {"dim": self._g0_dim, "mse_bits": self._g0_mse_bits,
                       "bytes": self.layout.group0.total_bytes},
            "group1": {"dim": self._g1_dim, "mse_bits": self._g1_mse_bits,
                       "bytes": self.layout.group1.total_bytes},
        }

    def compression_ratio(self) -> float:
        return (self.head_dim * 2) / self.layout.packed_dim

    def memory_report(self, seq_len: int, num_layers: int = 32, num_kv_heads: int = 8) -> dict:
        vectors = seq_len * num_layers * num_kv_heads * 2
        fp16, fp8 = vectors * self.head_dim * 2, vectors * self.head_dim
        hyb = vectors * self.layout.packed_dim
        return {
            "config": f"Hybrid-{self.mode.upper()} d={self.head_dim} seq={seq_len} "
                      f"L={num_layers} H={num_kv_heads}",
            "fp16_mb": fp16 / 2 ** 20,
            "fp8_mb": fp8 / 2 ** 20,
            f"{self.mode}_mb": hyb / 2 ** 20,
            "ratio_vs_fp16": fp16 / hyb,
            "ratio_vs_fp8": fp8 / hyb,
        }

    @property
    def packed_dim(self) -> int:
        return self.layout.packed_dim

    @staticmethod
    def packed_dim_for_mode(head_dim: int, mode: str) -> int:
        return _make_hybrid_layout(head_dim, mode).packed_dim

    def __repr__(self) -> str:
        state = "calibrated" if self._calibrated else "uncalibrated"
        return (f"HybridTurboQuant(d={self.head_dim}, mode={self.mode!r}, "
                f"packed={self.layout.packed_dim}B, compress={self.compression_ratio():.1f}x, {state})")
