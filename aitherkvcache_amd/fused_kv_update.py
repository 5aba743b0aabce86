"""Encode-on-write into the paged TurboQuant cache: one HIP kernel does norm, normalise,
rotation, codebook search, bit packing and the scatter through slot_mapping.

Same call surface as the reference's aither_kvcache/fused_kv_update.py
(fused_tq4_kv_update :300-405, fused_encode_and_store :412-468) with the semantics of its
torch fallback (:220-293): the stored norm is the plain L2 norm, the divisor is norm + 1e-10,
ties go to the lower bin, tokens with a negative slot or a block index >= max_blocks are
skipped.  Besides 4-bit (the only width the reference fuses) 3- and 2-bit are supported via
`bits=` / fused_kv_update().
"""
import logging

import torch

from . import _lib
from .packing import packed_size
from .quantizer import prepared_rotation_for

logger = logging.getLogger("aither.turboquant.fused_kv_update")

HAS_HIP = _lib.available()
HAS_TRITON = HAS_HIP
_DTYPE_OK = (torch.float16, torch.bfloat16, torch.float32)

__all__ = ["fused_tq4_kv_update", "fused_kv_update", "fused_encode_and_store", "HAS_TRITON", "HAS_HIP"]


def fused_kv_update(x, slot_mapping, out_packed, out_norms, rotation, boundaries, bits,
                    block_size=16, max_blocks=0, prepared=None) -> None:
    """Quantize-and-store for one cache tensor (K or V) at `bits` in {2, 3, 4}.

    x            [num_tokens, num_kv_heads, head_dim] float16 / bfloat16 / float32
    slot_mapping [num_tokens] int64 or int32; negative = padding
    out_packed   [max_blocks, block_size, num_kv_heads, >= packed_dim] uint8 (strides honoured)
    out_norms    [max_blocks, block_size, num_kv_heads] float32 (strides honoured)
    rotation     [head_dim, head_dim] float32;  boundaries [2**bits - 1] float32
    """
    if max_blocks == 0:
        max_blocks = out_packed.shape[0]
    num_tokens, num_kv_heads, head_dim = x.shape
    if num_tokens == 0:
        return
    if head_dim <= 0 or (head_dim & (head_dim - 1)) != 0:
        raise ValueError(f"head_dim must be a power of 2, got {head_dim}")
    dev = _lib.require_gpu(x, slot_mapping, out_packed, out_norms, rotation, boundaries)
    if out_packed.dtype != torch.uint8 or out_norms.dtype != torch.float32:
        raise ValueError("out_packed must be uint8 and out_norms float32")
    if out_packed.shape[-1] < packed_size(head_dim, bits) or out_packed.stride(-1) != 1:
        raise ValueError("out_packed rows are too short or not contiguous in the last dim")
    if x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        x = x.float()
    if x.stride(-1) != 1:
        x = x.contiguous()
    slots = slot_mapping if slot_mapping.is_contiguous() else slot_mapping.contiguous()
    prep = prepared if prepared is not None else prepared_rotation_for(rotation)
    bnd = boundaries if (boundaries.dtype == torch.float32 and boundaries.is_contiguous()) \
        else boundaries.float().contiguous()
    _lib.check(_lib.lib().akv_encode_paged(
        x.data_ptr(), _lib.dtype_code(x), num_tokens, num_kv_heads, head_dim, x.stride(0), x.stride(1),
        slots.data_ptr(), _lib.itype_code(slots), prep.ptr, bnd.data_ptr(), bits,
        out_packed.data_ptr(), out_packed.stride(0), out_packed.stride(1), out_packed.stride(2),
        out_norms.data_ptr(), out_norms.stride(0), out_norms.stride(1), out_norms.stride(2),
        block_size, max_blocks, _lib.stream_ptr(dev)))


def fused_tq4_kv_update(x, slot_mapping, out_packed, out_norms, rotation, boundaries,
                        block_size: int = 16, max_blocks: int = 0) -> None:
    """4-bit quantize-and-store, signature of the reference (fused_kv_update.py:300-309)."""
    fused_kv_update(x, slot_mapping, out_packed, out_norms, rotation, boundaries, 4,
                    block_size=block_size, max_blocks=max_blocks)


def fused_kv_update_pair(key, value, slot_mapping, k_packed, k_norms, v_packed, v_norms, rotation,
                         boundaries, bits, block_size=16, max_blocks=0, prepared=None) -> None:
    """K and V of one step ([num_tokens, num_kv_heads, head_dim] each) into their caches with ONE
    kernel launch when the two tensors and the two caches have the same dtype, shapes and strides
    (key / value of a layer and the halves of a serving cache tensor do); two launches otherwise.
    Results equal two fused_kv_update calls."""
    same = (key.shape == value.shape and key.dtype == value.dtype and key.stride() == value.stride()
            and key.stride(-1) == 1 and key.dtype in (torch.float16, torch.bfloat16, torch.float32)
            and k_packed.shape == v_packed.shape and k_packed.stride() == v_packed.stride()
            and k_norms.shape == v_norms.shape and k_norms.stride() == v_norms.stride())
    if not same:
        for x, packed, norms in ((key, k_packed, k_norms), (value, v_packed, v_norms)):
            fused_kv_update(x, slot_mapping, packed, norms, rotation, boundaries, bits,
                            block_size=block_size, max_blocks=max_blocks, prepared=prepared)
        return
    if max_blocks == 0:
        max_blocks = k_packed.shape[0]
    num_tokens, num_kv_heads, head_dim = key.shape
    if num_tokens == 0:
        return
    if head_dim <= 0 or (head_dim & (head_dim - 1)) != 0:
        raise ValueError(f"head_dim must be a power of 2, got {head_dim}")
    dev = _lib.require_gpu(key, value, slot_mapping, k_packed, v_packed, k_norms, v_norms, rotation, boundaries)
    if k_packed.dtype != torch.uint8 or v_packed.dtype != torch.uint8 \
            or k_norms.dtype != torch.float32 or v_norms.dtype != torch.float32:
        raise ValueError("packed caches must be uint8 and norms float32")
    if k_packed.shape[-1] < packed_size(head_dim, bits) or k_packed.stride(-1) != 1:
        raise ValueError("packed rows are too short or not contiguous in the last dim")
    slots = slot_mapping if slot_mapping.is_contiguous() else slot_mapping.contiguous()
    prep = prepared if prepared is not None else prepared_rotation_for(rotation)
    bnd = boundaries if (boundaries.dtype == torch.float32 and boundaries.is_contiguous()) \
        else boundaries.float().contiguous()
    _lib.check(_lib.lib().akv_encode_paged_kv(
        key.data_ptr(), value.data_ptr(), _lib.dtype_code(key), num_tokens, num_kv_heads, head_dim,
        key.stride(0), key.stride(1), slots.data_ptr(), _lib.itype_code(slots), prep.ptr, bnd.data_ptr(), bits,
        k_packed.data_ptr(), v_packed.data_ptr(), k_packed.stride(0), k_packed.stride(1), k_packed.stride(2),
        k_norms.data_ptr(), v_norms.data_ptr(), k_norms.stride(0), k_norms.stride(1), k_norms.stride(2),
        block_size, max_blocks, _lib.stream_ptr(dev)))


class _StorePlan:
    """What fused_encode_and_store needs for one (cache object, layer) once its tensors have been validated: the
    per-layer views, their strides and the prepared rotation.  A serving loop calls the function once per layer and
    step with the same cache; re-deriving views, shapes and strides each time costs more host time than the
    kernel runs.  A plan is valid while the cache object still holds the same tensors (same objects, same
    storage) and the same quantizer (matrix, boundaries and bit width, by object and version counter); the
    step's own tensors (key, value, slot_mapping) are checked on every call."""

    __slots__ = ("kp_all", "kn_all", "vp_all", "vn_all", "tq", "rot", "rot_version", "views", "prep", "bnd", "fixed",
                 "tail", "dev", "max_blocks", "block_size", "b_src", "b_version", "bits", "ptrs", "layer", "boxed")

    def __init__(self, tq_cache, layer_idx):
        tq = tq_cache.tq
        self.kp_all, self.kn_all = tq_cache.k_packed, tq_cache.k_norms
        self.vp_all, self.vn_all = tq_cache.v_packed, tq_cache.v_norms
        self.tq, self.rot, self.rot_version = tq, tq.rotation, tq.rotation._version
        self.b_src, self.b_version, self.bits = tq.boundaries_inner, tq.boundaries_inner._version, tq.bits
        kp, kn, vp, vn = (t[layer_idx] for t in (self.kp_all, self.kn_all, self.vp_all, self.vn_all))
        self.views = (kp, kn, vp, vn)
        self.layer = layer_idx
        self.boxed = all(isinstance(t, torch.Tensor) for t in (self.kp_all, self.kn_all, self.vp_all, self.vn_all))
        self.ptrs = self._storage()
        self.dev = _lib.require_gpu(kp, kn, vp, vn, tq.rotation, tq.boundaries_inner)
        head_dim = tq.head_dim
        same = (kp.shape == vp.shape and kp.stride() == vp.stride() and kn.shape == vn.shape
                and kn.stride() == vn.stride() and kp.dtype == torch.uint8 and vp.dtype == torch.uint8
                and kn.dtype == torch.float32 and vn.dtype == torch.float32 and kp.stride(-1) == 1
                and kp.shape[-1] >= packed_size(head_dim, tq.bits) and hasattr(tq, "prepared_rotation")
                and head_dim > 0 and (head_dim & (head_dim - 1)) == 0)
        self.fixed = None
        if not same:
            return
        self.prep = tq.prepared_rotation()
        b = tq.boundaries_inner
        self.bnd = b if (b.dtype == torch.float32 and b.is_contiguous()) else b.float().contiguous()
        self.block_size = tq_cache.block_size
        self.max_blocks = tq_cache.max_blocks or kp.shape[0]
        self.tail = (kp.shape[2], head_dim)
        self.fixed = (self.prep.ptr, self.bnd.data_ptr(), tq.bits, kp.data_ptr(), vp.data_ptr(), kp.stride(0),
                      kp.stride(1), kp.stride(2), kn.data_ptr(), vn.data_ptr(), kn.stride(0), kn.stride(1),
                      kn.stride(2), self.block_size, self.max_blocks)

    def _storage(self):
        """Where the layer's four tensors lie now, or None when one of them has been replaced.  A container that is
        one tensor per kind is asked for its own address (its per-layer view cannot move without it); a list of
        per-layer tensors must still hold the very tensor the view was taken from."""
        if self.boxed:
            return (self.kp_all.data_ptr(), self.kn_all.data_ptr(), self.vp_all.data_ptr(), self.vn_all.data_ptr())
        out = []
        for box, view in zip((self.kp_all, self.kn_all, self.vp_all, self.vn_all), self.views):
            if isinstance(box, torch.Tensor):
                out.append(box.data_ptr())
            elif box[self.layer] is view:
                out.append(view.data_ptr())
            else:
                return None
        return tuple(out)

    def valid_for(self, tq_cache) -> bool:
        tq = tq_cache.tq
        b = self.b_src
        return (tq_cache.k_packed is self.kp_all and tq_cache.v_packed is self.vp_all
                and tq_cache.k_norms is self.kn_all and tq_cache.v_norms is self.vn_all and tq is self.tq
                and tq.rotation is self.rot and self.rot._version == self.rot_version
                and tq.boundaries_inner is b and b._version == self.b_version and tq.bits == self.bits
                # (a tensor can be given other storage in place: set_, resize_, an assignment to .data)
                and self.ptrs is not None and self._storage() == self.ptrs
                and tq_cache.block_size == self.block_size
                and (tq_cache.max_blocks or self.views[0].shape[0]) == self.max_blocks)


def fused_encode_and_store(tq_cache, layer_idx: int, key, value, slot_mapping) -> None:
    """K and V for one layer into a cache object with attributes tq, k_packed, k_norms,
    v_packed, v_norms, block_size, max_blocks (reference: fused_kv_update.py:412-468)."""
    plans = tq_cache.__dict__.get("_akv_store_plans") if hasattr(tq_cache, "__dict__") else None
    if plans is None:
        plans = {}
        try:
            tq_cache._akv_store_plans = plans
        except AttributeError:
            pass
    plan = plans.get(layer_idx)
    if plan is None or plan.fixed is None or not plan.valid_for(tq_cache):
        plan = _StorePlan(tq_cache, layer_idx)
        plans[layer_idx] = plan
    f = plan.fixed
    if (f is not None and key.dtype in _DTYPE_OK and value.dtype is key.dtype and key.dim() == 3
            and key.shape[1:] == plan.tail and value.shape == key.shape and key.stride(2) == 1
            and key.stride() == value.stride() and key.device == plan.dev and value.device == plan.dev
            and slot_mapping.device == plan.dev and slot_mapping.is_contiguous()
            and slot_mapping.shape[0] == key.shape[0]):
        if key.shape[0] == 0:
            return
        _lib.check(_lib.lib().akv_encode_paged_kv(
            key.data_ptr(), value.data_ptr(), _lib.dtype_code(key), key.shape[0], plan.tail[0], plan.tail[1],
            key.stride(0), key.stride(1), slot_mapping.data_ptr(), _lib.itype_code(slot_mapping), f[0], f[1], f[2],
            f[3], f[4], f[5], f[6], f[7], f[8], f[9], f[10], f[11], f[12], f[13], f[14], _lib.stream_ptr(plan.dev)))
        return
    tq = tq_cache.tq
    prep = tq.prepared_rotation() if hasattr(tq, "prepared_rotation") else None
    fused_kv_update_pair(key, value, slot_mapping, tq_cache.k_packed[layer_idx], tq_cache.k_norms[layer_idx],
                         tq_cache.v_packed[layer_idx], tq_cache.v_norms[layer_idx], tq.rotation,
                         tq.boundaries_inner, tq.bits, block_size=tq_cache.block_size,
                         max_blocks=tq_cache.max_blocks, prepared=prep)
