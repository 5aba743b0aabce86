"""The attention backend vLLM loads with `--attention-backend CUSTOM`: TurboQuantBackend and its
TurboQuantImpl (reference: aither_kvcache/vllm/backend.py:247-311 for the lazily created
backend class, :324-562 for the impl's state, do_kv_cache_update and forward, :711-1091 for the
PRIMARY paths, :1280-1295 for the registration).

Importing this module imports neither vLLM nor anything that touches the GPU.  The two classes are
made on first attribute access (`backend.TurboQuantBackend`, `backend.TurboQuantImpl`), as vLLM
resolves a registered backend by `getattr(module, name)` while its own configuration modules may
still be half imported.  With vLLM importable they derive from its AttentionBackend and
TritonAttentionImpl; without it they derive from small stand-ins that keep the constructor
arguments, so the TurboQuant side (cache write, decode attention, block decompression) can run and
be tested on its own -- whatever is vLLM's own job (attention over an uncompressed cache, the
metadata builder) then raises with a message that says so.

What the impl does with the cache (PRIMARY mode: the tensor vLLM allocates IS the compressed cache,
uint8 [num_blocks, 2, block_size, num_kv_heads, tq_dim]):

  do_kv_cache_update   the step's new K and V rows go through the fused encode-on-write kernel
                       (uniform formats: codes into the cache rows, norms into per-layer float32
                       tensors; tq35: whole 64-byte rows)
  forward, decode      one call of the decode-attention kernel on the packed rows.  vLLM releases
                       that never call do_kv_cache_update get write + attend from one call of the
                       tq::decode_step / tq::hybrid_decode_step op.
  forward, prefill     the blocks the batch addresses are decompressed into a bf16 block buffer
                       (batch_decompress_active_blocks), the chunk's own rows are scattered in
                       uncompressed, and vLLM's unified_attention runs on that buffer.

In SHADOW mode vLLM's own cache stays authoritative and this impl keeps a compressed copy beside
it (TQGPUCache); decode may be served from the copy (AITHER_TQ_FUSED=1).  The format comes from
AITHER_TQ_MODE / AITHER_TQ_BITS as in the reference, or from a `tq-t*nc` kv-cache dtype name.
"""
import logging
import os
import sys
from typing import ClassVar, Optional

import torch

from .kv_cache_dtype import KV_CACHE_DTYPES, CacheFormat, resolve_kv_cache_dtype, tq_dim_for_head

logger = logging.getLogger("turboquant.vllm.backend")

_LAZY = ("TurboQuantBackend", "TurboQuantImpl")
_PLAIN_DTYPES = ["auto", "bfloat16", "fp8", "fp8_e4m3", "fp8_e5m2"]


def __getattr__(name):
    if name == "TurboQuantBackend":
        cls = _make_backend_class()
    elif name == "TurboQuantImpl":
        cls = _get_impl_class()
    elif name == "TQGPUCache":                 # defined in .cache here; the reference keeps it in this module
        from .cache import TQGPUCache as cls
    else:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
    globals()[name] = cls
    return cls


def format_from_env() -> CacheFormat:
    """AITHER_TQ_MODE names a format ("tq35", "tq-t3nc", with or without "-primary"); otherwise
    AITHER_TQ_BITS (default 4) picks a uniform one (reference: vllm/hooks.py:44-46)."""
    mode = os.environ.get("AITHER_TQ_MODE", "").replace("-primary", "").lower()
    if mode in KV_CACHE_DTYPES:
        return KV_CACHE_DTYPES[mode]
    bits = int(os.environ.get("AITHER_TQ_BITS", "4"))
    return resolve_kv_cache_dtype(f"tq-t{bits}nc")


def primary_from_env() -> bool:
    mode = os.environ.get("AITHER_TQ_MODE", "")
    return mode.endswith("-primary") if mode else os.environ.get("AITHER_TQ_PRIMARY", "0") == "1"


# --------------------------------------------------------------------------------------------
# stand-ins used when vLLM is not importable
# --------------------------------------------------------------------------------------------
class _StandaloneBackendBase:
    pass


class _StandaloneImplBase:
    """Keeps what vLLM's attention impl constructor receives."""

    def __init__(self, num_heads, head_size, scale, num_kv_heads=None, alibi_slopes=None,
                 sliding_window=None, kv_cache_dtype="auto", logits_soft_cap=None, **kwargs):
        self.num_heads = num_heads
        self.head_size = head_size
        self.scale = float(scale)
        self.num_kv_heads = num_heads if num_kv_heads is None else num_kv_heads
        self.alibi_slopes = alibi_slopes
        self.sliding_window = (-1, -1) if sliding_window is None else (sliding_window - 1, 0)
        self.kv_cache_dtype = kv_cache_dtype
        self.logits_soft_cap = 0 if logits_soft_cap is None else logits_soft_cap

    def forward(self, *args, **kwargs):
        raise RuntimeError("attention over an uncompressed cache is vLLM's TritonAttentionImpl; "
                           "vLLM is not importable in this process")


def _vllm_unified_attention(impl, q, k_buf, v_buf, out, attn_metadata):
    """vLLM's paged attention over an uncompressed [blocks, block_size, heads, d] buffer, called as
    the reference calls it (backend.py:1200-1236)."""
    from vllm.v1.attention.backends.triton_attn import unified_attention
    num_seqs = attn_metadata.query_start_loc.shape[0] - 1
    ones = torch.ones(num_seqs, impl.num_kv_heads, dtype=torch.float32, device=q.device)
    unified_attention(q=q, k=k_buf, v=v_buf, out=out, cu_seqlens_q=attn_metadata.query_start_loc,
                      max_seqlen_q=attn_metadata.max_query_len, seqused_k=attn_metadata.seq_lens,
                      max_seqlen_k=attn_metadata.max_seq_len, softmax_scale=impl.scale, causal=True,
                      alibi_slopes=impl.alibi_slopes, window_size=impl.sliding_window,
                      block_table=attn_metadata.block_table, softcap=impl.logits_soft_cap,
                      q_descale=None, k_descale=ones, v_descale=ones)


# --------------------------------------------------------------------------------------------
# backend class
# --------------------------------------------------------------------------------------------
def _make_backend_class():
    try:
        from vllm.v1.attention.backend import AttentionBackend as base
    except ImportError:
        base = _StandaloneBackendBase

    class TurboQuantBackend(base):
        supported_kv_cache_dtypes = _PLAIN_DTYPES + sorted(KV_CACHE_DTYPES)
        # vLLM's attention layer pre-allocates the output tensor and passes it to forward
        accept_output_buffer = True
        # the cache write is the impl's do_kv_cache_update, which vLLM calls as its own op
        forward_includes_kv_cache_update = False

        @staticmethod
        def get_name() -> str:
            return "CUSTOM"

        @staticmethod
        def get_impl_cls():
            return _get_impl_class()

        @staticmethod
        def get_builder_cls():
            try:
                from vllm.v1.attention.backend import AttentionCGSupport
                from vllm.v1.attention.backends.triton_attn import TritonAttentionMetadataBuilder
            except ImportError as e:
                raise RuntimeError("the attention metadata builder is vLLM's; vLLM is not importable") from e

            class TQMetadataBuilder(TritonAttentionMetadataBuilder):
                # the impl keeps Python-side state (lazy tensors, per-layer objects): attention
                # runs outside vLLM's captured graphs, everything around it is still captured
                _cudagraph_support = AttentionCGSupport.NEVER

            return TQMetadataBuilder

        @staticmethod
        def get_kv_cache_shape(num_blocks, block_size, num_kv_heads, head_size, cache_dtype_str="auto"):
            """(num_blocks, 2, block_size, num_kv_heads, row): row is head_size elements for vLLM's
            own dtypes (the reference's answer for every dtype, backend.py:303-306) and tq_dim bytes
            for a `tq-t*nc` name, the shape of the PRIMARY uint8 tensor."""
            if isinstance(cache_dtype_str, str) and cache_dtype_str.lower() in KV_CACHE_DTYPES:
                head_size = tq_dim_for_head(head_size, KV_CACHE_DTYPES[cache_dtype_str.lower()])
            return (num_blocks, 2, block_size, num_kv_heads, head_size)

        @staticmethod
        def get_supported_head_sizes():
            return [64, 96, 128, 256, 512]

    return TurboQuantBackend


# --------------------------------------------------------------------------------------------
# impl class
# --------------------------------------------------------------------------------------------
_impl_class = None


def _get_impl_class():
    global _impl_class
    if _impl_class is None:
        _impl_class = _make_impl_class()
    return _impl_class


def _make_impl_class():
    try:
        from vllm.v1.attention.backends.triton_attn import TritonAttentionImpl as base
    except ImportError:
        base = _StandaloneImplBase

    from ..fused_attention import TQPagedAttention
    from ..fused_kv_update import fused_encode_and_store, fused_kv_update_pair
    from ..hybrid_attention import HybridPagedAttention, hybrid_encode_and_store_pair
    from . import hooks
    from .cache import TQGPUCache
    from .decompress import batch_decompress_active_blocks
    from .engine import primary_views

    class TurboQuantImpl(base):
        # ---- state shared by the layers of one model (reference: backend.py:344-389) ----
        _tq_layer_counter: ClassVar[int] = 0
        _target_head_size: ClassVar[Optional[int]] = None
        _tq_primary: ClassVar[bool] = primary_from_env()
        _fused_enabled: ClassVar[bool] = os.environ.get("AITHER_TQ_FUSED", "0") == "1"
        _tq_format: ClassVar[Optional[CacheFormat]] = None
        _tq_quantizer: ClassVar[Optional[object]] = None
        _primary_k_norms: ClassVar[Optional[torch.Tensor]] = None
        _primary_v_norms: ClassVar[Optional[torch.Tensor]] = None
        _tq_gpu_cache: ClassVar[Optional[TQGPUCache]] = None
        _prefill_k_buf: ClassVar[Optional[torch.Tensor]] = None
        _prefill_v_buf: ClassVar[Optional[torch.Tensor]] = None
        _PREFILL_BUF_BLOCKS: ClassVar[int] = 512
        _forward_count: ClassVar[int] = 0
        _INIT_AFTER_FORWARDS: ClassVar[int] = 2
        _MIN_BLOCKS_FOR_INIT: ClassVar[int] = 16
        # attention over an uncompressed block buffer: vLLM's kernel; replaceable (tests, other engines)
        _dense_paged_attention = staticmethod(_vllm_unified_attention)

        @classmethod
        def reset_class_state(cls) -> None:
            """Forget every tensor and object shared between layers (a new model, a test)."""
            cls._tq_layer_counter = 0
            cls._target_head_size = None
            cls._tq_primary = primary_from_env()
            cls._fused_enabled = os.environ.get("AITHER_TQ_FUSED", "0") == "1"
            cls._tq_format = None
            cls._tq_quantizer = None
            cls._primary_k_norms = cls._primary_v_norms = None
            cls._tq_gpu_cache = None
            cls._prefill_k_buf = cls._prefill_v_buf = None
            cls._forward_count = 0
            hooks.reset_state()

        def __init__(self, *args, **kwargs):
            super().__init__(*args, **kwargs)
            cls = TurboQuantImpl
            # layers of a speculative-decoding draft model (another head size) pass through untouched
            if cls._target_head_size is None:
                cls._target_head_size = self.head_size
            self._is_draft = self.head_size != cls._target_head_size
            self._fused_attn = None
            self._kv_update_seen = False
            if self._is_draft:
                self._tq_layer_idx = -1
                return
            self._tq_layer_idx = cls._tq_layer_counter
            cls._tq_layer_counter += 1
            if cls._tq_format is None:
                name = str(getattr(self, "kv_cache_dtype", "auto")).lower()
                cls._tq_format = KV_CACHE_DTYPES[name] if name in KV_CACHE_DTYPES else format_from_env()
                if name in KV_CACHE_DTYPES:
                    cls._tq_primary = True       # a tq cache dtype can only mean the cache is compressed
            logger.info("TurboQuantImpl[L%d]: heads=%d, kv=%d, dim=%d, mode=%s", self._tq_layer_idx,
                        self.num_heads, self.num_kv_heads, self.head_size,
                        "PRIMARY" if cls._tq_primary else ("fused+standard" if cls._fused_enabled else "standard"))

        # ---- shared objects -----------------------------------------------------------
        def _quantizer(self, device):
            cls = TurboQuantImpl
            if cls._tq_quantizer is None:
                fmt = cls._tq_format
                cls._tq_quantizer = hooks.init_quantizer(self.head_size, bits=fmt.bits, mode=fmt.mode,
                                                         device=str(device), num_kv_heads=self.num_kv_heads)
            return cls._tq_quantizer

        def _ensure_norms(self, kv_cache) -> None:
            cls = TurboQuantImpl
            if cls._primary_k_norms is None and cls._tq_format.kind == "uniform":
                shape = (cls._tq_layer_counter, kv_cache.shape[0], kv_cache.shape[2], self.num_kv_heads)
                cls._primary_k_norms = torch.zeros(shape, dtype=torch.float32, device=kv_cache.device)
                cls._primary_v_norms = torch.zeros_like(cls._primary_k_norms)
                logger.info("[TQ] primary norms: %d layers x %d blocks x %d x %d heads (%.1f MB)",
                            *shape, 2 * 4 * cls._primary_k_norms.numel() / (1 << 20))

        def _ensure_fused_attn(self, device):
            if self._fused_attn is None:
                tq = self._quantizer(device)
                if TurboQuantImpl._tq_format.kind == "hybrid":
                    self._fused_attn = HybridPagedAttention(tq, self.num_heads)
                else:
                    self._fused_attn = TQPagedAttention(tq, self.num_heads)
            return self._fused_attn

        # ---- cache write ----------------------------------------------------------------
        def do_kv_cache_update(self, layer, key, value, kv_cache, slot_mapping):
            """The step's K and V rows into the compressed cache (reference: backend.py:425-468,
            792-868).  SHADOW mode leaves the write of vLLM's cache to the parent."""
            if self._is_draft or key is None or value is None:
                return
            self._kv_update_seen = True
            if not TurboQuantImpl._tq_primary:
                return
            self._write_primary(key, value, kv_cache, slot_mapping)

        def _write_primary(self, key, value, kv_cache, slot_mapping) -> None:
            if slot_mapping.shape[0] != key.shape[0]:      # reference: backend.py:815-817
                return
            cls = TurboQuantImpl
            fmt = cls._tq_format
            tq = self._quantizer(key.device)
            k_rows, v_rows = primary_views(kv_cache, self.head_size, fmt)
            block_size = kv_cache.shape[2]
            if fmt.kind == "hybrid":
                hybrid_encode_and_store_pair(tq, key, value, slot_mapping, k_rows, v_rows, block_size=block_size)
                return
            self._ensure_norms(kv_cache)
            li = self._tq_layer_idx
            prep = tq.prepared_rotation()
            fused_kv_update_pair(key, value, slot_mapping, k_rows, cls._primary_k_norms[li], v_rows,
                                 cls._primary_v_norms[li], tq.rotation, tq.boundaries_inner, tq.bits,
                                 block_size=block_size, prepared=prep)

        # ---- attention --------------------------------------------------------------------
        def forward(self, layer, query, key, value, kv_cache, attn_metadata, output=None,
                    output_scale=None, output_block_scale=None):
            """Reference: backend.py:471-562."""
            if self._is_draft:
                return super().forward(layer, query, key, value, kv_cache, attn_metadata, output=output,
                                       output_scale=output_scale, output_block_scale=output_block_scale)
            if attn_metadata is None:              # vLLM's memory-profiling run
                if output is not None:
                    output.fill_(0)
                    return output
                return super().forward(layer, query, key, value, kv_cache, attn_metadata, output=output,
                                       output_scale=output_scale, output_block_scale=output_block_scale)
            assert output is not None
            if TurboQuantImpl._tq_primary:
                return self._forward_primary(layer, query, key, value, kv_cache, attn_metadata, output)
            return self._forward_shadow(layer, query, key, value, kv_cache, attn_metadata, output,
                                        output_scale, output_block_scale)

        # PRIMARY -------------------------------------------------------------------------
        def _forward_primary(self, layer, query, key, value, kv_cache, attn_metadata, output):
            # torch.compile has been seen to hand over query and value swapped for GQA models
            # (reference: backend.py:730-738); the head counts tell
            if (query is not None and value is not None and query.dim() == 3 and value.dim() == 3
                    and query.shape[1] == self.num_kv_heads and value.shape[1] == self.num_heads
                    and self.num_heads != self.num_kv_heads):
                query, value = value, query
            if getattr(attn_metadata, "max_query_len", None) == 1:
                return self._primary_decode(query, key, value, kv_cache, attn_metadata, output)
            return self._primary_prefill(query, key, value, kv_cache, attn_metadata, output)

        def _primary_decode(self, query, key, value, kv_cache, attn_metadata, output):
            """Reference: backend.py:870-953 (fused kernel on the packed rows)."""
            cls = TurboQuantImpl
            fmt = cls._tq_format
            li = self._tq_layer_idx
            n = attn_metadata.num_actual_tokens
            if query.dim() == 2:
                query = query.view(query.shape[0], self.num_heads, self.head_size)
            out3 = output.view(output.shape[0], self.num_heads, self.head_size)
            if key is not None and value is not None and not self._kv_update_seen:
                # a vLLM release without the separate cache-update op: write + attend in one op
                return self._decode_step_op(query, key, value, kv_cache, attn_metadata, output, out3)
            attn = self._ensure_fused_attn(query.device)
            k_rows, v_rows = primary_views(kv_cache, self.head_size, fmt)
            if fmt.kind == "hybrid":
                res = attn.forward(query[:n], k_rows, v_rows, attn_metadata.block_table, attn_metadata.seq_lens,
                                   block_size=kv_cache.shape[2], num_kv_heads=self.num_kv_heads, scale=self.scale)
            else:
                self._ensure_norms(kv_cache)
                res = attn.forward(query[:n], k_rows, cls._primary_k_norms[li], v_rows, cls._primary_v_norms[li],
                                   attn_metadata.block_table, attn_metadata.seq_lens,
                                   block_size=kv_cache.shape[2], num_kv_heads=self.num_kv_heads)
            out3[:n] = res.to(output.dtype)
            return output

        def _decode_step_op(self, query, key, value, kv_cache, attn_metadata, output, out3):
            cls = TurboQuantImpl
            fmt = cls._tq_format
            self._quantizer(query.device)
            n = attn_metadata.num_actual_tokens
            registered = hooks.register_custom_ops()
            common = (attn_metadata.slot_mapping, attn_metadata.block_table, attn_metadata.seq_lens,
                      self._tq_layer_idx, self.num_heads, self.num_kv_heads, self.head_size, self.scale, n)
            if fmt.kind == "hybrid":
                fn = torch.ops.tq.hybrid_decode_step if registered else hooks.hybrid_decode_step
                fn(query, key, value, kv_cache, out3, *common)
            else:
                self._ensure_norms(kv_cache)
                fn = torch.ops.tq.decode_step if registered else hooks.decode_step
                fn(query, key, value, kv_cache, out3, cls._primary_k_norms, cls._primary_v_norms, *common)
            return output

        def _primary_prefill(self, query, key, value, kv_cache, attn_metadata, output):
            """Decompress the addressed blocks into a bf16 block buffer, put the chunk's own rows in
            uncompressed, attend with the dense paged kernel (reference: backend.py:1093-1245)."""
            cls = TurboQuantImpl
            fmt = cls._tq_format
            tq = self._quantizer(query.device)
            num_blocks, block_size = kv_cache.shape[0], kv_cache.shape[2]
            if (cls._prefill_k_buf is None or cls._prefill_k_buf.shape[0] < num_blocks
                    or cls._prefill_k_buf.device != query.device
                    or tuple(cls._prefill_k_buf.shape[1:]) != (block_size, self.num_kv_heads, self.head_size)):
                blocks = max(num_blocks, cls._PREFILL_BUF_BLOCKS)
                cls._prefill_k_buf = torch.zeros(blocks, block_size, self.num_kv_heads, self.head_size,
                                                 dtype=torch.bfloat16, device=query.device)
                cls._prefill_v_buf = torch.zeros_like(cls._prefill_k_buf)
            k_buf, v_buf = cls._prefill_k_buf[:num_blocks], cls._prefill_v_buf[:num_blocks]
            k_rows, v_rows = primary_views(kv_cache, self.head_size, fmt)
            if fmt.kind == "hybrid":
                ids = attn_metadata.block_table.reshape(-1).unique().long()
                ids = ids[(ids >= 0) & (ids < num_blocks)]
                if ids.numel():
                    k_buf[ids] = tq.decode(k_rows[ids]).to(k_buf.dtype)
                    v_buf[ids] = tq.decode(v_rows[ids]).to(v_buf.dtype)
            else:
                self._ensure_norms(kv_cache)
                li = self._tq_layer_idx
                batch_decompress_active_blocks(k_rows, v_rows, k_buf, v_buf, tq, tq._packed_dim,
                                               attn_metadata.block_table, num_blocks,
                                               cls._primary_k_norms[li], cls._primary_v_norms[li])
            if key is not None and value is not None:
                self._scatter_rows(key, value, k_buf, v_buf, attn_metadata.slot_mapping, block_size)
            n = attn_metadata.num_actual_tokens
            if query.dim() == 2:
                query = query.view(query.shape[0], self.num_heads, self.head_size)
            q = query[:n].to(k_buf.dtype)
            out = torch.empty_like(q)
            cls._dense_paged_attention(self, q, k_buf, v_buf, out, attn_metadata)
            output.view(output.shape[0], self.num_heads, self.head_size)[:n] = out.to(output.dtype)
            return output

        @staticmethod
        def _scatter_rows(key, value, k_buf, v_buf, slot_mapping, block_size) -> None:
            """Rows of the current chunk into the block buffers at their slots; negative slots and
            slots beyond the buffer are left out (reference: backend.py:1247-1272)."""
            n = min(key.shape[0], slot_mapping.shape[0])
            slots = slot_mapping[:n].long()
            ok = (slots >= 0) & (slots < k_buf.shape[0] * block_size)
            slots = torch.where(ok, slots, torch.zeros_like(slots))
            src = torch.nonzero(ok).squeeze(-1)
            bi, oi = slots[src] // block_size, slots[src] % block_size
            k_buf[bi, oi] = key[:n][src].to(k_buf.dtype)
            v_buf[bi, oi] = value[:n][src].to(v_buf.dtype)

        # SHADOW ---------------------------------------------------------------------------
        def _forward_shadow(self, layer, query, key, value, kv_cache, attn_metadata, output,
                            output_scale, output_block_scale):
            """vLLM's cache stays authoritative; a compressed copy is kept beside it and decode may be
            served from the copy (reference: backend.py:499-562, 608-686)."""
            cls = TurboQuantImpl
            if self._tq_layer_idx == 0:
                cls._forward_count += 1
            self._try_init_tq_cache(kv_cache)
            cache = cls._tq_gpu_cache
            if cache is not None and key is not None and value is not None:
                try:
                    fused_encode_and_store(cache, self._tq_layer_idx, key, value, attn_metadata.slot_mapping)
                except Exception as e:      # the copy is an optimisation: serving goes on without it
                    print(f"[TQ] encode error L{self._tq_layer_idx}: {e}", file=sys.stderr, flush=True)
            if (cls._fused_enabled and cache is not None
                    and getattr(attn_metadata, "max_query_len", None) == 1):
                li = self._tq_layer_idx
                n = attn_metadata.num_actual_tokens
                if query.dim() == 2:
                    query = query.view(query.shape[0], self.num_heads, self.head_size)
                if self._fused_attn is None:
                    self._fused_attn = TQPagedAttention(cache.tq, self.num_heads)
                res = self._fused_attn.forward(query[:n], cache.k_packed[li], cache.k_norms[li], cache.v_packed[li],
                                               cache.v_norms[li], attn_metadata.block_table, attn_metadata.seq_lens,
                                               block_size=cache.block_size, num_kv_heads=self.num_kv_heads)
                output.view(output.shape[0], self.num_heads, self.head_size)[:n] = res.to(output.dtype)
                return output
            return super().forward(layer, query, key, value, kv_cache, attn_metadata, output=output,
                                   output_scale=output_scale, output_block_scale=output_block_scale)

        def _try_init_tq_cache(self, kv_cache) -> None:
            """Create the compressed copy once vLLM's profiling forwards are over and the real cache
            tensor (more than a handful of blocks) is there (reference: backend.py:608-686)."""
            cls = TurboQuantImpl
            if cls._tq_gpu_cache is not None or cls._tq_format.kind != "uniform":
                return
            if cls._forward_count < cls._INIT_AFTER_FORWARDS or kv_cache is None or kv_cache.dim() != 5:
                return
            if kv_cache.shape[0] < cls._MIN_BLOCKS_FOR_INIT:
                return
            cls._tq_gpu_cache = TQGPUCache(cls._tq_layer_counter, kv_cache.shape[0], kv_cache.shape[2],
                                           self.num_kv_heads, self.head_size, bits=cls._tq_format.bits,
                                           device=str(kv_cache.device))

    return TurboQuantImpl


# --------------------------------------------------------------------------------------------
# registration (imports vLLM only inside the call)
# --------------------------------------------------------------------------------------------
def register_turboquant_backend() -> bool:
    """Register TurboQuantBackend as vLLM's CUSTOM attention backend (reference: backend.py:
    1280-1295).  Returns False, with a warning, when vLLM is missing or refuses."""
    try:
        from vllm.v1.attention.backends.registry import AttentionBackendEnum, register_backend
        register_backend(AttentionBackendEnum.CUSTOM, f"{__name__}.TurboQuantBackend")
        logger.info("Registered TurboQuant as CUSTOM attention backend")
        return True
    except Exception as e:
        logger.warning("Failed to register TQ backend: %s", e)
        return False
