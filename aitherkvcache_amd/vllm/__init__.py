"""Serving-side glue for the hot path: the CUSTOM attention backend (backend.TurboQuantBackend,
made on first access), the plugin entry point, the tq::decode_step / tq::hybrid_decode_step custom
ops and the kv-cache-dtype name map.  Importing this package does not import vLLM."""
from .kv_cache_dtype import resolve_kv_cache_dtype, KV_CACHE_DTYPES
from .decompress import batch_decompress_active_blocks, decode_blocks
from .hooks import register_custom_ops, init_quantizer, reset_state
from .engine import tq_page_size_bytes, align_page_size, reshape_primary, primary_views
from .cache import TQGPUCache
from .backend import register_turboquant_backend

__all__ = ["resolve_kv_cache_dtype", "KV_CACHE_DTYPES", "register_custom_ops", "init_quantizer",
           "reset_state", "batch_decompress_active_blocks", "decode_blocks", "tq_page_size_bytes",
           "align_page_size", "reshape_primary", "primary_views", "TQGPUCache", "register_turboquant_backend"]
