"""Serving-side glue for the hot path: the tq::decode_step / tq::hybrid_decode_step custom ops
and the kv-cache-dtype name map.  Importing this package does not import vLLM."""
from .kv_cache_dtype import resolve_kv_cache_dtype, KV_CACHE_DTYPES
from .decompress import batch_decompress_active_blocks, decode_blocks
from .hooks import register_custom_ops, init_quantizer, reset_state

__all__ = ["resolve_kv_cache_dtype", "KV_CACHE_DTYPES", "register_custom_ops", "init_quantizer",
           "reset_state", "batch_decompress_active_blocks", "decode_blocks"]
