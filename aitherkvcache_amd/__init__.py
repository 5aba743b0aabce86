"""MI355X-native TurboQuant KV-cache hot path.

Drop-in for the hot path of aither-kvcache (TurboQuant.encode/decode, HybridTurboQuant,
fused_tq4_kv_update / fused_encode_and_store, TQPagedAttention, TriAttention.decode_step and the
tq::decode_step / tq::hybrid_decode_step custom ops), running hand-written gfx950 HIP kernels
behind a C ABI (include/aitherkv.h).  HIP devices only -- there is no CPU implementation.
"""
from .quantizer import TurboQuant, TurboQuantConfig
from .hybrid_quantizer import HybridTurboQuant, HybridLayout, GroupLayout
from .fused_kv_update import fused_tq4_kv_update, fused_kv_update, fused_kv_update_pair, fused_encode_and_store
from .fused_attention import TQPagedAttention
from .hybrid_attention import HybridPagedAttention, hybrid_encode_and_store, hybrid_encode_and_store_pair

__all__ = [
    "TurboQuant", "TurboQuantConfig", "HybridTurboQuant", "HybridLayout", "GroupLayout",
    "fused_tq4_kv_update", "fused_kv_update", "fused_kv_update_pair", "fused_encode_and_store", "TQPagedAttention",
    "HybridPagedAttention", "hybrid_encode_and_store", "hybrid_encode_and_store_pair",
]
__version__ = "0.1.0"
