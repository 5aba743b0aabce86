"""TriAttention: spectral KV compression with trigonometric-series scoring (decode path)."""
from .config import TriAttentionConfig
from .encoder import SpectralEncoding, SpectralKVEncoder
from .attention import TriAttention
from .cache import SpectralKVCache
from .spectral import rope_frequencies

__all__ = ["TriAttentionConfig", "SpectralEncoding", "SpectralKVEncoder", "TriAttention",
           "SpectralKVCache", "rope_frequencies"]
