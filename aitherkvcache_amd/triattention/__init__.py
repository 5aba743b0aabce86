"""TriAttention: spectral KV compression with trigonometric-series scoring (decode path)."""
from .config import TriAttentionConfig
from .encoder import SpectralEncoding, SpectralKVEncoder
from .scorer import TrigSeriesScorer
from .attention import TriAttention
from .cache import SpectralKVCache
from .spectral import rope_frequencies

__all__ = ["TriAttentionConfig", "SpectralEncoding", "SpectralKVEncoder", "TrigSeriesScorer", "TriAttention",
           "SpectralKVCache", "rope_frequencies"]
