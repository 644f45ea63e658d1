"""Decode-time runtime: KV caches and the decode dispatch registry."""
from .cache import (FlashSVDDenseKVCache, FlashSVDLegacySparseKVCache, FlashSVDV15DenseKVCache, LowRankKVCache)

__all__ = ["FlashSVDDenseKVCache", "FlashSVDLegacySparseKVCache", "FlashSVDV15DenseKVCache", "LowRankKVCache"]
