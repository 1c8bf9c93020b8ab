"""Inference-side pieces of the sparse-attention path: the sparse FP8 KV cache."""

from .engine import SparseFP8KVCache, SparseFP8KVCacheConfig

__all__ = ["SparseFP8KVCache", "SparseFP8KVCacheConfig"]
