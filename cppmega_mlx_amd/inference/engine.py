"""The sparse FP8 side of the contiguous KV cache.

Mirrors the part of ``ContiguousKVCache`` that the sparse-attention path uses
(``cppmega_mlx/inference/engine.py:76-98``, validation ``:436-466``):
``update_and_fetch_sparse_fp8(layer_idx, kv_fp8, kv_scale)`` appends prepared e4m3 bytes
``[B, S, G, D]`` and float32 scales ``[B, S, G]`` along the sequence axis and returns the cache
up to the new position, as references to the cache's own buffers.

The reference grows MLX-LM ``KVCache`` objects by concatenation; here every layer owns
preallocated device buffers of ``max_seq_len`` positions and an append is one HIP kernel that
writes the new rows in place (torch only allocates the buffers and takes views).
``append_latent`` is the same append with the producer fused in: bf16 latent rows are quantised
to e4m3 with one float32 scale per 128 channels (the layout the latent decode kernel gathers)
and the rope tail is stored beside them.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import ops

__all__ = ["SparseFP8KVCacheConfig", "SparseFP8KVCache"]


def _validate_positive_int(name: str, value: int) -> None:
    if not isinstance(value, int) or isinstance(value, bool):
        raise TypeError(f"{name} must be an int")
    if value <= 0:
        raise ValueError(f"{name} must be positive")


@dataclass(frozen=True)
class SparseFP8KVCacheConfig:
    """Shape contract (the reference's ``ContiguousKVCacheConfig`` fields that apply)."""

    num_layers: int
    batch_size: int
    num_kv_heads: int
    head_dim: int
    max_seq_len: int
    rope_dim: int = 0           # > 0: a bf16 rope tail per token beside the latent bytes
    scale_block: int = 0        # 0: one scale per row (reference); 128: one per 128 channels
    pow2_scales: bool = False   # append_latent: round block scales up to powers of two

    def __post_init__(self) -> None:
        for name in ("num_layers", "batch_size", "num_kv_heads", "head_dim", "max_seq_len"):
            _validate_positive_int(name, getattr(self, name))
        if self.scale_block not in (0, 128):
            raise ValueError("scale_block must be 0 (per row) or 128")
        if self.head_dim % 128 != 0:
            raise ValueError("head_dim must be divisible by 128")
        if self.rope_dim < 0:
            raise ValueError("rope_dim must be non-negative")


class _Layer:
    def __init__(self, cfg: SparseFP8KVCacheConfig, device) -> None:
        B, T, G, D = cfg.batch_size, cfg.max_seq_len, cfg.num_kv_heads, cfg.head_dim
        self.kv = torch.zeros((B, T, G, D), dtype=torch.uint8, device=device)
        sshape = (B, T, G) if not cfg.scale_block else (B, T, G, D // cfg.scale_block)
        self.scale = torch.zeros(sshape, dtype=torch.float32, device=device)
        self.rope = torch.zeros((B, T, G, cfg.rope_dim), dtype=torch.bfloat16, device=device) if cfg.rope_dim else None
        self.offset = 0


class SparseFP8KVCache:
    """One preallocated (bytes, scales[, rope]) cache per layer."""

    def __init__(self, config: SparseFP8KVCacheConfig, device: torch.device | str = "cuda") -> None:
        self.config = config
        self.sparse_fp8_layers = [_Layer(config, device) for _ in range(config.num_layers)]

    def _sparse_fp8_layer(self, layer_idx: int) -> _Layer:
        if not isinstance(layer_idx, int):
            raise TypeError("layer_idx must be an int")
        if layer_idx < 0 or layer_idx >= len(self.sparse_fp8_layers):
            raise IndexError("layer_idx out of range")
        return self.sparse_fp8_layers[layer_idx]

    def layer_position(self, layer_idx: int) -> int:
        return self._sparse_fp8_layer(layer_idx).offset

    def position(self) -> int:
        offsets = [layer.offset for layer in self.sparse_fp8_layers]
        if any(o != offsets[0] for o in offsets):
            raise RuntimeError("contiguous KV cache layer offsets are not aligned")
        return offsets[0]

    def trim(self, num_tokens: int) -> int:
        """Drop the newest ``num_tokens`` positions of every layer; returns how many were dropped."""
        n = min(int(num_tokens), min(layer.offset for layer in self.sparse_fp8_layers))
        for layer in self.sparse_fp8_layers:
            layer.offset -= n
        return n

    def update_and_fetch_sparse_fp8(self, layer_idx: int, kv_fp8: torch.Tensor, kv_scale: torch.Tensor):
        """Append prepared FP8 KV bytes / scales; returns ``(kv[B, pos, G, D], scale[B, pos, G(, D/128)])``
        as views of the cache (reference: ``engine.py:76-98``)."""
        layer = self._sparse_fp8_layer(layer_idx)
        cfg = self.config
        if not isinstance(kv_fp8, torch.Tensor) or not isinstance(kv_scale, torch.Tensor):
            raise TypeError("kv_fp8 and kv_scale must be torch.Tensor instances")
        if kv_fp8.ndim != 4:
            raise ValueError("kv_fp8 must have shape (batch, sequence, kv_heads, head_dim)")
        want_scale_ndim = 3 if not cfg.scale_block else 4
        if kv_scale.ndim != want_scale_ndim:
            raise ValueError("kv_scale must have shape (batch, sequence, kv_heads)" + (" + (head_dim/128,)" if cfg.scale_block else ""))
        if tuple(kv_fp8.shape[:-1]) != tuple(kv_scale.shape[:3]):
            raise ValueError("kv_fp8 and kv_scale must agree on batch/sequence/kv_heads")
        if kv_fp8.dtype != torch.uint8:
            raise ValueError("kv_fp8 must be an FP8 byte buffer with dtype uint8")
        if kv_scale.dtype != torch.float32:
            raise ValueError("kv_scale must be float32")
        batch, sequence, num_kv_heads, head_dim = (int(d) for d in kv_fp8.shape)
        if batch != cfg.batch_size:
            raise ValueError("kv_fp8 batch dimension must match cache config batch_size")
        _validate_positive_int("sequence", sequence)
        if num_kv_heads != cfg.num_kv_heads:
            raise ValueError("kv_fp8 kv_heads dimension must match cache config num_kv_heads")
        if head_dim != cfg.head_dim:
            raise ValueError("kv_fp8 head_dim dimension must match cache config head_dim")
        if layer.offset + sequence > cfg.max_seq_len:
            raise RuntimeError("sparse FP8 cache update would exceed max_seq_len")
        ops.kv_cache_append(kv_fp8, src_scale=kv_scale, kv_cache=layer.kv, scale_cache=layer.scale,
                            position=layer.offset, scale_block=cfg.scale_block)
        layer.offset += sequence
        return layer.kv[:, :layer.offset], layer.scale[:, :layer.offset]

    def append_latent(self, layer_idx: int, latent: torch.Tensor, rope: torch.Tensor | None = None):
        """Quantise ``latent[B, S, G, D]`` (float) on the way into the cache and store ``rope``
        beside it; returns ``(kv, scale, rope)`` views up to the new position."""
        layer = self._sparse_fp8_layer(layer_idx)
        cfg = self.config
        if latent.ndim != 4 or tuple(latent.shape[0:1] + latent.shape[2:]) != (cfg.batch_size, cfg.num_kv_heads, cfg.head_dim):
            raise ValueError("latent must have shape (batch, sequence, kv_heads, head_dim) matching the cache config")
        sequence = int(latent.shape[1])
        _validate_positive_int("sequence", sequence)
        if (rope is None) != (layer.rope is None):
            raise ValueError("rope rows go with a cache configured with rope_dim > 0, and only with one")
        if layer.offset + sequence > cfg.max_seq_len:
            raise RuntimeError("sparse FP8 cache update would exceed max_seq_len")
        ops.kv_cache_append(latent, kv_cache=layer.kv, scale_cache=layer.scale, position=layer.offset,
                            rope=rope, rope_cache=layer.rope, scale_block=cfg.scale_block, pow2_scales=cfg.pow2_scales)
        layer.offset += sequence
        n = layer.offset
        return layer.kv[:, :n], layer.scale[:, :n], (None if layer.rope is None else layer.rope[:, :n])
