"""CPU oracle (test infrastructure only) for the cache append and the sparse index producers.

Restates, in NumPy:
* ``ContiguousKVCache.update_and_fetch_sparse_fp8`` (cppmega_mlx/inference/engine.py:76-98):
  prepared bytes and scales are appended along the sequence axis;
* the producer in front of it, ``fp8_per_token_quant`` (sparse_mla_fp8_path_c.py:2667-2753), via
  ``oracle.fp8.quantize_per_token``, and its per-128-channel form (same formula per block;
  with ``pow2`` the smallest power of two ``s`` with ``448 s >= amax``, 1.0 for a zero block);
* ``causal_sparse_indices`` (cppmega_mlx/nn/attention.py:251-284);
* ``sparse_indices_from_attention_mask`` (attention.py:287-360): positions of valid keys get
  their position as score, invalid ones -1; ascending argsort; the last min(topk, K) entries;
  entries whose score is negative become -1.

Pinned by the reference's own known answers (tests/test_attention.py:120-167, transcribed in
tests/golden/reference_kats.json), by brute force on small inputs and by closed forms
(tests/test_oracle_kv_cache.py).  Nothing in the product imports this module.
"""

from __future__ import annotations

import numpy as np

from . import fp8


def causal_sparse_indices(batch_size, seq_length, kv_group, topk, *, query_offset=0, key_length=None):
    key_length = seq_length if key_length is None else key_length
    q = (query_offset + np.arange(seq_length, dtype=np.int64))[:, None]
    idx = q - np.arange(topk, dtype=np.int64)[None, :]
    idx = np.where((idx >= 0) & (idx < key_length), idx, -1)
    return np.broadcast_to(idx.reshape(1, seq_length, 1, topk), (batch_size, seq_length, kv_group, topk)).astype(np.int32)


def sparse_indices_from_attention_mask(mask, *, batch_size, seq_length, kv_group, topk, key_length):
    mask = np.asarray(mask)
    valid = {2: lambda m: m[None, None], 3: lambda m: m[:, None], 4: lambda m: m}[mask.ndim](mask)
    valid_mask = valid if valid.dtype == np.bool_ else np.isfinite(valid.astype(np.float32))
    valid_mask = np.broadcast_to(valid_mask, (batch_size, kv_group, seq_length, key_length)).transpose(0, 2, 1, 3)
    pos = np.arange(key_length, dtype=np.int32)
    scores = np.where(valid_mask, pos, -1)
    ordered = np.argsort(scores, axis=-1, kind="stable")
    selected = ordered[..., -min(topk, key_length):].astype(np.int32)
    sel_scores = np.take_along_axis(scores, selected, axis=-1)
    return np.where(sel_scores >= 0, selected, -1).astype(np.int32)


def quantize_block128(x: np.ndarray, *, pow2: bool = False):
    """x [..., D] float32, D % 128 == 0 -> (codes uint8 [..., D], scale float32 [..., D/128])."""
    x = np.asarray(x, np.float32)
    xb = x.reshape(x.shape[:-1] + (x.shape[-1] // 128, 128))
    amax = np.abs(xb).max(axis=-1).astype(np.float32)
    if pow2:
        with np.errstate(divide="ignore"):
            e = np.ceil(np.log2(amax.astype(np.float64) / 448.0))
        scale = np.where(amax > 0, np.exp2(e), 1.0).astype(np.float32)
    else:
        scale = np.maximum(amax * np.float32(1.0 / 448.0), np.float32(1e-12)).astype(np.float32)
    q = np.clip((xb / scale[..., None]).astype(np.float32), -448.0, 448.0)
    return fp8.e4m3_encode(q).reshape(x.shape), scale


def append(cache_kv, cache_scale, position, kv_fp8, kv_scale):
    """In-place append of prepared rows at ``position`` (int or per-batch array)."""
    B, S = kv_fp8.shape[:2]
    pos = np.broadcast_to(np.asarray(position), (B,))
    for b in range(B):
        cache_kv[b, pos[b]:pos[b] + S] = kv_fp8[b]
        cache_scale[b, pos[b]:pos[b] + S] = kv_scale[b]
    return cache_kv, cache_scale
