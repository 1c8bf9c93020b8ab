"""Indexer scores -> top-k oracle.  TEST INFRASTRUCTURE ONLY.

Restates the tail of the reference's ``LightningIndexer.__call__``
(cppmega_v4/nn/lightning_indexer.py:132-145; the FP8 variant repeats the same
lines, cppmega_v4/nn/lightning_indexer_fp8.py:145-157)::

    scores = einsum("bqhd,bkd,bqh->bqk", q, k, weights) * sm_scale
    if mask is not None: scores = scores + mask
    topk = min(index_topk, scores.shape[-1])
    indices = argpartition(-scores, topk - 1, axis=-1)[..., :topk]   (int32)

and the non-interleaved rotation the module applies to the rope slice of q and k
before it (lightning_indexer.py:47-79).  ``argpartition`` fixes the selected set
only where scores are distinct and says nothing about order; this oracle fixes
both the way ``topk.topk_selector_oracle`` does (value descending, ties toward the
lower index; ascending index for order="index").  A position whose score is -inf
(a masked one) is not selectable and leaves a ``-1`` slot, where the reference's
partition would return some arbitrary masked position.

Pinned by: an explicit four-loop evaluation on tiny shapes, the identity
sum_h w_h (q_h . k) == (sum_h w_h q_h) . k, the set returned by ``np.argpartition``
on rows with distinct scores, and the reference's rope known answers
(tests/v4/test_lightning_indexer.py:36-57).
"""

from __future__ import annotations

import numpy as np

from . import topk as _topk


def apply_non_interleaved_rope(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """Rotate (x[..., :d], x[..., d:2d]) as planes; cos/sin are (T, d) with T on axis 1 of x
    (lightning_indexer.py:47-79)."""
    x = np.asarray(x, dtype=np.float64)
    if x.shape[-1] % 2 != 0:
        raise ValueError(f"rope dim must be even, got {x.shape[-1]}")
    d = x.shape[-1] // 2
    x1, x2 = x[..., :d], x[..., d:]
    cos = np.asarray(cos, dtype=np.float64)
    sin = np.asarray(sin, dtype=np.float64)
    if x.ndim > 2:
        shape = (1, cos.shape[0]) + (1,) * (x.ndim - 3) + (cos.shape[1],)
        cos, sin = cos.reshape(shape), sin.reshape(shape)
    return np.concatenate([x1 * cos - x2 * sin, x2 * cos + x1 * sin], axis=-1)


def indexer_scores_oracle(q, k, weights, *, sm_scale: float, mask=None) -> np.ndarray:
    """float64 scores [B, Sq, Skv] (lightning_indexer.py:132-142)."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    w = np.asarray(weights, dtype=np.float64)
    if q.ndim != 4 or k.ndim != 3 or w.ndim != 3:
        raise ValueError("indexer expects q [B,Sq,H,D], k [B,Skv,D], weights [B,Sq,H]")
    if q.shape[:3] != w.shape or q.shape[0] != k.shape[0] or q.shape[3] != k.shape[2]:
        raise ValueError(f"indexer shape mismatch: q {q.shape}, k {k.shape}, weights {w.shape}")
    scores = np.einsum("bqhd,bkd,bqh->bqk", q, k, w, optimize=False) * float(sm_scale)
    if mask is not None:
        scores = scores + np.asarray(mask, dtype=np.float64)
    return scores


def indexer_topk_oracle(q, k, weights, *, sm_scale: float, index_topk: int, mask=None, starts=None, ends=None,
                        order: str = "index", scores=None) -> np.ndarray:
    """int32 [B, Sq, min(index_topk, Skv)] (lightning_indexer.py:143-145).  ``scores`` replaces the
    evaluation of the score formula (to check a selection against given float32 scores)."""
    if scores is None:
        scores = indexer_scores_oracle(q, k, weights, sm_scale=sm_scale, mask=mask)
    scores = np.asarray(scores)
    B, Sq, Skv = scores.shape
    topk = min(int(index_topk), Skv)
    flat = _topk.topk_selector_oracle(scores.reshape(B * Sq, Skv).astype(np.float32), topk, starts=starts, ends=ends,
                                      order=order, neg_inf_is_masked=mask is not None)
    return flat.reshape(B, Sq, topk)
