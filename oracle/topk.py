"""Top-k selector oracle.  TEST INFRASTRUCTURE ONLY.

Restates ``topk_selector_reference``
(cppmega_mlx/nn/_tilelang/topk_selector.py:227-330): positions outside
``[clip(start), clip(end))`` are masked to -inf, the ``k`` largest entries are
selected, and slots whose rank is >= ``valid_count`` hold ``-1``.  Where the
reference's ``argpartition`` leaves tie membership and output order open, this
oracle fixes them the way the reference's own NumPy oracle does
(tests/test_tilelang_topk.py:47-73: stable argsort of the negated row, i.e.
value descending, lower index first among equals).  ``-0.0 == +0.0`` under the
float compare, so the stable sort breaks that tie by index as well.

NaN scores are outside the pinned contract (the reference tests never feed
them); this oracle treats a NaN like a masked position so that the behaviour is
at least defined: it is never selected and does not count as valid.
"""

from __future__ import annotations

import numpy as np


def _clip_bounds(starts, ends, rows: int, width: int) -> tuple[np.ndarray, np.ndarray]:
    lo = np.zeros(rows, dtype=np.int64) if starts is None else np.asarray(starts).astype(np.int64)
    hi = np.full(rows, width, dtype=np.int64) if ends is None else np.asarray(ends).astype(np.int64)
    if lo.shape != (rows,) or hi.shape != (rows,):
        raise ValueError(f"starts/ends must have shape ({rows},); got {lo.shape}, {hi.shape}")
    return np.clip(lo, 0, width), np.clip(hi, 0, width)


def topk_selector_oracle(
    scores: np.ndarray,
    k: int,
    *,
    starts=None,
    ends=None,
    order: str = "index",
    neg_inf_is_masked: bool = False,
) -> np.ndarray:
    """Return int32 ``(rows, k)`` indices of the k largest entries per row.

    order="value": value descending, ties toward the lower index (the order the
        reference's Path C kernel emits, tests/test_tilelang_topk.py:596-610).
    order="index": the same set, ascending by index.
    In both orders the ``-1`` padding sits at the tail.
    neg_inf_is_masked: also treat an in-range ``-inf`` score as masked (callers
        that mask by writing -inf into the scores instead of passing bounds,
        cppmega_v4/nn/lightning_indexer.py:140-145).
    """
    scores = np.asarray(scores)
    if scores.ndim != 2:
        raise ValueError(f"topk_selector expects a (B, T) array; got shape {scores.shape}")
    rows, width = scores.shape
    if k < 1:
        raise ValueError(f"topk must be >= 1; got {k}")
    if k > width:
        raise ValueError(f"topk={k} exceeds sequence length {width}")
    if order not in ("index", "value"):
        raise ValueError(f"unknown order {order!r}")
    lo, hi = _clip_bounds(starts, ends, rows, width)
    col = np.arange(width)
    out = np.full((rows, k), -1, dtype=np.int32)
    for r in range(rows):
        row = scores[r].astype(np.float32)
        live = (col >= lo[r]) & (col < hi[r]) & ~np.isnan(row)
        if neg_inf_is_masked:
            live &= row != -np.inf
        cand = col[live]
        vals = row[live]
        # stable sort on the negated values: descending value, ascending index.
        ranked = cand[np.argsort(-vals, kind="stable")][:k]
        if order == "index":
            ranked = np.sort(ranked)
        out[r, : ranked.size] = ranked
    return out


def topk_bruteforce(scores: np.ndarray, k: int) -> list[set[int]]:
    """O(T^2) ranker used to pin the oracle on tiny rows: element i is selected
    iff fewer than k elements beat it, where j beats i when s[j] > s[i] or
    (s[j] == s[i] and j < i)."""
    scores = np.asarray(scores, dtype=np.float32)
    sets = []
    for row in scores:
        chosen = set()
        for i, v in enumerate(row):
            beaten_by = sum(1 for j, w in enumerate(row) if w > v or (w == v and j < i))
            if beaten_by < k:
                chosen.add(i)
        sets.append(chosen)
    return sets
