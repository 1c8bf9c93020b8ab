"""DSA indexer KL loss oracle.  TEST INFRASTRUCTURE ONLY.

Float64 restatement of what the reference's two fused kernels compute together
(cppmega_mlx/nn/_tilelang/dsa_splitk_indexer_loss.py: stage 1 :398-656, stage 2 :855-1165,
wrapper :1327-1570): per (batch b, query position sq)

    s_h[j] = softmax_scale * query[sq,b,h,:] . key[j,b,h,:] (+ mask[b,sq,j])      j <= sq
    p[j]   = mean_h softmax_j(s_h)[j]
    q[j]   = softmax over ALL j < Sk of index_scores[b,sq,j] (+ mask[b,sq,j])
    loss[b,sq] = sum_{j <= sq} p[j] * (log(p[j] + 1e-10) - log(q[j] + 1e-10))

and the wrapper returns mean(loss) * loss_coeff.  The sparse variant's mask is 0 at a row's
top-k positions and -inf elsewhere (:1443-1445).  Guards as in the kernels: an all-masked
softmax has maximum 0 and denominator 1 (every probability 0).

Pinned in tests/test_oracle_dsa_loss.py by closed forms — zero query and key with a uniform
index give log(Sk) - log(sq + 1); an index equal to the log of the attention distribution over
a full causal row gives 0 — and by an explicit triple loop.
"""

from __future__ import annotations

import numpy as np

EPS = 1e-10


def sparse_index_mask(topk_indices, seq_k: int) -> np.ndarray:
    """[AB, ASq, Sk]: 0 at the listed positions, -inf elsewhere."""
    idx = np.asarray(topk_indices).astype(np.int64)
    if idx.size and (idx.min() < 0 or idx.max() >= seq_k):
        raise ValueError(f"topk_indices out of range [0, {seq_k}); got [{idx.min()}, {idx.max()}].")
    mask = np.full(idx.shape[:2] + (seq_k,), -np.inf)
    np.put_along_axis(mask, idx, 0.0, axis=-1)
    return mask


def _softmax_guarded(x: np.ndarray) -> np.ndarray:
    m = x.max()
    if not np.isfinite(m):
        m = 0.0
    e = np.exp(x - m)
    d = e.sum()
    return e / (d if d > 0 else 1.0)


def row_loss(index_row, q_row, k_b, n: int, softmax_scale: float, mask_row=None) -> float:
    """One (b, sq): ``index_row`` [Sk], ``q_row`` [AH, AD], ``k_b`` [Sk, AH, AD], ``n`` causally visible keys."""
    AH = q_row.shape[0]
    p = np.zeros(n)
    for h in range(AH):
        s = k_b[:n, h, :] @ q_row[h, :] * softmax_scale
        if mask_row is not None:
            s = s + mask_row[:n]
        p += _softmax_guarded(s)
    p /= AH
    qd = _softmax_guarded(index_row + (mask_row if mask_row is not None else 0.0))[:n]
    return float(np.sum(p * (np.log(p + EPS) - np.log(qd + EPS))))


def dsa_indexer_loss_per_position(index_scores, query, key, *, softmax_scale: float, index_mask=None) -> np.ndarray:
    """float64 [AB, ASq]."""
    q = np.asarray(query, dtype=np.float64)
    k = np.asarray(key, dtype=np.float64)
    idx = np.asarray(index_scores, dtype=np.float64)
    ASq, AB, AH, AD = q.shape
    Sk = k.shape[0]
    if k.shape[1:] != q.shape[1:]:
        raise ValueError(f"query/key shape mismatch: query {q.shape}, key {k.shape}")
    mask = None if index_mask is None else np.asarray(index_mask, dtype=np.float64)
    loss = np.zeros((AB, ASq))
    for b in range(AB):
        for sq in range(ASq):
            loss[b, sq] = row_loss(idx[b, sq], q[sq, b], k[:, b], min(sq + 1, Sk), float(softmax_scale),
                                   None if mask is None else mask[b, sq])
    return loss


def dsa_indexer_loss(index_scores, topk_indices, query, key, softmax_scale: float, loss_coeff: float, sparse_loss: bool) -> float:
    q = np.asarray(query)
    if 0 in q.shape or np.asarray(key).shape[0] == 0:
        return 0.0
    mask = sparse_index_mask(topk_indices, np.asarray(key).shape[0]) if sparse_loss else None
    return float(dsa_indexer_loss_per_position(index_scores, query, key, softmax_scale=softmax_scale, index_mask=mask).mean() * loss_coeff)
