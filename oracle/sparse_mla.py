"""Sparse multi-latent-attention oracle.  TEST INFRASTRUCTURE ONLY.

``sparse_mla_oracle`` restates ``sparse_mla_attention_reference``
(cppmega_mlx/nn/sparse_mla.py:125-210): gather ``kv[b, max(idx,0), g]``,
``scores = q . gathered^T * sm_scale``, invalid entries -> -inf, max-subtracted
softmax with the all-invalid guard (m = 0, output 0, lse 0), ``out = probs .
gathered[..., :d_v]``.  The kernels' wider validity rule (``idx < 0 or idx >=
Skv`` is invalid, cppmega_mlx/nn/_tilelang/sparse_mla_fp8_path_c.py:1864) is a
superset of the reference's ``idx == -1`` and agrees with it on every input the
reference defines, so the oracle uses the wider rule.  Attention sinks follow
sparse_mla_fp8_path_c.py:1900-1928: one extra logit per head that joins the max
and the denominator but contributes no value row.

The quantised variants are "dequantise, then the oracle":
  * per-token fp32 scale   -- sparse_mla_fp8.py:149-156, 500-509
  * E8M0 per 32 elements   -- sparse_mla_blockscaled_path_c.py:1086-1106
  * fp32 per 128 latent channels + bf16 rope tail -- the block-128 form of the
    same contract (docs/tilelang_ports/sparse_mla_blockscaled.md:17-36).
Arithmetic is float64 so the oracle's own rounding never enters a tolerance.
"""

from __future__ import annotations

import numpy as np

from . import fp8


def resolve_shapes(q, kv, indices, d_v):
    """Shape contract of cppmega_mlx/nn/sparse_mla.py:54-101."""
    if q.ndim != 4:
        raise ValueError(f"q must be 4D [B,S,H,D_qk], got shape {q.shape}")
    if kv.ndim != 4:
        raise ValueError(f"kv must be 4D [B,Skv,G,D_qk], got shape {kv.shape}")
    if indices.ndim != 4:
        raise ValueError(f"indices must be 4D [B,S,G,topk], got shape {indices.shape}")
    B, S, H, D = q.shape
    Bk, Skv, G, Dk = kv.shape
    if Bk != B:
        raise ValueError(f"q.batch={B} != kv.batch={Bk}")
    if Dk != D:
        raise ValueError(f"q last-dim {D} != kv last-dim {Dk}")
    if H % G:
        raise ValueError(f"heads {H} not divisible by kv_group {G}")
    if tuple(indices.shape[:3]) != (B, S, G):
        raise ValueError(f"indices shape {indices.shape} does not match (B,S,G,topk)=({B},{S},{G},*)")
    dv = D if d_v is None else int(d_v)
    if not 0 < dv <= D:
        raise ValueError(f"d_v must be in (0, {D}], got {dv}")
    return B, S, H, D, Skv, G, H // G, dv, indices.shape[3]


def sparse_mla_oracle(
    q: np.ndarray,
    kv: np.ndarray,
    indices: np.ndarray,
    *,
    sm_scale: float | None = None,
    d_v: int | None = None,
    sinks: np.ndarray | None = None,
    chunk: int = 64,
) -> tuple[np.ndarray, np.ndarray]:
    """Float64 forward.  Returns (out [B,S,H,d_v], lse [B,S,H]).

    ``q`` [B,S,H,D] and ``kv`` [B,Skv,G,D] are already-dequantised real numbers.
    Queries are processed ``chunk`` at a time so the gathered block stays small.
    """
    q = np.asarray(q, dtype=np.float64)
    kv = np.asarray(kv, dtype=np.float64)
    indices = np.asarray(indices)
    B, S, H, D, Skv, G, hpg, dv, topk = resolve_shapes(q, kv, indices, d_v)
    scale = D ** -0.5 if sm_scale is None else float(sm_scale)
    out = np.zeros((B, S, H, dv), dtype=np.float64)
    lse = np.zeros((B, S, H), dtype=np.float64)
    sink = None if sinks is None else np.asarray(sinks, dtype=np.float64).reshape(G, hpg)
    for b in range(B):
        for g in range(G):
            for s0 in range(0, S, chunk):
                s1 = min(S, s0 + chunk)
                idx = indices[b, s0:s1, g, :].astype(np.int64)            # [s, topk]
                valid = (idx >= 0) & (idx < Skv)
                rows = kv[b, np.where(valid, idx, 0), g, :]               # [s, topk, D]
                qq = q[b, s0:s1, g * hpg:(g + 1) * hpg, :]                # [s, hpg, D]
                sc = np.einsum("shd,skd->shk", qq, rows) * scale
                sc = np.where(valid[:, None, :], sc, -np.inf)
                m = sc.max(axis=-1)                                       # [s, hpg]
                if sink is not None:
                    m = np.maximum(m, sink[g][None, :])
                any_live = np.isfinite(m)
                m_safe = np.where(any_live, m, 0.0)
                e = np.where(valid[:, None, :], np.exp(sc - m_safe[..., None]), 0.0)
                denom = e.sum(axis=-1)
                if sink is not None:
                    denom = denom + np.exp(sink[g][None, :] - m_safe)
                safe = np.where(denom > 0, denom, 1.0)
                p = e / safe[..., None]
                o = np.einsum("shk,skd->shd", p, rows[..., :dv])
                out[b, s0:s1, g * hpg:(g + 1) * hpg, :] = o
                lse[b, s0:s1, g * hpg:(g + 1) * hpg] = np.where(denom > 0, m_safe + np.log(safe), 0.0)
    return out, lse


def sparse_mla_loop_oracle(q, kv, indices, *, sm_scale, d_v):
    """Independent per-(b,s,h) scalar-loop formulation used to pin the batched
    oracle (same role as tests/test_tilelang_sparse_mla.py:121-158)."""
    q = np.asarray(q, dtype=np.float64)
    kv = np.asarray(kv, dtype=np.float64)
    B, S, H, D = q.shape
    Skv, G = kv.shape[1], kv.shape[2]
    hpg = H // G
    out = np.zeros((B, S, H, d_v))
    lse = np.zeros((B, S, H))
    for b in range(B):
        for s in range(S):
            for h in range(H):
                g = h // hpg
                live = [int(j) for j in indices[b, s, g] if 0 <= j < Skv]
                if not live:
                    continue
                logits = np.array([np.dot(q[b, s, h], kv[b, j, g]) * sm_scale for j in live])
                top = logits.max()
                w = np.exp(logits - top)
                for wj, j in zip(w, live):
                    out[b, s, h] += (wj / w.sum()) * kv[b, j, g, :d_v]
                lse[b, s, h] = top + np.log(w.sum())
    return out, lse


# ---- dequantisers for the prepared-buffer ABIs --------------------------------

def dequant_per_token(codes: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """codes u8 [..., K], scale f32 [...] -> float64 (sparse_mla_fp8.py:149-156)."""
    return fp8.e4m3_decode(codes, np.float64) * np.asarray(scale, dtype=np.float64)[..., None]


def dequant_e8m0(codes: np.ndarray, scale_bytes: np.ndarray, block: int = 32) -> np.ndarray:
    """codes u8 [..., K], scale u8 [..., K/block] -> float64."""
    s = fp8.e8m0_decode(scale_bytes, np.float64)
    return fp8.e4m3_decode(codes, np.float64) * np.repeat(s, block, axis=-1)


def dequant_block_latent(codes: np.ndarray, scale: np.ndarray, rope: np.ndarray | None, block: int = 128) -> np.ndarray:
    """Latent cache record -> float64 rows.

    codes u8 [..., Kl]; scale f32 [..., Kl/block]; rope (already real numbers,
    bf16-representable) [..., R] or None.  Result [..., Kl+R]: the dequantised
    latent followed by the rope tail (packed-KV layout: V = first d_v channels).
    """
    lat = fp8.e4m3_decode(codes, np.float64) * np.repeat(np.asarray(scale, dtype=np.float64), block, axis=-1)
    if rope is None:
        return lat
    return np.concatenate([lat, np.asarray(rope, dtype=np.float64)], axis=-1)


INVALID_SCORE_SENTINEL = np.float32(-3.4028234663852886e38)


def sparse_mla_scores_oracle(q: np.ndarray, kv: np.ndarray, indices: np.ndarray, *, sm_scale: float) -> np.ndarray:
    """scores[b,s,h,j] = sm_scale * q[b,s,h] . kv[b, indices[b,s,g,j], g] in float64 -> float32; a slot
    whose index is negative or >= S_kv holds the finite sentinel.  Follows the score stage of the
    reference's fused kernel and its QK-only seam
    (cppmega_mlx/nn/_tilelang/sparse_mla_fp8_path_c.py:1862-1884, sentinel :80)."""
    B, S, H, D = q.shape
    _, Skv, G, _ = kv.shape
    topk = indices.shape[-1]
    hpg = H // G
    out = np.empty((B, S, H, topk), dtype=np.float32)
    for b in range(B):
        for s in range(S):
            for g in range(G):
                idx = indices[b, s, g]
                ok = (idx >= 0) & (idx < Skv)
                rows = kv[b, np.where(ok, idx, 0), g].astype(np.float64)            # [topk, D]
                qs = q[b, s, g * hpg:(g + 1) * hpg].astype(np.float64)               # [hpg, D]
                sc = (qs @ rows.T) * float(sm_scale)
                out[b, s, g * hpg:(g + 1) * hpg] = np.where(ok[None, :], sc, INVALID_SCORE_SENTINEL).astype(np.float32)
    return out


def sparse_mla_bwd_oracle(q, kv, indices, d_out, *, sm_scale: float | None = None, d_v: int | None = None):
    """Float64 gradients (dq [B,S,H,D], dkv [B,Skv,G,D]) of ``sparse_mla_oracle``'s output for the
    cotangent ``d_out`` [B,S,H,d_v]; the closed form of the reference's backward kernel
    (cppmega_mlx/nn/_tilelang/sparse_mla_path_c.py:2700-2814): p = softmax over the valid
    selected keys, dp_k = d_out . kv_k[:d_v], ds = p * (dp - sum p dp), dq = sm_scale * ds . K,
    dkv[i_k] += sm_scale * ds_k * q (+ p_k * d_out on the first d_v channels).  A key index
    < 0 or >= Skv is skipped (the forward's rule); repeated indices accumulate.
    Pinned in tests/test_oracle_sparse_mla.py by central finite differences of the forward
    oracle and by torch autograd through a dense masked attention."""
    q = np.asarray(q, dtype=np.float64)
    kv = np.asarray(kv, dtype=np.float64)
    d_out = np.asarray(d_out, dtype=np.float64)
    indices = np.asarray(indices)
    B, S, H, D, Skv, G, hpg, dv, topk = resolve_shapes(q, kv, indices, d_v)
    scale = D ** -0.5 if sm_scale is None else float(sm_scale)
    dq = np.zeros_like(q)
    dkv = np.zeros_like(kv)
    for b in range(B):
        for s in range(S):
            for g in range(G):
                idx = indices[b, s, g].astype(np.int64)
                valid = (idx >= 0) & (idx < Skv)
                if not valid.any():
                    continue
                sel = idx[valid]
                rows = kv[b, sel, g, :]                                    # [n, D]
                for h in range(g * hpg, (g + 1) * hpg):
                    sc = rows @ q[b, s, h] * scale
                    e = np.exp(sc - sc.max())
                    p = e / e.sum()
                    dp = rows[:, :dv] @ d_out[b, s, h]
                    ds = p * (dp - np.dot(p, dp))
                    dq[b, s, h] = scale * (ds @ rows)
                    contrib = scale * np.outer(ds, q[b, s, h])
                    contrib[:, :dv] += np.outer(p, d_out[b, s, h])
                    np.add.at(dkv[b, :, g, :], sel, contrib)
    return dq, dkv
