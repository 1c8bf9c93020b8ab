"""The reference's CPU fallback restated op for op in float32 torch, for timing on the host cores.

TEST INFRASTRUCTURE ONLY -- the shipped package never imports this module; ``bench.py`` times it
as the ``cpu_baseline`` (kind "port": the reference itself is Python on MLX, which cannot be
installed here).  Each function follows the reference's own sequence of array operations, so that
the host time is what that fallback would cost on these cores, not what a tuned CPU kernel could
reach.  Results are checked against the float64 NumPy oracle in tests/test_oracle_torch_cpu.py.
"""

from __future__ import annotations

import torch


def sparse_mla_fallback(q: torch.Tensor, kv: torch.Tensor, indices: torch.Tensor, *, sm_scale: float | None = None,
                        d_v: int | None = None, chunk: int = 64):
    """cppmega_mlx/nn/sparse_mla.py:104-210 (``_gather_kv`` + ``sparse_mla_attention_reference``):
    gather kv[b, max(idx, 0), g] -> [B,S,G,topk,D]; scores = q . gathered^T * sm_scale in float32;
    invalid (idx == -1) -> -inf; stable softmax with all-invalid rows -> zeros; out = probs . gathered[..., :d_v];
    lse = m + log(sumexp) (0 for all-invalid rows).  Chunked over the query axis: the reference gathers
    all of [B,S,G,topk,D] at once (:18-19), which at the prefill configuration is 38.7 GB.

    q [B,S,H,D] float32, kv [B,Skv,G,D] float32, indices [B,S,G,topk] int64.  Returns (out [B,S,H,d_v], lse [B,S,H])."""
    B, S, H, D = q.shape
    G = kv.shape[2]
    topk = indices.shape[-1]
    d_v = D if d_v is None else d_v
    sm_scale = D ** -0.5 if sm_scale is None else sm_scale
    hg = H // G
    out = torch.empty((B, S, H, d_v), dtype=torch.float32)
    lse = torch.empty((B, S, H), dtype=torch.float32)
    kv_g = kv.permute(0, 2, 1, 3)                                          # [B,G,Skv,D]
    for s0 in range(0, S, chunk):
        s1 = min(S, s0 + chunk)
        idx = indices[:, s0:s1]                                            # [B,s,G,topk]
        valid = idx != -1
        safe = idx.clamp_min(0).permute(0, 2, 1, 3)                        # [B,G,s,topk]
        gathered = torch.gather(kv_g[:, :, None].expand(B, G, s1 - s0, kv.shape[1], D), 3,
                                safe[..., None].expand(B, G, s1 - s0, topk, D))    # [B,G,s,topk,D]
        qc = q[:, s0:s1].reshape(B, s1 - s0, G, hg, D).permute(0, 2, 1, 3, 4)      # [B,G,s,hg,D]
        scores = torch.matmul(qc, gathered.transpose(-1, -2)) * sm_scale           # [B,G,s,hg,topk]
        mask = valid.permute(0, 2, 1, 3)[:, :, :, None, :]
        scores = torch.where(mask, scores, torch.full_like(scores, float("-inf")))
        m = scores.max(dim=-1, keepdim=True).values
        m = torch.where(torch.isfinite(m), m, torch.zeros_like(m))
        e = torch.exp(scores - m)
        e = torch.where(mask, e, torch.zeros_like(e))
        denom = e.sum(dim=-1, keepdim=True)
        probs = e / torch.where(denom > 0, denom, torch.ones_like(denom))
        o = torch.matmul(probs, gathered[..., :d_v])                               # [B,G,s,hg,d_v]
        out[:, s0:s1] = o.permute(0, 2, 1, 3, 4).reshape(B, s1 - s0, H, d_v)
        l = torch.where(denom > 0, m + torch.log(torch.where(denom > 0, denom, torch.ones_like(denom))), torch.zeros_like(m))
        lse[:, s0:s1] = l[..., 0].permute(0, 2, 1, 3).reshape(B, s1 - s0, H)
    return out, lse


def topk_fallback(scores: torch.Tensor, k: int, *, ends: torch.Tensor | None = None) -> torch.Tensor:
    """cppmega_mlx/nn/_tilelang/topk_selector.py:227-330 with the canonical order of
    tests/test_tilelang_topk.py:47-73: mask outside [0, end) to -inf, stable sort by descending score,
    keep the first k, -1 where the rank is not below the valid count; returned ascending by index."""
    rows, width = scores.shape
    s = scores.float()
    if ends is not None:
        col = torch.arange(width)[None, :]
        s = torch.where(col < ends[:, None].long(), s, torch.full_like(s, float("-inf")))
    order = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :k]
    valid = torch.gather(s, 1, order) > float("-inf")
    picked = torch.where(valid, order, torch.full_like(order, width))
    picked = torch.sort(picked, dim=-1).values
    return torch.where(picked < width, picked, torch.full_like(picked, -1)).to(torch.int32)


def fused_fp8_gemm_fallback(w_f32: torch.Tensor, scale: torch.Tensor, x: torch.Tensor, block: int = 128) -> torch.Tensor:
    """cppmega_v4/nn/_external/_mlx_lm_fp8_dequant_vendored.py:24-46 then a float32 matmul
    (cppmega_v4/_tilelang/fused_fp8_gemm.py:34-146 computes the same sum without materialising the
    dequantised weight): w_f32 is the decoded e4m3 weight [N,K], scale [N, K/block] float32, x [M,K]."""
    n, k = w_f32.shape
    deq = (w_f32.reshape(n, k // block, block) * scale[..., None]).reshape(n, k)
    return torch.matmul(x.float(), deq.t())
