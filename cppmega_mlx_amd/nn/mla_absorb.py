"""Absorbed MLA decode: attention in the latent space of the compressed KV cache.

Surface of the reference's ``cppmega_v4/nn/mla_absorb.py``: ``absorb_weights`` :39-77,
``absorbed_mla_decode`` :80-138, ``standard_mla_decode`` :141-172 (the reference's own
numerical oracle for the identity absorbed == standard).

The two per-head projections that bracket the attention call run on ``ops.head_gemm``
(Y[m,g,n] = sum_k X[m,g,k] W[g,n,k], weights streamed once with the contraction index
contiguous).  ``absorb_weights`` therefore returns tensors with the reference's shapes whose
memory is already in that order: ``w_uk_abs`` [H, D_k, D_kv] is the transposed view of the
dense ``w_uk`` [H, D_kv, D_k], and ``w_uv_w_o`` [H, D_kv, D_model] is a view of a dense
[D_model, H, D_kv] buffer, so the output projection is one product over k = H * D_kv.  Weights
that arrive in another memory order are re-laid out on every call.  The attention between the
two projections is the sparse-MLA kernel over every cached position; an additive mask takes
the scores kernel plus tensor operations instead.
"""

from __future__ import annotations

import torch

from .. import ops

__all__ = ["absorb_weights", "absorbed_mla_decode", "standard_mla_decode", "absorb_query", "unabsorb_output"]


def absorb_weights(w_uk: torch.Tensor, w_uv: torch.Tensor, w_o: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """(w_uk_abs [H, D_k, D_kv] = W_UK^T per head, w_uv_w_o [H, D_kv, D_model] = W_UV @ W_O[h])."""
    if w_uk.ndim != 3:
        raise ValueError(f"w_uk must be [H, D_kv, D_k], got {tuple(w_uk.shape)}")
    if w_uv.ndim != 3 or w_uv.shape[0] != w_uk.shape[0] or w_uv.shape[1] != w_uk.shape[1]:
        raise ValueError(f"w_uv shape {tuple(w_uv.shape)} inconsistent with w_uk {tuple(w_uk.shape)}")
    h, d_kv, d_v = w_uv.shape
    if w_o.ndim != 2 or w_o.shape[0] != h * d_v:
        raise ValueError(f"w_o shape {tuple(w_o.shape)} must be (H*D_v={h * d_v}, D_model)")
    d_model = w_o.shape[1]
    w_uk_abs = w_uk.contiguous().transpose(1, 2)
    # P[m, h, v] = sum_d w_o[h * D_v + d, m] * w_uv[h, v, d]
    w_o_t = w_o.reshape(h, d_v, d_model).permute(2, 0, 1).contiguous()            # [D_model, H, D_v], once at load time
    fused = torch.empty((d_model, h, d_kv), dtype=w_uv.dtype, device=w_uv.device)
    ops.head_gemm(w_o_t, w_uv.contiguous(), out=fused)
    return w_uk_abs, fused.permute(1, 2, 0)


def _dense(t: torch.Tensor) -> torch.Tensor:
    return t if t.is_contiguous() else t.contiguous()


def absorb_query(q: torch.Tensor, w_uk_abs: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """q_abs[b,t,h,:] = q[b,t,h,:] @ w_uk_abs[h] ("bthk,hkv->bthv"); ``out`` may be the leading D_kv
    channels of wider query rows (a view with its own strides)."""
    b, t, h, d_k = q.shape
    d_kv = w_uk_abs.shape[2]
    if out is None:
        out = torch.empty((b, t, h, d_kv), dtype=q.dtype, device=q.device)
    x = _dense(q).view(b * t, h, d_k)
    if out.stride(-1) != 1 or out.stride(0) != t * out.stride(1):
        raise ValueError(f"out must be a [B, T, H, D_kv] view with dense rows; got strides {out.stride()}")
    y = out.as_strided((b * t, h, d_kv), (out.stride(1), out.stride(2), 1), out.storage_offset())
    ops.head_gemm(x, _dense(w_uk_abs.transpose(1, 2)), out=y)
    return out


def unabsorb_output(v_abs: torch.Tensor, w_uv_w_o: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[b,t,:] = sum_h v_abs[b,t,h,:] @ w_uv_w_o[h] ("bthv,hvm->btm")."""
    b, t, h, d_kv = v_abs.shape
    d_model = w_uv_w_o.shape[2]
    if out is None:
        out = torch.empty((b, t, d_model), dtype=v_abs.dtype, device=v_abs.device)
    w = _dense(w_uv_w_o.permute(2, 0, 1)).view(1, d_model, h * d_kv)
    ops.head_gemm(_dense(v_abs).view(b * t, 1, h * d_kv), w, out=out.view(b * t, 1, d_model))
    return out


def absorbed_mla_decode(q: torch.Tensor, c_kv: torch.Tensor, w_uk_abs: torch.Tensor, w_uv_w_o: torch.Tensor, *,
                        sm_scale: float | None = None, mask: torch.Tensor | None = None) -> torch.Tensor:
    """MLA decode step in the absorbed form: [B, T, D_model]."""
    if q.ndim != 4:
        raise ValueError(f"q must be [B, T, H, D_k], got {tuple(q.shape)}")
    if c_kv.ndim != 3:
        raise ValueError(f"c_kv must be [B, T_kv, D_kv], got {tuple(c_kv.shape)}")
    if w_uk_abs.ndim != 3 or w_uv_w_o.ndim != 3:
        raise ValueError("absorbed weights must be 3D (H, ..., ...)")
    b, t, h, d_k = q.shape
    t_kv, d_kv = c_kv.shape[1], c_kv.shape[2]
    if tuple(w_uk_abs.shape) != (h, d_k, d_kv):
        raise ValueError(f"w_uk_abs must be (H={h}, D_k={d_k}, D_kv={d_kv}), got {tuple(w_uk_abs.shape)}")
    if w_uv_w_o.shape[0] != h or w_uv_w_o.shape[1] != d_kv:
        raise ValueError(f"w_uv_w_o must be (H={h}, D_kv={d_kv}, D_model), got {tuple(w_uv_w_o.shape)}")
    if sm_scale is None:
        sm_scale = d_k ** -0.5
    q_abs = absorb_query(q, w_uk_abs)
    kv = _dense(c_kv).to(q_abs.dtype).view(b, t_kv, 1, d_kv)
    indices = torch.arange(t_kv, dtype=torch.int32, device=q.device).expand(b, t, 1, t_kv).contiguous()
    if mask is None:
        v_abs = torch.empty((b, t, h, d_kv), dtype=q_abs.dtype, device=q.device)
        ops.sparse_mla_forward(q_abs, kv, indices, sm_scale=float(sm_scale), d_v=d_kv, out=v_abs)
    else:
        logits = torch.empty((b, t, h, t_kv), dtype=torch.float32, device=q.device)
        ops.sparse_mla_scores(q_abs, kv, indices, sm_scale=float(sm_scale), scores=logits)
        weights = torch.softmax(logits + mask.to(torch.float32), dim=-1)
        v_abs = torch.einsum("bthk,bkv->bthv", weights, c_kv.to(torch.float32)).to(q_abs.dtype)
    return unabsorb_output(v_abs, w_uv_w_o)


def standard_mla_decode(q: torch.Tensor, c_kv: torch.Tensor, w_uk: torch.Tensor, w_uv: torch.Tensor, w_o: torch.Tensor, *,
                        sm_scale: float | None = None, mask: torch.Tensor | None = None) -> torch.Tensor:
    """The non-absorbed form (K and V materialised), kept as tensor operations: the comparison the
    reference uses to state the identity."""
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    k = torch.einsum("bkv,hvd->bkhd", c_kv, w_uk)
    v = torch.einsum("bkv,hvd->bkhd", c_kv, w_uv)
    logits = torch.einsum("bthk,bnhk->bthn", q, k) * sm_scale
    if mask is not None:
        logits = logits + mask
    weights = torch.softmax(logits, dim=-1)
    o_h = torch.einsum("bthn,bnhv->bthv", weights, v)
    b, t, h, d_v = o_h.shape
    return o_h.reshape(b, t, h * d_v) @ w_o
