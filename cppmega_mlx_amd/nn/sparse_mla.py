"""Sparse multi-latent attention: shape contract, reference-path kernel and the
policy dispatcher.

Mirrors the public surface of the reference's ``cppmega_mlx/nn/sparse_mla.py``
(``SparseMLAShapes`` :38-51, ``_resolve_shapes`` :54-101,
``sparse_mla_attention_reference`` :125-210, ``sparse_mla_attention`` :337-446)
with ``torch.Tensor`` on the MI355X in place of ``mx.array``.

Semantics (reference :9-16): per query position the heads of kv-group ``g``
attend over ``kv[b, indices[b,s,g,:], g, :]``; an index of ``-1`` (any index
outside ``[0, Skv)`` here) contributes nothing; all ``qk_dim`` channels enter
QK^T and the first ``d_v`` channels are V; a row with nothing to attend to
yields zeros and ``lse == 0``.

Every function here launches a HIP kernel; there is no host-side math path.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import torch

from .. import ops
from ..runtime.kernel_policy import KernelPath, record_dispatch, selected_path

__all__ = ["SparseMLAShapes", "sparse_mla_attention", "sparse_mla_attention_reference"]

_FLOAT_CARRIERS = (torch.float32, torch.float16, torch.bfloat16)


@dataclass(frozen=True)
class SparseMLAShapes:
    """Resolved shape descriptors for sparse-MLA tensors."""

    batch: int
    seq_len: int
    seq_len_kv: int
    heads: int
    kv_group: int
    head_kv: int
    d_v: int
    qk_dim: int
    tail_dim: int
    topk: int


def _resolve_shapes(q: torch.Tensor, kv: torch.Tensor, indices: torch.Tensor, *, d_v: int | None) -> SparseMLAShapes:
    if q.ndim != 4:
        raise ValueError(f"q must be 4D [B,S,H,D_qk], got shape {tuple(q.shape)}")
    if kv.ndim != 4:
        raise ValueError(f"kv must be 4D [B,Skv,G,D_qk], got shape {tuple(kv.shape)}")
    if indices.ndim != 4:
        raise ValueError(f"indices must be 4D [B,S,G,topk], got shape {tuple(indices.shape)}")
    batch, seq_len, heads, qk_dim = q.shape
    batch_kv, seq_len_kv, kv_group, kv_dim = kv.shape
    if batch_kv != batch:
        raise ValueError(f"q.batch={batch} != kv.batch={batch_kv}")
    if kv_dim != qk_dim:
        raise ValueError(f"q last-dim {qk_dim} != kv last-dim {kv_dim}")
    if heads % kv_group != 0:
        raise ValueError(f"heads {heads} not divisible by kv_group {kv_group}")
    if tuple(indices.shape[:3]) != (batch, seq_len, kv_group):
        raise ValueError(
            f"indices shape {tuple(indices.shape)} does not match (B,S,G,topk)=({batch},{seq_len},{kv_group},*)"
        )
    d_v_resolved = qk_dim if d_v is None else int(d_v)
    if not (0 < d_v_resolved <= qk_dim):
        raise ValueError(f"d_v must be in (0, {qk_dim}], got {d_v_resolved}")
    return SparseMLAShapes(
        batch=batch, seq_len=seq_len, seq_len_kv=seq_len_kv, heads=heads, kv_group=kv_group,
        head_kv=heads // kv_group, d_v=d_v_resolved, qk_dim=qk_dim, tail_dim=qk_dim - d_v_resolved,
        topk=indices.shape[3],
    )


def _check_carriers(q: torch.Tensor, kv: torch.Tensor, indices: torch.Tensor) -> None:
    if q.dtype not in _FLOAT_CARRIERS or kv.dtype not in _FLOAT_CARRIERS:
        raise TypeError(f"q/kv must be float32, float16 or bfloat16; got {q.dtype}, {kv.dtype}")
    if indices.dtype not in (torch.int32, torch.int64):
        raise TypeError(f"indices must be int32 or int64; got {indices.dtype}")


def _float_carrier_forward(
    q: torch.Tensor,
    kv: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float | torch.Tensor | None,
    d_v: int | None,
    return_lse: bool,
    kernel: str,
    out: torch.Tensor | None = None,
    lse: torch.Tensor | None = None,
    out_dtype: torch.dtype | None = None,
):
    shapes = _resolve_shapes(q, kv, indices, d_v=d_v)
    _check_carriers(q, kv, indices)
    if isinstance(sm_scale, torch.Tensor):                # a device float32[1], read by the kernel on the stream
        scale = sm_scale
    else:
        scale = shapes.qk_dim ** -0.5 if sm_scale is None else float(sm_scale)
    if out is None:
        out = torch.empty((shapes.batch, shapes.seq_len, shapes.heads, shapes.d_v),
                          dtype=out_dtype or q.dtype, device=q.device)
    if lse is None and return_lse:
        lse = torch.empty((shapes.batch, shapes.seq_len, shapes.heads), dtype=torch.float32, device=q.device)
    ops.sparse_mla_forward(q, kv, indices, sm_scale=scale, d_v=shapes.d_v, out=out, lse=lse, kernel=kernel)
    return (out, lse) if return_lse else out


def sparse_mla_attention_reference(
    q: torch.Tensor,
    kv: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float | None = None,
    d_v: int | None = None,
    return_lse: bool = False,
) -> torch.Tensor | Tuple[torch.Tensor, torch.Tensor]:
    """Reference-path forward: the fp32 one-wavefront-per-head kernel.

    Same signature and result contract as the reference's pure-MLX fallback
    (``out`` in ``q.dtype`` ``[B,S,H,d_v]``; ``lse`` fp32 ``[B,S,H]``, natural
    log, 0 for a row without valid indices).
    """
    return _float_carrier_forward(q, kv, indices, sm_scale=sm_scale, d_v=d_v, return_lse=return_lse,
                                  kernel="scalar")


def sparse_mla_attention(
    q: torch.Tensor,
    kv: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float | None = None,
    d_v: int | None = None,
    return_lse: bool = False,
) -> torch.Tensor | Tuple[torch.Tensor, torch.Tensor]:
    """Production entry point routed by ``CPPMEGA_KERNEL_PATH[__SPARSE_MLA]``.

    AUTO: the MFMA kernel when it covers the shape, else the reference-path
    kernel.  REFERENCE: the reference-path kernel.  PATH_C: the MFMA kernel,
    error if it does not cover the shape.  PATH_B: raises (retired surface).
    """
    path = selected_path("sparse_mla")
    if path is KernelPath.PATH_B:
        record_dispatch("sparse_mla", path, "direct_msl_path_b_retired")
        raise RuntimeError("sparse_mla_apply: Metal path unavailable: the direct-MSL Path B surface is retired")
    if path is KernelPath.REFERENCE:
        record_dispatch("sparse_mla", path, "hip_scalar_fp32")
        return sparse_mla_attention_reference(q, kv, indices, sm_scale=sm_scale, d_v=d_v, return_lse=return_lse)
    if path is KernelPath.PATH_C:
        record_dispatch("sparse_mla", path, "hip_mfma_gfx950")
        try:
            return _float_carrier_forward(q, kv, indices, sm_scale=sm_scale, d_v=d_v, return_lse=return_lse,
                                          kernel="mfma")
        except ops._lib.NativeCallError as exc:
            raise RuntimeError(f"sparse_mla_attention: Path C unavailable: {exc}") from exc
    shapes = _resolve_shapes(q, kv, indices, d_v=d_v)
    _check_carriers(q, kv, indices)
    chosen = ops.sparse_mla_selected_kernel(q, kv, indices, d_v=shapes.d_v)
    record_dispatch("sparse_mla", path, "hip_mfma_gfx950" if chosen == "mfma" else "hip_scalar_fp32")
    return _float_carrier_forward(q, kv, indices, sm_scale=sm_scale, d_v=d_v, return_lse=return_lse, kernel=chosen)
