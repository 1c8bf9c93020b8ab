"""Float-carrier sparse-MLA forward through the tuned HIP kernels ("Path C").

Surface of the reference's ``cppmega_mlx/nn/_tilelang/sparse_mla_path_c.py``:
``sparse_mla_fwd_path_c_direct`` :3232-3311, ``sparse_mla_fwd_path_c``
:3424-3502, ``sparse_mla_path_c_apply`` :3660-3748,
``SparseMLAPathCDirectError``, ``sparse_mla_path_c_status``; the training side:
``_sparse_mla_bwd_path_c_direct`` :3314-3421, ``sparse_mla_bwd_path_c`` :3505-3552 and the
differentiable ``sparse_mla_path_c_metal_apply`` with its vjp :3555-3605.

The reference's kernel needs fp16 carriers; here q/kv may be bfloat16, float16
or float32 and ``out`` takes the carrier's dtype (any of the three when the
caller owns it).  ``lse`` is fp32 ``[B,S,H]``.  Indices may be int32 or int64
and are never cast.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import torch

from ... import _lib, ops
from ..sparse_mla import _check_carriers, _float_carrier_forward, _resolve_shapes

__all__ = [
    "SparseMLAPathCDirectError",
    "SparseMLAPathCStatus",
    "sparse_mla_bwd_path_c",
    "sparse_mla_fwd_path_c",
    "sparse_mla_fwd_path_c_direct",
    "sparse_mla_path_c_metal_apply",
    "sparse_mla_path_c_apply",
    "sparse_mla_path_c_status",
]


class SparseMLAPathCDirectError(RuntimeError):
    """Raised when the owner-output forward route cannot run."""


@dataclass(frozen=True)
class SparseMLAPathCStatus:
    available: bool
    reason: str


def sparse_mla_path_c_status() -> SparseMLAPathCStatus:
    try:
        st = _lib.status()
    except _lib.NativeLibraryError as exc:
        return SparseMLAPathCStatus(False, str(exc))
    if st["gfx950_devices"] < 1:
        return SparseMLAPathCStatus(False, st["message"])
    return SparseMLAPathCStatus(True, "sparse-MLA HIP kernels (gfx950) are available")


def _validate_owner_outputs(q, out, lse, shapes) -> None:
    if not isinstance(out, torch.Tensor) or not isinstance(lse, torch.Tensor):
        raise TypeError("out and lse must be torch.Tensor")
    want_out = (shapes.batch, shapes.seq_len, shapes.heads, shapes.d_v)
    want_lse = (shapes.batch, shapes.seq_len, shapes.heads)
    if tuple(out.shape) != want_out:
        raise ValueError(f"out must have shape {want_out}; got {tuple(out.shape)}")
    if tuple(lse.shape) != want_lse:
        raise ValueError(f"lse must have shape {want_lse}; got {tuple(lse.shape)}")
    if out.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise TypeError(f"out must be float32, float16 or bfloat16; got {out.dtype}")
    if lse.dtype != torch.float32:
        raise TypeError(f"lse must be torch.float32; got {lse.dtype}")


def sparse_mla_fwd_path_c_direct(
    q: torch.Tensor,
    kv: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale_buf: torch.Tensor,
    out: torch.Tensor,
    lse: torch.Tensor,
    d_v: int | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Owner-output forward.  ``sm_scale_buf`` is the reference's 1-element
    float32 scalar buffer; it stays on the device and the kernel reads it on the stream."""
    status = sparse_mla_path_c_status()
    if not status.available:
        raise SparseMLAPathCDirectError(status.reason)
    shapes = _resolve_shapes(q, kv, indices, d_v=d_v)
    _check_carriers(q, kv, indices)
    if not isinstance(sm_scale_buf, torch.Tensor) or sm_scale_buf.numel() != 1 or sm_scale_buf.dtype != torch.float32:
        raise ValueError("sm_scale_buf must be a 1-element float32 tensor")
    _validate_owner_outputs(q, out, lse, shapes)
    try:
        _float_carrier_forward(q, kv, indices, sm_scale=sm_scale_buf, d_v=shapes.d_v,
                               return_lse=True, kernel="auto", out=out, lse=lse)
    except (_lib.NativeCallError, _lib.NativeLibraryError) as exc:
        raise SparseMLAPathCDirectError(f"sparse-MLA forward dispatch failed: {type(exc).__name__}: {exc}") from exc
    return out, lse


def sparse_mla_fwd_path_c(
    q: torch.Tensor,
    kv: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float | None = None,
    d_v: int | None = None,
    sm_scale_buf: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
    lse: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor] | None:
    """Forward returning ``(out, lse)``, or ``None`` when the kernels cannot run."""
    owner_args = (sm_scale_buf, out, lse)
    if any(arg is not None for arg in owner_args):
        if any(arg is None for arg in owner_args):
            raise SparseMLAPathCDirectError("owner-output route requires sm_scale_buf, out and lse together")
        return sparse_mla_fwd_path_c_direct(q, kv, indices, sm_scale_buf=sm_scale_buf, out=out, lse=lse, d_v=d_v)
    shapes = _resolve_shapes(q, kv, indices, d_v=d_v)
    if not sparse_mla_path_c_status().available:
        return None
    return _float_carrier_forward(q, kv, indices, sm_scale=sm_scale, d_v=shapes.d_v, return_lse=True, kernel="auto")


def sparse_mla_path_c_apply(
    q: torch.Tensor,
    kv: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float | None = None,
    d_v: int | None = None,
    return_lse: bool = False,
    force_path_c: bool = False,
) -> torch.Tensor | Tuple[torch.Tensor, torch.Tensor]:
    """Apply sparse MLA through the tuned kernels (forward only)."""
    shapes = _resolve_shapes(q, kv, indices, d_v=d_v)
    status = sparse_mla_path_c_status()
    if not status.available:
        raise RuntimeError(f"sparse_mla_path_c_apply: Path C unavailable: {status.reason}")
    del force_path_c  # nothing to fall back to: the HIP kernels are the only path
    return _float_carrier_forward(q, kv, indices, sm_scale=sm_scale, d_v=shapes.d_v, return_lse=return_lse,
                                  kernel="auto")


def _sparse_mla_bwd_path_c_direct(q: torch.Tensor, kv: torch.Tensor, d_out: torch.Tensor, indices: torch.Tensor, *,
                                  sm_scale_buf: torch.Tensor, d_v: int | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """Backward into fresh owner outputs: ``dq`` in q's dtype, ``dkv`` float32 (cleared, then
    accumulated with atomic adds).  The reference requires fp16 carriers; any of float32 /
    float16 / bfloat16 is taken here, all three operands alike."""
    status = sparse_mla_path_c_status()
    if not status.available:
        raise SparseMLAPathCDirectError(status.reason)
    shapes = _resolve_shapes(q, kv, indices, d_v=d_v)
    _check_carriers(q, kv, indices)
    if d_out.dtype != q.dtype or kv.dtype != q.dtype:
        raise SparseMLAPathCDirectError("Sparse-MLA backward takes q, kv and d_out in one carrier dtype without hidden casts; got "
                                        f"q={q.dtype}, kv={kv.dtype}, d_out={d_out.dtype}")
    if not isinstance(sm_scale_buf, torch.Tensor) or tuple(sm_scale_buf.shape) != (1,) or sm_scale_buf.dtype != torch.float32:
        raise SparseMLAPathCDirectError("Sparse-MLA backward requires sm_scale_buf with shape (1,) and dtype torch.float32")
    dq = torch.empty_like(q)
    dkv = torch.empty(tuple(kv.shape), dtype=torch.float32, device=kv.device)
    try:
        ops.sparse_mla_backward(q.contiguous(), kv.contiguous(), d_out.contiguous(), indices.contiguous(), sm_scale=sm_scale_buf,
                                d_v=shapes.d_v, dq=dq, dkv=dkv, clear_dkv=True)
    except (_lib.NativeCallError, _lib.NativeLibraryError) as exc:
        raise SparseMLAPathCDirectError(f"sparse-MLA backward dispatch failed: {type(exc).__name__}: {exc}") from exc
    return dq, dkv


def sparse_mla_bwd_path_c(q: torch.Tensor, kv: torch.Tensor, d_out: torch.Tensor, indices: torch.Tensor, *,
                          sm_scale: float | None = None, d_v: int | None = None) -> tuple[torch.Tensor, torch.Tensor] | None:
    """``(dq, dkv)`` for the cotangent ``d_out``, or ``None`` when the kernels cannot run."""
    if not sparse_mla_path_c_status().available:
        return None
    shapes = _resolve_shapes(q, kv, indices, d_v=d_v)
    scale = shapes.qk_dim ** -0.5 if sm_scale is None else float(sm_scale)
    buf = torch.tensor([scale], dtype=torch.float32, device=q.device)
    try:
        return _sparse_mla_bwd_path_c_direct(q, kv, d_out, indices, sm_scale_buf=buf, d_v=shapes.d_v)
    except SparseMLAPathCDirectError:
        return None


class _SparseMLAPathCFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, kv, indices):
        ctx.save_for_backward(q, kv, indices)
        out = sparse_mla_path_c_apply(q, kv, indices)
        return out

    @staticmethod
    def backward(ctx, cotangent):
        q, kv, indices = ctx.saved_tensors
        # (the direct form: a carrier or shape error surfaces as what it is instead of as "unavailable")
        shapes = _resolve_shapes(q, kv, indices, d_v=None)
        buf = torch.tensor([shapes.qk_dim ** -0.5], dtype=torch.float32, device=q.device)
        dq, dkv = _sparse_mla_bwd_path_c_direct(q, kv, cotangent.to(q.dtype).contiguous(), indices, sm_scale_buf=buf, d_v=shapes.d_v)
        return dq, dkv.to(kv.dtype), None


def sparse_mla_path_c_metal_apply(q: torch.Tensor, kv: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """Differentiable default-parameter forward (sm_scale = D^-0.5, d_v = D); gradients come from
    the backward kernel.  Keeps the reference's name; there is no Metal here."""
    return _SparseMLAPathCFunction.apply(q, kv, indices)
