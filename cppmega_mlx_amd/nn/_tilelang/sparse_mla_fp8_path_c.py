"""Per-token-scaled FP8 sparse-MLA forward over prepared buffers, with sinks.

Surface of the reference's ``cppmega_mlx/nn/_tilelang/sparse_mla_fp8_path_c.py``:
``sparse_mla_fp8_path_c_apply_direct`` :2756-2869 and
``sparse_mla_fp8_path_c_apply`` :2872-3004 with the kernel contract of
:1821-1956: ``q_scale`` float32 ``[B,S,H]``, ``kv_scale`` float32 ``[B,Skv,G]``,
score = (sum dec*dec) * qs * ks * sm_scale, optional attention ``sinks`` ``[H]``
(one extra logit per head in the max and the denominator, no value row),
``out`` float32/float16/bfloat16 (``output_dtype``), ``lse`` float32.

``sparse_mla_fp8_bwd_path_c`` :3007-3080 is the backward over the same prepared
buffers (kernel :1966-2214): float32 gradients with respect to the dequantised q and kv.
``sparse_mla_fp8_path_c_apply_prepared_float`` :3138-3252 is the differentiable owner wrapper
(forward over the prepared buffers, gradients delivered straight through to the float q / kv
the buffers were produced from); ``sparse_mla_fp8_path_c_apply_from_float`` :3255-3280 fails
closed, as in the reference.

A float32 ``kv_scale`` of rank 4 selects the block-128 latent layout described
in ``sparse_mla_blockscaled_path_c`` (per-token is its one-block case), so the
sink path is available for the latent KV cache as well.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ... import _lib, ops
from . import _prepared

__all__ = [
    "SparseMLAFp8PathCDirectError",
    "SparseMLAFp8PathCStatus",
    "sparse_mla_fp8_path_c_apply",
    "sparse_mla_fp8_path_c_apply_direct",
    "sparse_mla_fp8_path_c_status",
    "sparse_mla_fp8_bwd_path_c",
    "sparse_mla_fp8_path_c_apply_from_float",
    "sparse_mla_fp8_path_c_apply_prepared_float",
    "fp8_sparse_mla_indexed_qk_reduce_path_c",
    "fp8_sparse_mla_qk_reduce_path_c",
]

_OP = "FP8 Sparse-MLA Path C apply"
_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


class SparseMLAFp8PathCDirectError(RuntimeError):
    """Raised when the prepared-buffer owner-output path cannot run."""


@dataclass(frozen=True)
class SparseMLAFp8PathCStatus:
    available: bool
    reason: str
    target: str = "hip-gfx950"


def sparse_mla_fp8_path_c_status() -> SparseMLAFp8PathCStatus:
    try:
        st = _lib.status()
    except _lib.NativeLibraryError as exc:
        return SparseMLAFp8PathCStatus(False, str(exc))
    if st["gfx950_devices"] < 1:
        return SparseMLAFp8PathCStatus(False, st["message"])
    return SparseMLAFp8PathCStatus(True, "FP8 sparse-MLA HIP kernels (gfx950) are available")


def _float_dtype(dtype, *, name: str = "dtype"):
    if dtype not in _FLOATS:
        raise TypeError(f"{name} must be float32, float16, or bfloat16; got {dtype}")
    return dtype


def _check_sinks(sinks, heads: int):
    if sinks is None:
        return None
    if not isinstance(sinks, torch.Tensor):
        raise TypeError("sinks must be a torch.Tensor")
    if tuple(sinks.shape) != (heads,):
        raise ValueError(f"sinks must have shape ({heads},), got {tuple(sinks.shape)}")
    if sinks.dtype != torch.float32:
        raise ValueError("sinks must be float32")
    return sinks


def sparse_mla_fp8_path_c_apply_direct(
    q_fp8: torch.Tensor,
    q_scale: torch.Tensor | None,
    kv_fp8: torch.Tensor,
    kv_scale: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float,
    out: torch.Tensor,
    lse: torch.Tensor,
    d_v: int | None = None,
    sinks: torch.Tensor | None = None,
    output_dtype: torch.dtype | None = None,
    kv_rope: torch.Tensor | None = None,
    kernel: str = "auto",
) -> tuple[torch.Tensor, torch.Tensor]:
    """Forward into caller-owned ``out``/``lse``; returns those same objects."""
    status = sparse_mla_fp8_path_c_status()
    if not status.available:
        raise SparseMLAFp8PathCDirectError(status.reason)
    plan = _prepared.plan_prepared(q_fp8, q_scale, kv_fp8, kv_scale, indices, d_v=d_v, kv_rope=kv_rope,
                                   op_name=_OP, family="fp8")
    want = _float_dtype(out.dtype if output_dtype is None else output_dtype, name="output_dtype") \
        if isinstance(out, torch.Tensor) else None
    _prepared.validate_owner_outputs(out, lse, plan, out_dtype=want)
    sinks = _check_sinks(sinks, plan.heads)
    try:
        _prepared.launch_prepared(q_fp8, kv_fp8, indices, plan, sm_scale=sm_scale, out=out, lse=lse,
                                  kv_rope=kv_rope, sinks=sinks, kernel=kernel)
    except (_lib.NativeCallError, _lib.NativeLibraryError) as exc:
        raise SparseMLAFp8PathCDirectError(
            f"FP8 Sparse-MLA forward dispatch failed: {type(exc).__name__}: {exc}"
        ) from exc
    return out, lse


def sparse_mla_fp8_path_c_apply(
    q_fp8: torch.Tensor,
    q_scale: torch.Tensor | None,
    kv_fp8: torch.Tensor,
    kv_scale: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float,
    d_v: int | None = None,
    sinks: torch.Tensor | None = None,
    return_lse: bool = False,
    force_path_c: bool = False,
    out: torch.Tensor | None = None,
    lse: torch.Tensor | None = None,
    output_dtype: torch.dtype | None = None,
    kv_rope: torch.Tensor | None = None,
    kernel: str = "auto",
):
    """Fused FP8 sparse-MLA forward over prepared GPU buffers."""
    if (out is None) != (lse is None):
        raise ValueError("sparse_mla_fp8_path_c_apply owner-output route requires both out and lse buffers")
    if out is not None and lse is not None:
        direct_out, direct_lse = sparse_mla_fp8_path_c_apply_direct(
            q_fp8, q_scale, kv_fp8, kv_scale, indices, sm_scale=sm_scale, out=out, lse=lse, d_v=d_v, sinks=sinks,
            output_dtype=output_dtype, kv_rope=kv_rope, kernel=kernel)
        return (direct_out, direct_lse) if return_lse else direct_out

    status = sparse_mla_fp8_path_c_status()
    if not status.available:
        if force_path_c:
            raise RuntimeError(f"sparse_mla_fp8_path_c_apply: {status.reason}")
        return None
    plan = _prepared.plan_prepared(q_fp8, q_scale, kv_fp8, kv_scale, indices, d_v=d_v, kv_rope=kv_rope,
                                   op_name=_OP, family="fp8")
    default = torch.float16 if q_fp8.dtype == torch.uint8 else q_fp8.dtype
    out_dtype = _float_dtype(default if output_dtype is None else output_dtype, name="output_dtype")
    sinks = _check_sinks(sinks, plan.heads)
    out = torch.empty((plan.batch, plan.seq_len, plan.heads, plan.d_v), dtype=out_dtype, device=q_fp8.device)
    lse = torch.empty((plan.batch, plan.seq_len, plan.heads), dtype=torch.float32, device=q_fp8.device)
    try:
        _prepared.launch_prepared(q_fp8, kv_fp8, indices, plan, sm_scale=sm_scale, out=out, lse=lse,
                                  kv_rope=kv_rope, sinks=sinks, kernel=kernel)
    except (_lib.NativeCallError, _lib.NativeLibraryError) as exc:
        raise RuntimeError(
            f"sparse_mla_fp8_path_c_apply: kernel dispatch failed: {type(exc).__name__}: {exc}"
        ) from exc
    return (out, lse) if return_lse else out


def sparse_mla_fp8_bwd_path_c(
    q_fp8: torch.Tensor,
    q_scale: torch.Tensor,
    kv_fp8: torch.Tensor,
    kv_scale: torch.Tensor,
    d_out: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float,
    d_v: int | None = None,
    force_path_c: bool = False,
    causal: bool = False,
    dq_buffer: torch.Tensor | None = None,
    dkv_buffer: torch.Tensor | None = None,
):
    """Backward over prepared per-token FP8 buffers: ``(dq_dequant [B,S,H,K], dkv_dequant
    [B,Skv,G,K])`` float32, written into ``dq_buffer`` / ``dkv_buffer`` when given."""
    status = sparse_mla_fp8_path_c_status()
    if not status.available:
        if force_path_c:
            raise RuntimeError(f"sparse_mla_fp8_bwd_path_c: {status.reason}")
        return None
    del causal  # the sparse indices define the scatter pattern; kept for call compatibility
    plan = _prepared.plan_prepared(q_fp8, q_scale, kv_fp8, kv_scale, indices, d_v=d_v, kv_rope=None, op_name=_OP, family="fp8")
    if plan.layout != "per_token":
        raise ValueError("sparse_mla_fp8_bwd_path_c takes per-token float32 scales (q_scale [B,S,H], kv_scale [B,Skv,G])")
    want = (plan.batch, plan.seq_len, plan.heads, plan.d_v)
    if tuple(d_out.shape) != want:
        raise ValueError(f"d_out must have shape {want}; got {tuple(d_out.shape)}")
    _float_dtype(d_out.dtype, name="d_out dtype")
    dq_shape = (plan.batch, plan.seq_len, plan.heads, plan.qk_dim)
    dkv_shape = (plan.batch, plan.seq_len_kv, plan.kv_group, plan.qk_dim)
    for name, buf, shape in (("dq_buffer", dq_buffer, dq_shape), ("dkv_buffer", dkv_buffer, dkv_shape)):
        if buf is not None and (tuple(buf.shape) != shape or buf.dtype != torch.float32):
            raise ValueError(f"{name} must be float32 with shape {shape}; got {buf.dtype} {tuple(buf.shape)}")
    dq = dq_buffer if dq_buffer is not None else torch.empty(dq_shape, dtype=torch.float32, device=q_fp8.device)
    dkv = dkv_buffer if dkv_buffer is not None else torch.empty(dkv_shape, dtype=torch.float32, device=q_fp8.device)
    try:
        ops.sparse_mla_backward(q_fp8, kv_fp8, d_out.contiguous(), indices, sm_scale=float(sm_scale), d_v=plan.d_v, dq=dq, dkv=dkv,
                                clear_dkv=True, q_scale=q_scale, kv_scale=kv_scale)
    except (_lib.NativeCallError, _lib.NativeLibraryError) as exc:
        raise SparseMLAFp8PathCDirectError(f"FP8 sparse-MLA backward dispatch failed: {type(exc).__name__}: {exc}") from exc
    return dq, dkv


class _PreparedFloatFunction(torch.autograd.Function):
    """Forward over prepared FP8 buffers; the cotangent goes back to the float producers."""

    @staticmethod
    def forward(ctx, q, kv, q_fp8, q_scale, kv_fp8, kv_scale, indices, sm_scale, d_v, sinks, output_dtype):
        out = sparse_mla_fp8_path_c_apply(q_fp8, q_scale, kv_fp8, kv_scale, indices, sm_scale=sm_scale, d_v=d_v, sinks=sinks,
                                          force_path_c=True, output_dtype=_float_dtype(q.dtype if output_dtype is None else output_dtype,
                                                                                       name="output_dtype"))
        ctx.save_for_backward(q_fp8, q_scale, kv_fp8, kv_scale, indices)
        ctx.meta = (float(sm_scale), d_v, sinks is not None, q.dtype, kv.dtype)
        return out

    @staticmethod
    def backward(ctx, d_out):
        q_fp8, q_scale, kv_fp8, kv_scale, indices = ctx.saved_tensors
        sm_scale, d_v, has_sinks, q_dtype, kv_dtype = ctx.meta
        if has_sinks:
            raise RuntimeError("sparse_mla_fp8_path_c_apply_prepared_float: sinks backward is not implemented")
        dq, dkv = sparse_mla_fp8_bwd_path_c(q_fp8, q_scale, kv_fp8, kv_scale, d_out, indices, sm_scale=sm_scale, d_v=d_v,
                                            force_path_c=True)
        return (dq.to(q_dtype), dkv.to(kv_dtype)) + (None,) * 9


def sparse_mla_fp8_path_c_apply_prepared_float(
    q: torch.Tensor,
    kv: torch.Tensor,
    q_fp8: torch.Tensor,
    q_scale: torch.Tensor,
    kv_fp8: torch.Tensor,
    kv_scale: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float,
    d_v: int | None = None,
    sinks: torch.Tensor | None = None,
    force_path_c: bool = False,
    causal: bool = False,
    output_dtype: torch.dtype | None = None,
) -> torch.Tensor:
    """Differentiable owner wrapper: the forward reads only the prepared ``q_fp8 / q_scale /
    kv_fp8 / kv_scale``; the backward kernel's gradients (with respect to the dequantised values)
    are handed to the float ``q`` / ``kv`` they were quantised from, in their dtypes.  There is no
    float fallback here: without the library the call raises."""
    del force_path_c, causal
    status = sparse_mla_fp8_path_c_status()
    if not status.available:
        raise RuntimeError(f"sparse_mla_fp8_path_c_apply_prepared_float: Path C forward unavailable: {status.reason}")
    return _PreparedFloatFunction.apply(q, kv, q_fp8, q_scale, kv_fp8, kv_scale, indices, sm_scale, d_v, sinks, output_dtype)


def sparse_mla_fp8_path_c_apply_from_float(q, kv, indices, *, sm_scale, d_v=None, sinks=None, force_path_c=False):
    """Fail-closed hook for float q / kv callers: the FP8 ABI is prepared-buffer only."""
    del q, kv, indices, sm_scale, d_v, sinks, force_path_c
    raise RuntimeError(
        "sparse_mla_fp8_path_c_apply_from_float requires prepared FP8 buffers; use "
        "sparse_mla_fp8_path_c_apply_prepared_float with existing q_fp8/q_scale/kv_fp8/kv_scale buffers instead of "
        "materializing them inside the Path C wrapper")


# invalid slots of the score-only kernels hold this finite sentinel
# (reference sparse_mla_fp8_path_c.py:80)
_SMFP8_INVALID_SCORE_SENTINEL = -3.4028234663852886e38


def fp8_sparse_mla_qk_reduce_path_c(A_fp8, A_scale, B_fp8, B_scale, *, outputs_per_block=None, reduce_threads=None,
                                    vec=None):
    """``(1, N)`` float32 scores ``(dec(B) . dec(A)) * A_scale * B_scale`` for one query row
    ``A_fp8 u8[1,K]`` against ``B_fp8 u8[N,K]`` (reference :1548-1608; validation :1419-1462).
    ``A_scale`` holds one float32, ``B_scale`` one or N.  Returns ``None`` when no gfx950
    device is usable.  The schedule keywords are accepted and ignored."""
    if A_fp8.ndim != 2 or A_fp8.shape[0] != 1:
        raise ValueError(f"A_fp8 must have shape (1, K); got {tuple(A_fp8.shape)}")
    if B_fp8.ndim != 2:
        raise ValueError(f"B_fp8 must have shape (N, K); got {tuple(B_fp8.shape)}")
    if A_fp8.dtype != torch.uint8 or B_fp8.dtype != torch.uint8:
        raise ValueError(f"A_fp8/B_fp8 must be uint8 e4m3 storage; got {A_fp8.dtype}, {B_fp8.dtype}")
    n, k = int(B_fp8.shape[0]), int(A_fp8.shape[1])
    if n <= 0 or k <= 0 or int(B_fp8.shape[1]) != k:
        raise ValueError(f"A_fp8/B_fp8 shape mismatch: A={tuple(A_fp8.shape)}, B={tuple(B_fp8.shape)}")
    if A_scale.numel() != 1:
        raise ValueError(f"A_scale must contain exactly one FP32 scale; got shape {tuple(A_scale.shape)}")
    if B_scale.numel() not in (1, n):
        raise ValueError(f"B_scale must contain one scalar scale or N={n} row scales; got shape {tuple(B_scale.shape)}")
    if A_scale.dtype != torch.float32 or B_scale.dtype != torch.float32:
        raise TypeError(f"A_scale/B_scale must be float32; got {A_scale.dtype}, {B_scale.dtype}")
    if not sparse_mla_fp8_path_c_status().available:
        return None
    out = torch.empty((1, n), dtype=torch.float32, device=A_fp8.device)
    kind = _lib.WSCALE_SCALAR if B_scale.numel() == 1 else _lib.WSCALE_PER_ROW
    ops.fp8_vecmat(A_fp8, B_fp8, B_scale.reshape(-1), out=out, scale_x=A_scale.reshape(1), scale_w_kind=kind)
    return out


def fp8_sparse_mla_indexed_qk_reduce_path_c(q_fp8, q_scale, kv_fp8, kv_scale, indices, *, sm_scale,
                                            outputs_per_block=None, reduce_threads=None, vec=None):
    """``scores[B,S,H,TOPK]`` float32 of the per-token-scaled FP8 layout (reference :1611-1690;
    validation :1465-1545): ``sm_scale * q_scale * kv_scale * (dec(q) . dec(kv[index]))``; a slot
    whose index is negative or >= S_kv holds the finite sentinel -3.4028234663852886e38.
    Returns ``None`` when no gfx950 device is usable."""
    plan = _prepared.plan_prepared(q_fp8, q_scale, kv_fp8, kv_scale, indices, d_v=None, kv_rope=None,
                                   op_name="FP8 Sparse-MLA indexed QK reducer", family="fp8")
    if q_fp8.dtype != torch.uint8:
        raise ValueError(f"q_fp8/kv_fp8 must be uint8 e4m3 storage; got {q_fp8.dtype}, {kv_fp8.dtype}")
    if not sparse_mla_fp8_path_c_status().available:
        return None
    scores = torch.empty((plan.batch, plan.seq_len, plan.heads, int(indices.shape[-1])), dtype=torch.float32,
                         device=q_fp8.device)
    return ops.sparse_mla_scores(q_fp8, kv_fp8, indices, sm_scale=float(sm_scale), scores=scores,
                                 q_spec=plan.q_spec, kv_spec=plan.kv_spec)
