"""Block-scaled FP8 sparse-MLA forward over prepared buffers.

Surface of the reference's
``cppmega_mlx/nn/_tilelang/sparse_mla_blockscaled_path_c.py``:
``sparse_mla_blockscaled_path_c_apply_direct`` :1298-1388 and
``sparse_mla_blockscaled_path_c_apply`` :1391-1504 with the kernel contract of
:1054-1164 (invalid index <=> ``idx < 0 or idx >= Skv``; ``lse`` natural log,
0 when nothing is attended).

Two storage layouts are accepted, told apart by the scale tensors:

* reference (MXFP8): ``q_fp8``/``kv_fp8`` uint8 e4m3 ``[.., K]`` with uint8
  E8M0 scales per 32 channels ``[.., K/32]`` on both operands;
* latent KV cache: ``kv_fp8`` uint8 e4m3 ``[B,Skv,G,Kl]`` with **float32**
  scales per 128 latent channels ``[B,Skv,G,Kl/128]``, ``kv_rope=`` a bf16
  ``[B,Skv,G,R]`` tail that joins QK only, and a bf16 (or fp16/fp32) query
  ``[B,S,H,Kl+R]`` passed in the ``q_fp8`` slot with ``q_scale=None``.

``out`` may be float16 (the reference's dtype), bfloat16 or float32.  Without
``out``/``lse`` the result tensors are allocated here: float16 for an FP8
query, the query dtype otherwise.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ... import _lib, ops
from . import _prepared

__all__ = [
    "E8M0_BLOCK_SIZE",
    "SparseMLABlockScaledPathCDirectError",
    "SparseMLABlockScaledPathCStatus",
    "sparse_mla_blockscaled_path_c_apply",
    "sparse_mla_blockscaled_path_c_apply_direct",
    "sparse_mla_blockscaled_path_c_status",
    "blockscaled_sparse_mla_qk_reduce_path_c",
]

E8M0_BLOCK_SIZE = _prepared.E8M0_BLOCK_SIZE
_OP = "blockscaled Sparse-MLA Path C apply"


class SparseMLABlockScaledPathCDirectError(RuntimeError):
    """Raised when the prepared-buffer owner-output path cannot run."""


@dataclass(frozen=True)
class SparseMLABlockScaledPathCStatus:
    available: bool
    reason: str
    scale_block_size: int = E8M0_BLOCK_SIZE
    target: str = "hip-gfx950"


def sparse_mla_blockscaled_path_c_status() -> SparseMLABlockScaledPathCStatus:
    try:
        st = _lib.status()
    except _lib.NativeLibraryError as exc:
        return SparseMLABlockScaledPathCStatus(False, str(exc))
    if st["gfx950_devices"] < 1:
        return SparseMLABlockScaledPathCStatus(False, st["message"])
    return SparseMLABlockScaledPathCStatus(True, "block-scaled sparse-MLA HIP kernels (gfx950) are available")


def sparse_mla_blockscaled_path_c_apply_direct(
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
    kv_rope: torch.Tensor | None = None,
    kernel: str = "auto",
) -> tuple[torch.Tensor, torch.Tensor]:
    """Forward into caller-owned ``out``/``lse``; returns those same objects."""
    status = sparse_mla_blockscaled_path_c_status()
    if not status.available:
        raise SparseMLABlockScaledPathCDirectError(status.reason)
    plan = _prepared.plan_prepared(q_fp8, q_scale, kv_fp8, kv_scale, indices, d_v=d_v, kv_rope=kv_rope,
                                   op_name=_OP, family="blockscaled")
    _prepared.validate_owner_outputs(out, lse, plan, out_dtype=None)
    try:
        _prepared.launch_prepared(q_fp8, kv_fp8, indices, plan, sm_scale=sm_scale, out=out, lse=lse,
                                  kv_rope=kv_rope, sinks=None, kernel=kernel)
    except (_lib.NativeCallError, _lib.NativeLibraryError) as exc:
        raise SparseMLABlockScaledPathCDirectError(
            f"block-scaled Sparse-MLA forward dispatch failed: {type(exc).__name__}: {exc}"
        ) from exc
    return out, lse


def sparse_mla_blockscaled_path_c_apply(
    q_fp8: torch.Tensor,
    q_scale: torch.Tensor | None,
    kv_fp8: torch.Tensor,
    kv_scale: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float,
    d_v: int | None = None,
    return_lse: bool = False,
    force_path_c: bool = False,
    out: torch.Tensor | None = None,
    lse: torch.Tensor | None = None,
    kv_rope: torch.Tensor | None = None,
    kernel: str = "auto",
):
    """Fused block-scaled sparse-MLA forward over prepared GPU buffers."""
    if (out is None) != (lse is None):
        raise ValueError(
            "sparse_mla_blockscaled_path_c_apply owner-output route requires both out and lse buffers"
        )
    if out is not None and lse is not None:
        direct_out, direct_lse = sparse_mla_blockscaled_path_c_apply_direct(
            q_fp8, q_scale, kv_fp8, kv_scale, indices, sm_scale=sm_scale, out=out, lse=lse, d_v=d_v,
            kv_rope=kv_rope, kernel=kernel)
        return (direct_out, direct_lse) if return_lse else direct_out

    status = sparse_mla_blockscaled_path_c_status()
    if not status.available:
        if force_path_c:
            raise RuntimeError(f"sparse_mla_blockscaled_path_c_apply: {status.reason}")
        return None
    plan = _prepared.plan_prepared(q_fp8, q_scale, kv_fp8, kv_scale, indices, d_v=d_v, kv_rope=kv_rope,
                                   op_name=_OP, family="blockscaled")
    out_dtype = torch.float16 if q_fp8.dtype == torch.uint8 else q_fp8.dtype
    out = torch.empty((plan.batch, plan.seq_len, plan.heads, plan.d_v), dtype=out_dtype, device=q_fp8.device)
    lse = torch.empty((plan.batch, plan.seq_len, plan.heads), dtype=torch.float32, device=q_fp8.device)
    try:
        _prepared.launch_prepared(q_fp8, kv_fp8, indices, plan, sm_scale=sm_scale, out=out, lse=lse,
                                  kv_rope=kv_rope, sinks=None, kernel=kernel)
    except (_lib.NativeCallError, _lib.NativeLibraryError) as exc:
        raise RuntimeError(
            f"sparse_mla_blockscaled_path_c_apply: kernel dispatch failed: {type(exc).__name__}: {exc}"
        ) from exc
    return (out, lse) if return_lse else out


E8M0_BLOCK_SIZE = 32


def blockscaled_sparse_mla_qk_reduce_path_c(A_fp8, A_scale, B_fp8, B_scale, *, outputs_per_block: int = 4,
                                            reduce_threads: int = 32, vec: int = 4):
    """``(1, N)`` float32 scores of one E8M0 block-scaled query row ``A_fp8 u8[1,K]`` (scales
    ``u8[K/32]``) against ``B_fp8 u8[N,K]`` (scales ``u8[K/32]`` broadcast or ``u8[N,K/32]``):
    reference ``sparse_mla_blockscaled_path_c.py:883-932``, validation ``:820-880``.
    Returns ``None`` when no gfx950 device is usable.  The schedule keywords are ignored."""
    if A_fp8.ndim != 2 or A_fp8.shape[0] != 1:
        raise ValueError(f"A_fp8 must have shape (1, K); got {tuple(A_fp8.shape)}")
    if B_fp8.ndim != 2:
        raise ValueError(f"B_fp8 must have shape (N, K); got {tuple(B_fp8.shape)}")
    if A_fp8.dtype != torch.uint8 or B_fp8.dtype != torch.uint8:
        raise ValueError(f"A_fp8/B_fp8 must be uint8 e4m3 storage; got {A_fp8.dtype}, {B_fp8.dtype}")
    if A_scale.dtype != torch.uint8 or B_scale.dtype != torch.uint8:
        raise TypeError(f"A_scale/B_scale must be uint8 E8M0 storage; got {A_scale.dtype}, {B_scale.dtype}")
    n, k = int(B_fp8.shape[0]), int(A_fp8.shape[1])
    if n <= 0 or k <= 0 or int(B_fp8.shape[1]) != k:
        raise ValueError(f"A_fp8/B_fp8 shape mismatch: A={tuple(A_fp8.shape)}, B={tuple(B_fp8.shape)}")
    if k % E8M0_BLOCK_SIZE != 0:
        raise ValueError(f"E8M0 QK reducer requires K divisible by {E8M0_BLOCK_SIZE}; got K={k}")
    blocks = k // E8M0_BLOCK_SIZE
    if A_scale.numel() != blocks:
        raise ValueError(f"A_scale must contain K/{E8M0_BLOCK_SIZE}={blocks} E8M0 bytes; got shape {tuple(A_scale.shape)}")
    if B_scale.numel() not in (blocks, n * blocks):
        raise ValueError(
            f"B_scale must contain K/{E8M0_BLOCK_SIZE}={blocks} broadcast bytes or N*K/{E8M0_BLOCK_SIZE}={n * blocks} "
            f"row-block bytes; got shape {tuple(B_scale.shape)}")
    if not sparse_mla_blockscaled_path_c_status().available:
        return None
    # one query, one head, N keys in order: the score-only attention kernel with identity indices
    b_rows = B_scale.reshape(1, blocks).expand(n, blocks).contiguous() if B_scale.numel() == blocks else B_scale.reshape(n, blocks)
    q = A_fp8.reshape(1, 1, 1, k)
    kv = B_fp8.reshape(1, n, 1, k)
    idx = torch.arange(n, dtype=torch.int32, device=A_fp8.device).reshape(1, 1, 1, n)
    scores = torch.empty((1, 1, 1, n), dtype=torch.float32, device=A_fp8.device)
    ops.sparse_mla_scores(q, kv, idx, sm_scale=1.0, scores=scores,
                          q_spec=ops.QuantSpec(_lib.SCALE_E8M0, A_scale.reshape(1, 1, 1, blocks), E8M0_BLOCK_SIZE),
                          kv_spec=ops.QuantSpec(_lib.SCALE_E8M0, b_rows.reshape(1, n, 1, blocks), E8M0_BLOCK_SIZE))
    return scores.reshape(1, n)
