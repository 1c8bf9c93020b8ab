"""Shared validation + launch for the prepared-buffer sparse-MLA entry points.

The checks and their messages follow the reference's
``_validate_blockscaled_apply_inputs``
(sparse_mla_blockscaled_path_c.py:943-1005) and ``_validate_fp8_apply_inputs``
(sparse_mla_fp8_path_c.py:1701-1772); the block-128 latent layout (fp32 scale
per 128 latent channels + bf16 rope tail, bf16 query) is the keyword-only
extension both entry points accept.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ... import _lib, ops

E8M0_BLOCK_SIZE = 32
LATENT_BLOCK_SIZE = 128
_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


@dataclass(frozen=True)
class PreparedPlan:
    batch: int
    seq_len: int
    heads: int
    seq_len_kv: int
    kv_group: int
    topk: int
    qk_dim: int
    d_v: int
    q_spec: ops.QuantSpec
    kv_spec: ops.QuantSpec
    layout: str  # "e8m0", "per_token" or "latent128"


def index_dtype_name(indices: torch.Tensor, *, op_name: str) -> str:
    if indices.dtype == torch.int32:
        return "int32"
    if indices.dtype == torch.int64:
        return "int64"
    raise TypeError(
        f"{op_name} requires torch.int32 or torch.int64 indices; got {indices.dtype}. "
        "The kernel boundary will not cast or copy sparse index tensors."
    )


def plan_prepared(q, q_scale, kv, kv_scale, indices, *, d_v, kv_rope, op_name: str, family: str) -> PreparedPlan:
    """Classify the call by the dtypes/shapes of its scales and validate it.

    family "blockscaled": uint8 scales are E8M0 per 32 on q and kv (reference);
        float32 ``kv_scale`` of rank 4 is the fp32-per-128 latent layout.
    family "fp8": float32 rank-3 scales are per-token (reference); a float32
        rank-4 ``kv_scale`` is again the latent layout.
    """
    if q.ndim != 4:
        raise ValueError(f"q_fp8 must have shape (B, S, H, K); got {tuple(q.shape)}")
    if kv.ndim != 4:
        raise ValueError(f"kv_fp8 must have shape (B, S_kv, G, K); got {tuple(kv.shape)}")
    if indices.ndim != 4:
        raise ValueError(f"indices must have shape (B, S, G, TOPK); got {tuple(indices.shape)}")
    if kv.dtype != torch.uint8:
        raise TypeError(f"q_fp8/kv_fp8 must be uint8 FP8 storage; got {q.dtype}, {kv.dtype}")
    index_dtype_name(indices, op_name=op_name)

    batch, seq_len, heads, qk_dim = (int(x) for x in q.shape)
    kv_batch, seq_len_kv, kv_group, kv_dim = (int(x) for x in kv.shape)
    idx_batch, idx_seq, idx_group, topk = (int(x) for x in indices.shape)
    if kv_batch != batch or idx_batch != batch or idx_seq != seq_len:
        raise ValueError(
            "q_fp8/kv_fp8/indices batch or sequence mismatch: "
            f"q={tuple(q.shape)} kv={tuple(kv.shape)} indices={tuple(indices.shape)}"
        )
    if idx_group != kv_group:
        raise ValueError(f"indices kv_group mismatch: indices={tuple(indices.shape)} kv={tuple(kv.shape)}")
    if heads % kv_group != 0:
        raise ValueError(f"heads {heads} must be divisible by kv_group {kv_group}")

    latent = isinstance(kv_scale, torch.Tensor) and kv_scale.dtype == torch.float32 and kv_scale.ndim == 4
    if latent:
        rope_dim = 0 if kv_rope is None else int(kv_rope.shape[-1])
        if kv_rope is not None:
            if kv_rope.dtype not in _FLOATS or tuple(kv_rope.shape[:3]) != (batch, seq_len_kv, kv_group):
                raise ValueError(
                    f"kv_rope must be float [{batch}, {seq_len_kv}, {kv_group}, R]; got {kv_rope.dtype} {tuple(kv_rope.shape)}"
                )
        if kv_dim + rope_dim != qk_dim:
            raise ValueError(f"q width {qk_dim} != latent width {kv_dim} + rope width {rope_dim}")
        blocks = int(kv_scale.shape[-1])
        if blocks < 1 or kv_dim % blocks != 0:
            raise ValueError(f"kv_scale last dim {blocks} does not divide the latent width {kv_dim}")
        if tuple(kv_scale.shape) != (batch, seq_len_kv, kv_group, blocks):
            raise ValueError(
                f"kv_scale must have shape {(batch, seq_len_kv, kv_group, blocks)}; got {tuple(kv_scale.shape)}"
            )
        if q.dtype in _FLOATS:
            if q_scale is not None:
                raise ValueError("a float query takes q_scale=None")
            q_spec = ops.QuantSpec()
        elif q.dtype == torch.uint8:
            if not isinstance(q_scale, torch.Tensor) or q_scale.dtype != torch.float32 or tuple(q_scale.shape) != (batch, seq_len, heads):
                raise ValueError(f"an FP8 query in the latent layout takes a float32 per-token q_scale {(batch, seq_len, heads)}")
            q_spec = ops.QuantSpec(_lib.SCALE_PER_TOKEN, q_scale)
        else:
            raise TypeError(f"q must be bfloat16/float16/float32 or uint8 FP8 storage; got {q.dtype}")
        d_v_resolved = kv_dim if d_v is None else int(d_v)
        if d_v_resolved <= 0 or d_v_resolved > kv_dim:
            raise ValueError(f"d_v must be in (0, {kv_dim}], got {d_v_resolved}")
        kv_spec = ops.QuantSpec(_lib.SCALE_F32_BLOCK, kv_scale, kv_dim // blocks)
        return PreparedPlan(batch, seq_len, heads, seq_len_kv, kv_group, topk, qk_dim, d_v_resolved, q_spec, kv_spec,
                            "latent128")

    if kv_rope is not None:
        raise ValueError("kv_rope is only defined for the float32 block-scaled latent layout")
    if q.dtype != torch.uint8:
        raise TypeError(f"q_fp8/kv_fp8 must be uint8 FP8 storage; got {q.dtype}, {kv.dtype}")
    if kv_dim != qk_dim:
        raise ValueError(f"q_fp8/kv_fp8 K mismatch: q={tuple(q.shape)} kv={tuple(kv.shape)}")
    d_v_resolved = qk_dim if d_v is None else int(d_v)

    if family == "blockscaled":
        if not isinstance(q_scale, torch.Tensor) or not isinstance(kv_scale, torch.Tensor) or \
                q_scale.dtype != torch.uint8 or kv_scale.dtype != torch.uint8:
            got = tuple(getattr(s, "dtype", type(s).__name__) for s in (q_scale, kv_scale))
            raise TypeError(f"q_scale/kv_scale must be uint8 E8M0 scales; got {got[0]}, {got[1]}")
        if qk_dim % E8M0_BLOCK_SIZE != 0:
            raise ValueError(f"blockscaled Path C requires K divisible by {E8M0_BLOCK_SIZE}; got {qk_dim}")
        scale_blocks = qk_dim // E8M0_BLOCK_SIZE
        if tuple(q_scale.shape) != (batch, seq_len, heads, scale_blocks):
            raise ValueError(f"q_scale must have shape {(batch, seq_len, heads, scale_blocks)}; got {tuple(q_scale.shape)}")
        if tuple(kv_scale.shape) != (batch, seq_len_kv, kv_group, scale_blocks):
            raise ValueError(
                f"kv_scale must have shape {(batch, seq_len_kv, kv_group, scale_blocks)}; got {tuple(kv_scale.shape)}"
            )
        if d_v_resolved <= 0 or d_v_resolved > qk_dim:
            raise ValueError(f"d_v must be in (0, {qk_dim}], got {d_v_resolved}")
        return PreparedPlan(batch, seq_len, heads, seq_len_kv, kv_group, topk, qk_dim, d_v_resolved,
                            ops.QuantSpec(_lib.SCALE_E8M0, q_scale, E8M0_BLOCK_SIZE),
                            ops.QuantSpec(_lib.SCALE_E8M0, kv_scale, E8M0_BLOCK_SIZE), "e8m0")

    if not isinstance(q_scale, torch.Tensor) or not isinstance(kv_scale, torch.Tensor) or \
            q_scale.dtype != torch.float32 or kv_scale.dtype != torch.float32:
        got = tuple(getattr(s, "dtype", type(s).__name__) for s in (q_scale, kv_scale))
        raise TypeError(f"q_scale/kv_scale must be float32; got {got[0]}, {got[1]}")
    if tuple(q_scale.shape) != (batch, seq_len, heads):
        raise ValueError(f"q_scale must have shape {(batch, seq_len, heads)}; got {tuple(q_scale.shape)}")
    if tuple(kv_scale.shape) != (batch, seq_len_kv, kv_group):
        raise ValueError(f"kv_scale must have shape {(batch, seq_len_kv, kv_group)}; got {tuple(kv_scale.shape)}")
    if d_v_resolved <= 0 or d_v_resolved > qk_dim:
        raise ValueError(f"d_v must be in (0, {qk_dim}], got {d_v_resolved}")
    return PreparedPlan(batch, seq_len, heads, seq_len_kv, kv_group, topk, qk_dim, d_v_resolved,
                        ops.QuantSpec(_lib.SCALE_PER_TOKEN, q_scale), ops.QuantSpec(_lib.SCALE_PER_TOKEN, kv_scale),
                        "per_token")


def validate_owner_outputs(out, lse, plan: PreparedPlan, *, out_dtype: torch.dtype | None) -> None:
    if not isinstance(out, torch.Tensor):
        raise TypeError(f"out must be a torch.Tensor; got {type(out).__name__}")
    if not isinstance(lse, torch.Tensor):
        raise TypeError(f"lse must be a torch.Tensor; got {type(lse).__name__}")
    want_out = (plan.batch, plan.seq_len, plan.heads, plan.d_v)
    want_lse = (plan.batch, plan.seq_len, plan.heads)
    if tuple(out.shape) != want_out:
        raise ValueError(f"out must have shape {want_out}; got {tuple(out.shape)}")
    if tuple(lse.shape) != want_lse:
        raise ValueError(f"lse must have shape {want_lse}; got {tuple(lse.shape)}")
    if out_dtype is not None and out.dtype != out_dtype:
        raise TypeError(f"out must be {out_dtype}; got {out.dtype}")
    if out.dtype not in _FLOATS:
        raise TypeError(f"out must be float32, float16, or bfloat16; got {out.dtype}")
    if lse.dtype != torch.float32:
        raise TypeError(f"lse must be torch.float32; got {lse.dtype}")


def launch_prepared(q, kv, indices, plan: PreparedPlan, *, sm_scale, out, lse, kv_rope, sinks, kernel="auto"):
    return ops.sparse_mla_forward(
        q, kv, indices, sm_scale=float(sm_scale), d_v=plan.d_v, out=out, lse=lse,
        q_spec=plan.q_spec, kv_spec=plan.kv_spec, kv_rope=kv_rope, sinks=sinks, kernel=kernel,
    )
