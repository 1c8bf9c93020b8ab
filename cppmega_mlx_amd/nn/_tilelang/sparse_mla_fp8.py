"""Float-carrier FP8 sparse MLA: quantise q and kv per tensor, dequantise, attend.

Surface of the reference's ``cppmega_mlx/nn/_tilelang/sparse_mla_fp8.py``:
``_to_fp8_with_per_tensor_scale`` :123-145, ``_from_fp8_with_scale`` :148-157,
``sparse_mla_fp8_reference`` :489-511 (round trip of q and kv through e4m3 with one
amax scale per tensor, back to the carrier dtype, then the plain sparse attention),
``sparse_mla_quantized_matmul_reference`` :514-563 (the same attention stated with
matmuls) and ``sparse_mla_fp8_apply`` :600-657.  Quantiser, dequantiser and attention
all run as HIP kernels; the Metal-only ``force_metal`` route raises as the reference
does when that path is unavailable.
"""

from __future__ import annotations

from typing import Tuple

import torch

from ... import ops
from ..sparse_mla import _resolve_shapes, sparse_mla_attention_reference

__all__ = [
    "sparse_mla_fp8_apply",
    "sparse_mla_fp8_reference",
    "sparse_mla_quantized_matmul_reference",
]

_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


def _to_fp8_with_per_tensor_scale(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(e4m3 bytes uint8 like x, float32 scale of shape x.shape[:-1]); scale =
    max(amax(x) / 448, 1e-12) for the whole tensor, replicated per row."""
    if x.dtype not in _FLOATS:
        raise TypeError(f"FP8 producer input must be floating, got {x.dtype}")
    scale_shape = tuple(x.shape[:-1]) if x.ndim > 1 else (1,)
    codes = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    scale = torch.ones(scale_shape, dtype=torch.float32, device=x.device)
    if x.numel() == 0:
        return codes.zero_(), scale
    xs = x if x.ndim > 1 else x.reshape(1, -1)
    ops.fp8_quantize(xs.contiguous(), "per_tensor", codes=codes.reshape(xs.shape), scale=scale.reshape(xs.shape[:-1]))
    return codes, scale


def _from_fp8_with_scale(fp8: torch.Tensor, scale: torch.Tensor, *, dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """dec(fp8) * scale[..., None] in ``dtype``."""
    out = torch.empty(fp8.shape, dtype=dtype, device=fp8.device)
    if fp8.numel() == 0:
        return out
    f2 = fp8 if fp8.ndim > 1 else fp8.reshape(1, -1)
    ops.fp8_dequantize(f2.contiguous(), scale.reshape(f2.shape[:-1]).contiguous(), out=out.reshape(f2.shape))
    return out


def _fp8_roundtrip(x: torch.Tensor) -> torch.Tensor:
    """x -> e4m3 with a per-tensor scale -> x.dtype, in one kernel sequence."""
    if x.numel() == 0:
        return x.clone()
    xs = (x if x.ndim > 1 else x.reshape(1, -1)).contiguous()
    rec = torch.empty_like(xs)
    ops.fp8_quantize(xs, "per_tensor", recovered=rec)
    return rec.reshape(x.shape)


def sparse_mla_fp8_reference(q, kv, indices, *, sm_scale: float | None = None, d_v: int | None = None,
                             return_lse: bool = False):
    """FP8 round trip of q and kv, then the fp32 sparse attention."""
    _resolve_shapes(q, kv, indices, d_v=d_v)
    return sparse_mla_attention_reference(_fp8_roundtrip(q), _fp8_roundtrip(kv), indices, sm_scale=sm_scale, d_v=d_v,
                                          return_lse=return_lse)


def sparse_mla_quantized_matmul_reference(q, kv, indices, *, sm_scale: float | None = None, d_v: int | None = None,
                                          return_lse: bool = False):
    """The sparse attention on already-dequantised carriers (the reference spells it with
    matmuls; here it is the same fp32 kernel)."""
    return sparse_mla_attention_reference(q, kv, indices, sm_scale=sm_scale, d_v=d_v, return_lse=return_lse)


def sparse_mla_fp8_apply(q, kv, indices, *, sm_scale: float | None = None, d_v: int | None = None,
                         return_lse: bool = False, force_metal: bool = False):
    """Float-carrier FP8 sparse MLA.  ``force_metal`` asks for the reference's direct-MSL
    path, which does not exist on this device: it raises, like the reference when Metal is
    unavailable."""
    shapes = _resolve_shapes(q, kv, indices, d_v=d_v)
    if sm_scale is None:
        sm_scale = shapes.qk_dim ** -0.5
    if force_metal:
        raise RuntimeError("sparse_mla_fp8_apply: Metal path unavailable: this build runs HIP kernels on gfx950")
    return sparse_mla_fp8_reference(q, kv, indices, sm_scale=sm_scale, d_v=d_v, return_lse=return_lse)
