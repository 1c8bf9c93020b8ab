"""Float-carrier MXFP8 block-scaled sparse MLA: quantise, dequantise, attend.

Surface of the reference's ``cppmega_mlx/nn/_tilelang/sparse_mla_blockscaled.py``:
``MXFP8_BLOCK_SIZE`` :39, ``_quantize_mxfp8`` :60-76, ``_dequantize_mxfp8`` :79-87,
``_unpack_mxfp8_to_uint8`` :106-122, ``sparse_mla_blockscaled_reference`` :186-212 (round
trip of q and kv through e4m3 with one E8M0 scale per 32 channels, back to the carrier
dtype, then the plain sparse attention; a width not divisible by 32 skips the round
trip) and ``sparse_mla_blockscaled_apply`` :246-273.

The packed form is four e4m3 bytes per uint32, byte 0 in the low bits.  The scale byte of
the reference's quantiser (``mx.quantize(mode="mxfp8")``) is
byte = clamp(127 + rint(log2(amax / 448)), 1, 254) with codes saturating at +-448: the rule
that reproduces the reference's seeded receipt
``bench/tilelang_ports/sparse_mla_blockscaled.json`` (``parity.blockscaled_vs_bf16``).
"""

from __future__ import annotations

from typing import Tuple

import torch

from ... import ops
from ..sparse_mla import _resolve_shapes, sparse_mla_attention_reference

__all__ = [
    "MXFP8_BLOCK_SIZE",
    "sparse_mla_blockscaled_apply",
    "sparse_mla_blockscaled_reference",
]

MXFP8_BLOCK_SIZE = 32


def _quantize_mxfp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(packed int32 [..., K/4] holding four e4m3 bytes each, E8M0 scales uint8 [..., K/32])."""
    if x.ndim >= 1 and x.numel() == 0:
        last = max(x.shape[-1] // 4, 0)
        return (torch.zeros(tuple(x.shape[:-1]) + (last,), dtype=torch.int32, device=x.device),
                torch.zeros(tuple(x.shape[:-1]) + (max(x.shape[-1] // MXFP8_BLOCK_SIZE, 0),), dtype=torch.uint8, device=x.device))
    if x.shape[-1] % MXFP8_BLOCK_SIZE != 0:
        raise ValueError(f"MXFP8 last dim must be divisible by {MXFP8_BLOCK_SIZE}, got shape {tuple(x.shape)}.")
    xs = x.contiguous()
    codes = torch.empty(xs.shape, dtype=torch.uint8, device=x.device)
    scales = torch.empty(tuple(xs.shape[:-1]) + (xs.shape[-1] // MXFP8_BLOCK_SIZE,), dtype=torch.uint8, device=x.device)
    ops.fp8_quantize(xs, "mxfp8", codes=codes, scale=scales)
    return codes.view(torch.int32), scales


def _unpack_mxfp8_to_uint8(packed: torch.Tensor, last_dim: int) -> torch.Tensor:
    """The flat e4m3 byte view of the packed form."""
    expected_last = packed.shape[-1] * 4
    if expected_last != last_dim:
        raise ValueError(f"_unpack_mxfp8_to_uint8: expected unpacked last_dim={expected_last} to match {last_dim}")
    return packed.view(torch.uint8)


def _dequantize_mxfp8(w_packed: torch.Tensor, scales: torch.Tensor, *, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    codes = w_packed.view(torch.uint8) if w_packed.dtype != torch.uint8 else w_packed
    out = torch.empty(codes.shape, dtype=out_dtype, device=codes.device)
    if codes.numel():
        ops.fp8_dequantize(codes.contiguous(), scales.contiguous(), out=out)
    return out


def _mxfp8_roundtrip(x: torch.Tensor) -> torch.Tensor:
    if x.shape[-1] % MXFP8_BLOCK_SIZE != 0 or x.numel() == 0:
        return x
    xs = x.contiguous()
    rec = torch.empty_like(xs)
    ops.fp8_quantize(xs, "mxfp8", recovered=rec)
    return rec


def sparse_mla_blockscaled_reference(q, kv, indices, *, sm_scale: float | None = None, d_v: int | None = None,
                                     return_lse: bool = False):
    """MXFP8 round trip of q and kv, then the fp32 sparse attention."""
    shapes = _resolve_shapes(q, kv, indices, d_v=d_v)
    if shapes.qk_dim % MXFP8_BLOCK_SIZE != 0:
        return sparse_mla_attention_reference(q, kv, indices, sm_scale=sm_scale, d_v=d_v, return_lse=return_lse)
    return sparse_mla_attention_reference(_mxfp8_roundtrip(q), _mxfp8_roundtrip(kv), indices, sm_scale=sm_scale, d_v=d_v,
                                          return_lse=return_lse)


def sparse_mla_blockscaled_apply(q, kv, indices, *, sm_scale: float | None = None, d_v: int | None = None,
                                 return_lse: bool = False, force_metal: bool = False):
    """Float-carrier block-scaled sparse MLA; ``force_metal`` (the retired direct-MSL surface)
    raises, as in the reference."""
    shapes = _resolve_shapes(q, kv, indices, d_v=d_v)
    if sm_scale is None:
        sm_scale = shapes.qk_dim ** -0.5
    if force_metal:
        raise RuntimeError("sparse_mla_blockscaled_apply: Metal path unavailable: this build runs HIP kernels on gfx950")
    return sparse_mla_blockscaled_reference(q, kv, indices, sm_scale=sm_scale, d_v=d_v, return_lse=return_lse)
