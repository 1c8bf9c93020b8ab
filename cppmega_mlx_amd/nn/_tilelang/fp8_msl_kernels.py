"""FP8 scaled vecmat with the reference's Path B names.

``fp8_scaled_vecmat(x_fp8, W_fp8, *, scale_x, scale_w)`` follows the contract of
the reference's ``cppmega_mlx/nn/_tilelang/fp8_msl_kernels.py:145-180``:
``x_fp8`` uint8 e4m3 ``(K,)``, ``W_fp8`` uint8 e4m3 ``(N, K)`` (already
transposed), ``scale_x`` scalar, ``scale_w`` scalar or ``(N,)``; the result is
float32 ``(N,)`` = ``(dec(W) @ dec(x)) * scale_x * scale_w``.  It allocates its
result (as the reference does) and runs the HIP GEMV kernel.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import torch

from ... import _lib, ops

__all__ = ["FP8MSLKernelStatus", "fp8_msl_status", "fp8_scaled_vecmat", "fp8_to_half", "half_to_fp8"]


@dataclass(frozen=True)
class FP8MSLKernelStatus:
    available: bool
    reason: str


def fp8_msl_status() -> FP8MSLKernelStatus:
    return FP8MSLKernelStatus(False, "direct-MSL FP8 kernels are retired; the HIP GEMV serves fp8_scaled_vecmat")


def _check_dtype(name: str, arr: torch.Tensor, expected: torch.dtype) -> None:
    if arr.dtype != expected:
        raise TypeError(f"fp8_msl_kernels.{name}: expected dtype {expected}, got {arr.dtype}")


def fp8_to_half(fp8_uchar: torch.Tensor) -> torch.Tensor:
    """uint8 e4m3fn storage -> float16 (cppmega_mlx/nn/_tilelang/fp8_msl_kernels.py:65-71).  Allocates
    its result, as the reference does."""
    _check_dtype("fp8_to_half", fp8_uchar, torch.uint8)
    out = torch.zeros(fp8_uchar.shape, dtype=torch.float16, device=fp8_uchar.device)
    if fp8_uchar.numel() == 0:
        return out
    return ops.e4m3_convert(fp8_uchar.contiguous(), out=out)


def half_to_fp8(half_arr: torch.Tensor) -> torch.Tensor:
    """float16 -> e4m3fn bytes, round to nearest even, saturating at +-448
    (cppmega_mlx/nn/_tilelang/fp8_msl_kernels.py:74-81)."""
    _check_dtype("half_to_fp8", half_arr, torch.float16)
    out = torch.zeros(half_arr.shape, dtype=torch.uint8, device=half_arr.device)
    if half_arr.numel() == 0:
        return out
    return ops.e4m3_convert(half_arr.contiguous(), out=out)


def _resolve_scale(scale, *, length: int, name: str, device) -> Tuple[torch.Tensor, int]:
    """Normalise ``scale`` to a 1-D float32 device tensor; mode 0 = scalar, 1 = per channel."""
    if isinstance(scale, (int, float)):
        return torch.tensor([float(scale)], dtype=torch.float32, device=device), 0
    if scale.numel() == 1:
        return scale.reshape(1).to(torch.float32), 0
    if scale.numel() == length:
        return scale.reshape(length).to(torch.float32), 1
    raise ValueError(
        f"fp8_msl_kernels: expected {name} to have size 1 (per-tensor) or {length} (per-channel), "
        f"got size {scale.numel()}"
    )


def fp8_scaled_vecmat(x_fp8: torch.Tensor, W_fp8: torch.Tensor, *, scale_x, scale_w) -> torch.Tensor:
    _check_dtype("fp8_scaled_vecmat[x]", x_fp8, torch.uint8)
    _check_dtype("fp8_scaled_vecmat[W]", W_fp8, torch.uint8)
    if x_fp8.ndim != 1 or W_fp8.ndim != 2:
        raise ValueError(f"fp8_scaled_vecmat expects 1D x and 2D W; got x.ndim={x_fp8.ndim}, W.ndim={W_fp8.ndim}")
    (K,) = x_fp8.shape
    N, K_w = W_fp8.shape
    if K != K_w:
        raise ValueError(f"fp8_scaled_vecmat shape mismatch: x is (K={K},), W is (N={N}, K={K_w})")
    if K % 4 != 0:
        raise ValueError(f"fp8_scaled_vecmat: K must be a multiple of 4 (packed dot4 contract); got K={K}")
    sx, _ = _resolve_scale(scale_x, length=1, name="scale_x", device=W_fp8.device)
    sw, mode = _resolve_scale(scale_w, length=N, name="scale_w", device=W_fp8.device)
    out = torch.empty((N,), dtype=torch.float32, device=W_fp8.device)
    ops.fp8_vecmat(x_fp8, W_fp8, sw, out=out, scale_x=sx,
                   scale_w_kind=_lib.WSCALE_PER_ROW if mode == 1 else _lib.WSCALE_SCALAR)
    return out
