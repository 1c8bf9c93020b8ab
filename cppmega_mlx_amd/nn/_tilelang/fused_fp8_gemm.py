"""Block-128 FP8 weight GEMV/GEMM: ``out = a @ dequant(W).T``.

Contract of the reference's ``cppmega_v4/_tilelang/fused_fp8_gemm.py:34-146``
(operator caller ``FP8Linear.__call__``, cppmega_v4/nn/moe_fp8.py:89-93):
``w_fp8`` uint8 e4m3 ``[M, K]``, ``w_scale_inv`` float32
``[ceil(M/128), ceil(K/128)]``, ``a`` ``[..., K]`` bfloat16/float16/float32;
fp32 accumulation; the result ``[..., M]`` has ``a``'s dtype.  A per-row scale
grid ``[M, ceil(K/128)]`` is accepted as well.  NaN weight bytes (0x7F/0xFF)
are outside the contract of this kernel family and propagate as NaN.
"""

from __future__ import annotations

import torch

from ... import _lib, ops

__all__ = ["fused_fp8_gemm"]

_BLOCK = 128


def fused_fp8_gemm(w_fp8: torch.Tensor, w_scale_inv: torch.Tensor, a: torch.Tensor, *, out: torch.Tensor | None = None) -> torch.Tensor:
    if w_fp8.dtype != torch.uint8:
        raise TypeError(f"w_fp8 must be uint8 (fp8 storage); got {w_fp8.dtype}")
    if w_fp8.ndim != 2:
        raise ValueError(f"w_fp8 must be 2D [M, K]; got {tuple(w_fp8.shape)}")
    M, K = (int(v) for v in w_fp8.shape)
    if a.shape[-1] != K:
        raise ValueError(f"a.shape[-1] ({a.shape[-1]}) must equal w_fp8.shape[1] ({K})")
    blocks_m = (M + _BLOCK - 1) // _BLOCK
    blocks_k = (K + _BLOCK - 1) // _BLOCK
    if tuple(w_scale_inv.shape) == (blocks_m, blocks_k):
        kind = _lib.WSCALE_GRID_128
    elif tuple(w_scale_inv.shape) == (M, blocks_k):
        kind = _lib.WSCALE_ROW_BLOCK
    else:
        raise ValueError(
            f"w_scale_inv shape {tuple(w_scale_inv.shape)} != expected ({blocks_m}, {blocks_k}) "
            f"for W={M, K} with block={_BLOCK}"
        )
    if w_scale_inv.dtype != torch.float32:
        raise TypeError(f"w_scale_inv must be float32; got {w_scale_inv.dtype}")
    if a.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise TypeError(f"a must be bfloat16, float16 or float32; got {a.dtype}")
    leading = tuple(a.shape[:-1])
    rows = 1
    for d in leading:
        rows *= int(d)
    a2 = a.reshape(rows, K)
    if out is None:
        out = torch.empty((*leading, M), dtype=a.dtype, device=a.device)
    elif tuple(out.shape) != (*leading, M):
        raise ValueError(f"out must have shape {(*leading, M)}; got {tuple(out.shape)}")
    if rows == 0:
        return out
    ops.fp8_vecmat(a2, w_fp8, w_scale_inv, out=out.reshape(rows, M), scale_x=None, scale_w_kind=kind)
    return out
