"""FP8 vecmat / block-scaled GEMV oracle.  TEST INFRASTRUCTURE ONLY.

  * ``fp8_scaled_vecmat_oracle`` restates ``fp8_scaled_vecmat``
    (cppmega_mlx/nn/_tilelang/fp8_msl_kernels.py:145-180):
    out[n] = (sum_k dec(W[n,k]) * dec(x[k])) * scale_x * scale_w[n or 0].
  * ``fused_fp8_gemm_oracle`` restates ``fused_fp8_gemm``
    (cppmega_v4/_tilelang/fused_fp8_gemm.py:34-146):
    out[row, n] = sum_k dec(W[n,k]) * scale[n // bn, k // 128] * a[row, k]
    with fp32-or-better accumulation, cast to the activation dtype by the
    caller.  ``scale`` may be the reference's [ceil(N/128), ceil(K/128)] grid or
    the finer [N, ceil(K/128)] (one scale per row and 128-wide K block), of
    which the grid is the special case of 128 identical rows.
Arithmetic is float64.
"""

from __future__ import annotations

import numpy as np

from . import fp8


def fp8_scaled_vecmat_oracle(x_codes, w_codes, *, scale_x, scale_w) -> np.ndarray:
    x_codes = np.asarray(x_codes)
    w_codes = np.asarray(w_codes)
    if x_codes.ndim != 1 or w_codes.ndim != 2:
        raise ValueError(
            f"fp8_scaled_vecmat expects 1D x and 2D W; got x.ndim={x_codes.ndim}, W.ndim={w_codes.ndim}")
    (K,) = x_codes.shape
    N, Kw = w_codes.shape
    if K != Kw:
        raise ValueError(f"fp8_scaled_vecmat shape mismatch: x is (K={K},), W is (N={N}, K={Kw})")
    if K % 4:
        raise ValueError(f"fp8_scaled_vecmat: K must be a multiple of 4; got K={K}")
    sx = np.asarray(scale_x, dtype=np.float64).reshape(-1)
    sw = np.asarray(scale_w, dtype=np.float64).reshape(-1)
    if sx.size != 1:
        raise ValueError(f"expected scale_x to have size 1, got size {sx.size}")
    if sw.size not in (1, N):
        raise ValueError(f"expected scale_w to have size 1 or {N}, got size {sw.size}")
    acc = fp8.e4m3_decode(w_codes, np.float64) @ fp8.e4m3_decode(x_codes, np.float64)
    return acc * sx[0] * (sw if sw.size == N else sw[0])


def expand_block_scale(scale: np.ndarray, N: int, K: int, block: int = 128) -> np.ndarray:
    """Broadcast a [N or ceil(N/block), ceil(K/block)] scale to [N, K]."""
    scale = np.asarray(scale, dtype=np.float64)
    kb = -(-K // block)
    nb = -(-N // block)
    if scale.shape == (N, kb):
        rows = scale
    elif scale.shape == (nb, kb):
        rows = np.repeat(scale, block, axis=0)[:N]
    else:
        raise ValueError(f"scale shape {scale.shape} matches neither ({N},{kb}) nor ({nb},{kb})")
    return np.repeat(rows, block, axis=1)[:, :K]


def fused_fp8_gemm_oracle(w_codes, w_scale, a) -> np.ndarray:
    """a [..., K] real numbers -> float64 [..., N]."""
    w_codes = np.asarray(w_codes)
    if w_codes.dtype != np.uint8:
        raise TypeError(f"w_fp8 must be uint8 (fp8 storage); got {w_codes.dtype}")
    if w_codes.ndim != 2:
        raise ValueError(f"w_fp8 must be 2D [M, K]; got {w_codes.shape}")
    N, K = w_codes.shape
    a = np.asarray(a, dtype=np.float64)
    if a.shape[-1] != K:
        raise ValueError(f"a.shape[-1] ({a.shape[-1]}) must equal w_fp8.shape[1] ({K})")
    w = fp8.e4m3_decode(w_codes, np.float64) * expand_block_scale(w_scale, N, K)
    return a @ w.T
