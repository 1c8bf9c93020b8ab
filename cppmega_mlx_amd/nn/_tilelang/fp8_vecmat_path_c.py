"""FP8 vecmat / skinny GEMM through the HIP streaming kernels ("Path C").

Surface of the reference's ``cppmega_mlx/nn/_tilelang/fp8_vecmat_path_c.py``:
``fp8_scaled_vecmat_path_c_direct`` :983-1100, ``fp8_scaled_vecmat_path_c``
:1103-1137, ``FP8VecmatPathCDirectError`` / ``FP8VecmatPathCLegacyError``
:182-197, ``FP8VecmatPathCStatus`` :170-180.

Reference-shaped call: ``x_fp8`` uint8 ``(K,)``, ``W_fp8`` uint8 ``(N, K)``,
``scale_x`` float32 ``(1,)`` tensor, ``scale_w`` float32 ``(1,)`` or ``(N,)``
tensor (Python scalars are rejected: the boundary allocates nothing),
caller-owned ``out`` ``(N,)``.  The launch is asynchronous on the current
stream and ``out`` itself is returned.

Decode-projection extension (keyword-compatible):
``x`` may be bfloat16/float16/float32 ``(K,)`` or ``(M, K)`` with
``scale_x=None``; ``scale_w`` may be float32 ``(N, K/128)`` (one scale per row
and 128-wide K block) or ``(ceil(N/128), ceil(K/128))`` (the 128x128 grid of
``fused_fp8_gemm``); ``out`` is then ``(N,)`` or ``(M, N)`` in
float32/float16/bfloat16.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ... import _lib, ops

__all__ = [
    "FP8VecmatPathCDirectError",
    "FP8VecmatPathCLegacyError",
    "FP8VecmatPathCStatus",
    "fp8_scaled_vecmat_path_c",
    "fp8_scaled_vecmat_path_c_direct",
    "fp8_vecmat_path_c_status",
]

_OUT_DTYPES = (torch.float32, torch.float16, torch.bfloat16)
_X_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


@dataclass(frozen=True)
class FP8VecmatPathCStatus:
    available: bool
    reason: str
    target: str = "hip-gfx950"
    transpose_B: bool = True
    m_equals_1: bool = False


class FP8VecmatPathCDirectError(RuntimeError):
    """Raised when the owner-output vecmat path cannot run."""


class FP8VecmatPathCLegacyError(RuntimeError):
    """Raised when callers request the retired no-out allocation path."""


def fp8_vecmat_path_c_status() -> FP8VecmatPathCStatus:
    try:
        st = _lib.status()
    except _lib.NativeLibraryError as exc:
        return FP8VecmatPathCStatus(False, str(exc))
    if st["gfx950_devices"] < 1:
        return FP8VecmatPathCStatus(False, st["message"])
    return FP8VecmatPathCStatus(True, "FP8 vecmat HIP kernels (gfx950) are available")


def _raise_owner_output_required(op_name: str) -> None:
    raise FP8VecmatPathCLegacyError(
        f"{op_name}: no-out dispatch is retired. The only supported FP8 vecmat route is owner-output "
        "dispatch; pass out=existing_tensor."
    )


def _scale_w_kind(scale_w: torch.Tensor, n: int, k: int) -> int:
    kb = (k + 127) // 128
    nb = (n + 127) // 128
    if scale_w.ndim == 1:
        if scale_w.numel() == 1:
            return _lib.WSCALE_SCALAR
        if scale_w.numel() == n:
            return _lib.WSCALE_PER_ROW
        raise ValueError(
            f"fp8_scaled_vecmat_path_c direct owner-output route expected scale_w size 1 or {n}; "
            f"got shape {tuple(scale_w.shape)}"
        )
    if scale_w.ndim == 2 and tuple(scale_w.shape) == (n, kb):
        return _lib.WSCALE_ROW_BLOCK
    if scale_w.ndim == 2 and tuple(scale_w.shape) == (nb, kb):
        return _lib.WSCALE_GRID_128
    raise ValueError(
        f"scale_w must be (1,), ({n},), ({n}, {kb}) or ({nb}, {kb}); got {tuple(scale_w.shape)}"
    )


def fp8_scaled_vecmat_path_c_direct(
    x_fp8: torch.Tensor,
    W_fp8: torch.Tensor,
    *,
    scale_x,
    scale_w,
    out: torch.Tensor,
    outputs_per_block: int = 4,
    reduce_threads: int = 32,
    vec: int = 4,
) -> torch.Tensor:
    """Run the vecmat into caller-owned ``out``; returns ``out``.

    ``outputs_per_block`` / ``reduce_threads`` / ``vec`` are the reference
    kernel's tuning knobs; the HIP kernels pick their own tiling and ignore them.
    """
    del outputs_per_block, reduce_threads, vec
    if not fp8_vecmat_path_c_status().available:
        raise FP8VecmatPathCDirectError(fp8_vecmat_path_c_status().reason)
    if W_fp8.ndim != 2 or x_fp8.ndim not in (1, 2):
        raise ValueError(
            f"fp8_scaled_vecmat_path_c direct owner-output route expects 1D x and 2D W; "
            f"got x.ndim={x_fp8.ndim}, W.ndim={W_fp8.ndim}"
        )
    if W_fp8.dtype != torch.uint8:
        raise ValueError(f"fp8_scaled_vecmat_path_c direct owner-output route expects torch.uint8 e4m3 storage for W; got {W_fp8.dtype}")
    n, k_w = (int(v) for v in W_fp8.shape)
    k = int(x_fp8.shape[-1])
    if k != k_w:
        raise ValueError(
            f"fp8_scaled_vecmat_path_c direct owner-output route shape mismatch: x=(K={k}), W=(N={n}, K={k_w})"
        )
    if isinstance(scale_w, (int, float)) or isinstance(scale_x, (int, float)):
        raise TypeError(
            "fp8_scaled_vecmat_path_c direct owner-output route requires scales as existing float32 tensors; "
            "Python scalars would allocate a new tensor at the wrapper boundary"
        )
    if not isinstance(scale_w, torch.Tensor) or scale_w.dtype != torch.float32:
        raise ValueError("scale_w must be a float32 tensor")
    if x_fp8.dtype == torch.uint8:
        if x_fp8.ndim != 1:
            raise ValueError("an FP8 activation is a single (K,) vector")
        if k % 4 != 0:
            raise ValueError(f"fp8_scaled_vecmat_path_c direct owner-output route requires K multiple of 4; got K={k}")
        if not isinstance(scale_x, torch.Tensor) or scale_x.ndim != 1 or scale_x.dtype != torch.float32 or scale_x.numel() != 1:
            raise ValueError("fp8_scaled_vecmat_path_c direct owner-output route expects scale_x as 1D float32 of size 1")
    elif x_fp8.dtype in _X_FLOATS:
        if scale_x is not None:
            raise ValueError("a float activation takes scale_x=None")
    else:
        raise ValueError(f"x must be uint8 e4m3 storage or a float tensor; got {x_fp8.dtype}")
    kind = _scale_w_kind(scale_w, n, k)
    if not isinstance(out, torch.Tensor):
        raise TypeError(f"fp8_scaled_vecmat_path_c: out must be a torch.Tensor; got {type(out).__name__}")
    want = (n,) if x_fp8.ndim == 1 else (int(x_fp8.shape[0]), n)
    if tuple(out.shape) != want:
        raise ValueError(f"fp8_scaled_vecmat_path_c: out shape must be {want}; got {tuple(out.shape)}")
    if out.dtype not in _OUT_DTYPES:
        raise ValueError(f"fp8_scaled_vecmat_path_c: out dtype must be float32, float16 or bfloat16; got {out.dtype}")
    try:
        return ops.fp8_vecmat(x_fp8, W_fp8, scale_w, out=out, scale_x=scale_x, scale_w_kind=kind)
    except (_lib.NativeCallError, _lib.NativeLibraryError) as exc:
        raise FP8VecmatPathCDirectError(f"FP8 vecmat dispatch failed: {type(exc).__name__}: {exc}") from exc


def fp8_scaled_vecmat_path_c(
    x_fp8: torch.Tensor,
    W_fp8: torch.Tensor,
    *,
    scale_x,
    scale_w,
    outputs_per_block: int = 4,
    reduce_threads: int = 32,
    vec: int = 4,
    out: torch.Tensor | None = None,
) -> torch.Tensor | None:
    """Owner-output FP8 vecmat; without ``out`` it fails explicitly."""
    if out is not None:
        return fp8_scaled_vecmat_path_c_direct(
            x_fp8, W_fp8, scale_x=scale_x, scale_w=scale_w, out=out,
            outputs_per_block=outputs_per_block, reduce_threads=reduce_threads, vec=vec)
    _raise_owner_output_required("fp8_scaled_vecmat_path_c")
