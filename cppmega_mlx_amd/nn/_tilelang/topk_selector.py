"""Top-k indexer selector on MI355X.

Public surface of the reference's ``cppmega_mlx/nn/_tilelang/topk_selector.py``
(``topk_selector_reference`` :227-330, ``topk_selector_tilelang_direct``
:714-790, ``topk_selector_tilelang`` :793-830, ``topk_selector`` :868-909,
``PathCStatus`` :362-367, ``TopKPathCDirectError`` :370-371), served by one HIP
kernel: a wavefront radix select that keeps the score row in registers.

Contract: int32 ``(B, k)`` indices of the ``k`` largest scores per row among
columns ``[clip(start), clip(end))``; ties go to the lower index; slots past
the number of selectable columns hold ``-1``.  The reference leaves the order
of the selected indices open (its tests compare sets, :251-254); here the order
is chosen by ``order=``:

* ``"index"`` (default) -- ascending column index, ``-1`` padding last;
* ``"value"`` -- value descending, lower index first among equal values: the
  order the reference's Path C kernel produces
  (tests/test_tilelang_topk.py:596-610).

Differences from the reference, all additive: masked rows run on the GPU path
too (the reference's Path C rejects them, :728-733); bfloat16 scores are
accepted; ``(B, S, T)`` scores are accepted by ``topk_selector`` and flattened;
``neg_inf_is_masked=True`` makes an in-range ``-inf`` score unselectable.  NaN
scores are never selected.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ... import _lib, ops

__all__ = [
    "PathBStatus",
    "PathCStatus",
    "TopKPathCDirectError",
    "topk_selector",
    "topk_selector_metal",
    "topk_selector_path_b_status",
    "topk_selector_path_c_status",
    "topk_selector_reference",
    "topk_selector_tilelang",
    "topk_selector_tilelang_direct",
]

MAX_WIDTH = 65536  # columns one workgroup keeps in registers
_SCORE_DTYPES = (torch.float32, torch.float16, torch.bfloat16)


@dataclass(frozen=True)
class PathCStatus:
    """Why the HIP kernel path is or is not available."""

    available: bool
    reason: str


@dataclass(frozen=True)
class PathBStatus:
    available: bool
    reason: str


class TopKPathCDirectError(RuntimeError):
    """Raised when the owner-output kernel route cannot run."""


_PATH_B_RETIRED_REASON = (
    "topk_selector direct-MSL Path B is retired; every call is served by the HIP radix-select kernel."
)


def topk_selector_path_c_status() -> PathCStatus:
    try:
        st = _lib.status()
    except _lib.NativeLibraryError as exc:
        return PathCStatus(False, str(exc))
    if st["gfx950_devices"] < 1:
        return PathCStatus(False, st["message"])
    return PathCStatus(True, "topk_selector HIP radix-select kernel (gfx950) is available")


def topk_selector_path_b_status() -> PathBStatus:
    return PathBStatus(False, _PATH_B_RETIRED_REASON)


def _check_scores(scores: torch.Tensor, k: int) -> tuple[int, int]:
    if scores.ndim != 2:
        raise ValueError(f"topk_selector expects a (B, T) array; got shape {tuple(scores.shape)}")
    batch, seq_len = int(scores.shape[0]), int(scores.shape[1])
    if k < 1 or k > seq_len:
        raise ValueError(f"topk must be in [1, {seq_len}]; got {k}")
    return batch, seq_len


def _bounds(bound: torch.Tensor | None, batch: int, name: str) -> torch.Tensor | None:
    if bound is None:
        return None
    if tuple(bound.shape) != (batch,):
        raise ValueError(f"starts/ends must have shape (B,); got {name}={tuple(bound.shape)}")
    if bound.dtype != torch.int32:
        raise TypeError(f"{name} must be int32 (the boundary does not cast); got {bound.dtype}")
    return bound


def topk_selector_tilelang_direct(
    scores: torch.Tensor,
    k: int,
    *,
    out: torch.Tensor,
    starts: torch.Tensor | None = None,
    ends: torch.Tensor | None = None,
    order: str = "value",
    neg_inf_is_masked: bool = False,
) -> torch.Tensor:
    """Run the kernel into caller-owned ``out`` (int32 ``(B, k)``) and return ``out``.

    Stream-ordered: the result is valid for work enqueued afterwards on the
    current stream; no host synchronisation happens here.  The default order
    is value-descending, the order of the reference kernel this entry replaces.
    """
    batch, _ = _check_scores(scores, k)
    if batch <= 0 or scores.numel() == 0:
        raise TopKPathCDirectError("empty topk inputs are not dispatchable")
    if scores.dtype not in _SCORE_DTYPES:
        raise TopKPathCDirectError(
            f"topk_selector kernel supports float32/float16/bfloat16 scores without hidden casts; got {scores.dtype}"
        )
    if not isinstance(out, torch.Tensor):
        raise TypeError(f"topk_selector_tilelang: out must be a torch.Tensor; got {type(out).__name__}")
    if tuple(out.shape) != (batch, int(k)):
        raise ValueError(f"topk_selector_tilelang: out shape must be ({batch}, {int(k)}); got {tuple(out.shape)}")
    if out.dtype != torch.int32:
        raise ValueError(f"topk_selector_tilelang: out dtype must be torch.int32; got {out.dtype}")
    starts = _bounds(starts, batch, "starts")
    ends = _bounds(ends, batch, "ends")
    if scores.shape[1] > MAX_WIDTH:
        raise TopKPathCDirectError(f"topk_selector kernel handles rows of up to {MAX_WIDTH} columns; got {scores.shape[1]}")
    try:
        returned = ops.topk_select(scores, int(k), out=out, starts=starts, ends=ends, order=order,
                                   neg_inf_is_masked=neg_inf_is_masked)
    except (_lib.NativeCallError, _lib.NativeLibraryError) as exc:
        raise TopKPathCDirectError(f"topk kernel dispatch failed: {type(exc).__name__}: {exc}") from exc
    if returned is not out:
        raise TopKPathCDirectError("topk kernel did not return the caller-owned output")
    return out


def topk_selector_tilelang(
    scores: torch.Tensor,
    k: int,
    *,
    starts: torch.Tensor | None = None,
    ends: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
    order: str = "value",
) -> torch.Tensor | None:
    """Kernel forward; ``None`` when it cannot dispatch or no ``out`` is given."""
    batch, _ = _check_scores(scores, k)
    if batch <= 0 or scores.numel() == 0:
        return None
    if not topk_selector_path_c_status().available:
        return None
    if out is None:
        return None
    return topk_selector_tilelang_direct(scores, k, starts=starts, ends=ends, out=out, order=order)


def topk_selector_metal(scores, k, *, starts=None, ends=None):
    """Retired Path B surface: validates and returns ``None``."""
    _check_scores(scores, k)
    del starts, ends
    return None


def topk_selector_reference(
    scores: torch.Tensor,
    k: int,
    *,
    starts: torch.Tensor | None = None,
    ends: torch.Tensor | None = None,
    order: str = "value",
) -> torch.Tensor:
    """Reference-named entry (``(B, T)`` scores, ``1 <= k <= T``).

    Same validation messages as the reference; computed by the HIP kernel in
    value-descending order, which is within the reference's "any order"
    contract and matches every exact-order answer its tests pin.
    """
    if scores.ndim != 2:
        raise ValueError(f"topk_selector expects a (B, T) array; got shape {tuple(scores.shape)}")
    if k < 1:
        raise ValueError(f"topk must be >= 1; got {k}")
    seq_len = int(scores.shape[1])
    if k > seq_len:
        raise ValueError(f"topk={k} exceeds sequence length {seq_len}")
    batch = int(scores.shape[0])
    out = torch.empty((batch, int(k)), dtype=torch.int32, device=scores.device)
    if batch == 0:
        return out
    if starts is not None and starts.dtype != torch.int32:
        starts = starts.to(torch.int32)
    if ends is not None and ends.dtype != torch.int32:
        ends = ends.to(torch.int32)
    return ops.topk_select(scores, int(k), out=out, starts=_bounds(starts, batch, "starts"),
                           ends=_bounds(ends, batch, "ends"), order=order)


def topk_selector(
    scores: torch.Tensor,
    k: int,
    *,
    starts: torch.Tensor | None = None,
    ends: torch.Tensor | None = None,
    backend: str = "auto",
    order: str = "index",
    neg_inf_is_masked: bool = False,
) -> torch.Tensor:
    """Top-k selector matching the reference's source contract.

    ``backend``: ``"auto"``, ``"hip"``, ``"tilelang"``, ``"path_c"`` and
    ``"mlx"`` all run the HIP kernel (there is no other implementation);
    ``"metal"`` raises because Path B is retired.  ``scores`` may be ``(B, T)``
    or ``(B, S, T)`` (then ``starts``/``ends`` are ``(B*S,)`` and the result is
    ``(B, S, k)``).
    """
    if backend not in {"auto", "mlx", "metal", "tilelang", "path_c", "hip"}:
        raise ValueError(f"unknown backend {backend!r}")
    if backend == "metal":
        raise RuntimeError("topk_selector: direct-MSL Path B is retired")
    lead = None
    if scores.ndim == 3:
        lead = tuple(scores.shape[:2])
        scores = scores.reshape(lead[0] * lead[1], scores.shape[2])
    batch, _ = _check_scores(scores, k)
    out = torch.empty((batch, int(k)), dtype=torch.int32, device=scores.device)
    if batch > 0:
        try:
            topk_selector_tilelang_direct(scores, k, out=out, starts=starts, ends=ends, order=order,
                                          neg_inf_is_masked=neg_inf_is_masked)
        except TopKPathCDirectError as exc:
            raise RuntimeError(f"topk_selector: HIP kernel path unavailable: {exc}") from exc
    return out.reshape(*lead, int(k)) if lead is not None else out
