"""Float-carrier sparse-MLA apply with the reference's Path B wrapper names.

Surface of the reference's ``cppmega_mlx/nn/_tilelang/sparse_mla.py:126-158``:
``sparse_mla_apply(q, kv, indices, *, sm_scale, d_v, return_lse, force_metal)``.
The reference's direct-MSL Path B is retired and a forced request raises; the
unforced call runs the reference-path HIP kernel.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import torch

from ..sparse_mla import _resolve_shapes, sparse_mla_attention_reference

__all__ = ["SparseMLAMetalStatus", "sparse_mla_apply", "sparse_mla_metal_status"]

_RETIRED = "sparse_mla direct-MSL Path B is retired; use sparse_mla_path_c_apply or sparse_mla_attention"


@dataclass(frozen=True)
class SparseMLAMetalStatus:
    available: bool
    reason: str


def sparse_mla_metal_status(*arrays: torch.Tensor) -> SparseMLAMetalStatus:
    if len(arrays) == 3:
        _resolve_shapes(arrays[0], arrays[1], arrays[2], d_v=None)
    return SparseMLAMetalStatus(False, _RETIRED)


def sparse_mla_apply(
    q: torch.Tensor,
    kv: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float | None = None,
    d_v: int | None = None,
    return_lse: bool = False,
    force_metal: bool = False,
) -> torch.Tensor | Tuple[torch.Tensor, torch.Tensor]:
    shapes = _resolve_shapes(q, kv, indices, d_v=d_v)
    if sm_scale is None:
        sm_scale = shapes.qk_dim ** -0.5
    if force_metal:
        raise RuntimeError(f"sparse_mla_apply: Metal path unavailable: {_RETIRED}")
    return sparse_mla_attention_reference(q, kv, indices, sm_scale=sm_scale, d_v=d_v, return_lse=return_lse)
