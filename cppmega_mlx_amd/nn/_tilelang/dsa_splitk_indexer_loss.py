"""DSA indexer KL-divergence loss on MI355X.

Public surface of the reference's ``cppmega_mlx/nn/_tilelang/dsa_splitk_indexer_loss.py``
(``DSASplitKPathCStatus`` :253-259, ``dsa_splitk_path_c_status`` :272-281, ``tilelang_supports``
:284-305, ``dsa_splitk_indexer_loss_tilelang`` :1327-1570): same signature, same checks and
messages, same return contract (a 0-d float32 tensor ``mean(per_position_loss) * loss_coeff``).

One HIP kernel does what the reference's two stages do, one workgroup per (batch, query position),
so the four softmax-statistics buffers the reference allocates (:1467-1471) do not exist, and the
sparse variant hands the index list to the kernel instead of scattering a float [AB, ASq, Sk]
mask (:1443-1445).  ``pg_collection`` is accepted and ignored, as in the reference.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ... import _lib, ops

__all__ = [
    "DSASplitKPathCStatus",
    "dsa_splitk_indexer_loss_per_position",
    "dsa_splitk_indexer_loss_tilelang",
    "dsa_splitk_path_c_status",
    "tilelang_supports",
]

_NAME = "dsa_splitk_indexer_loss_tilelang"
_IN_DTYPES = (torch.float16, torch.bfloat16, torch.float32)


@dataclass(frozen=True)
class DSASplitKPathCStatus:
    """Whether the HIP kernel can run; the two target fields keep the reference's shape."""

    available: bool
    reason: str
    cuda_target: str = "gfx950"
    metal_target: str = "unavailable"


def dsa_splitk_path_c_status() -> DSASplitKPathCStatus:
    try:
        st = _lib.status()
    except _lib.NativeLibraryError as exc:
        return DSASplitKPathCStatus(False, str(exc))
    if st["gfx950_devices"] < 1:
        return DSASplitKPathCStatus(False, st["message"])
    return DSASplitKPathCStatus(True, "DSA split-K indexer-loss HIP kernel (gfx950) is available")


def tilelang_supports(device: torch.device | str | None) -> bool:
    """True when the kernel can dispatch on *device*: a ``cuda`` (HIP) device with the library built."""
    if device is None:
        return False
    dev_type = torch.device(device).type if isinstance(device, str) else device.type
    return dev_type == "cuda" and dsa_splitk_path_c_status().available


def _check_in_dtype(t: torch.Tensor) -> torch.dtype:
    if t.dtype not in _IN_DTYPES:
        raise TypeError(f"{_NAME}: unsupported Q/K dtype {t.dtype!r}; expected one of fp16/bf16/fp32")
    return t.dtype


def _validated_topk(topk_indices: torch.Tensor, query: torch.Tensor, AB: int, ASq: int, Sk: int) -> torch.Tensor:
    if topk_indices.device != query.device:
        raise ValueError(f"{_NAME}: topk_indices.device ({topk_indices.device}) != query.device ({query.device})")
    if topk_indices.dim() != 3 or tuple(topk_indices.shape[:2]) != (AB, ASq):
        raise ValueError(f"{_NAME}: topk_indices must have shape (AB={AB}, ASq={ASq}, TOPK); got {tuple(topk_indices.shape)}")
    if topk_indices.shape[2] == 0:
        raise ValueError(f"{_NAME}: topk_indices.shape[2] (TOPK) must be >= 1 when sparse_loss=True; got 0 — would produce "
                         "all-(-inf) index_mask -> NaN softmax -> NaN loss.")
    if topk_indices.dtype not in (torch.int32, torch.int64):
        raise TypeError(f"{_NAME}: topk_indices.dtype must be int32 or int64; got {topk_indices.dtype}")
    idx = topk_indices if topk_indices.is_contiguous() else topk_indices.contiguous()
    # One fused reduction and one host read, as the reference does on every call (:1404-1415).
    if bool(((idx < 0) | (idx >= Sk)).any().item()):
        raise ValueError(f"{_NAME}: topk_indices out of range [0, {Sk}); got [{int(idx.min().item())}, {int(idx.max().item())}].")
    return idx


def dsa_splitk_indexer_loss_per_position(index_scores: torch.Tensor, topk_indices: torch.Tensor | None, query: torch.Tensor,
                                         key: torch.Tensor, softmax_scale: float, sparse_loss: bool,
                                         out: torch.Tensor | None = None) -> torch.Tensor:
    """The [AB, ASq] float32 losses the wrapper averages (the reference's ``out_loss``, :1473)."""
    if query.shape[1] != key.shape[1] or query.shape[2] != key.shape[2] or query.shape[3] != key.shape[3]:
        raise ValueError(f"{_NAME}: query/key shape mismatch: query {tuple(query.shape)}, key {tuple(key.shape)}")
    ASq, AB, AH, AD = (int(v) for v in query.shape)
    Sk = int(key.shape[0])
    if out is None:
        out = torch.empty((AB, ASq), dtype=torch.float32, device=query.device)
    if ASq == 0 or AB == 0 or AH == 0 or AD == 0 or Sk == 0:
        return out.zero_()
    if AH > 128:
        raise ValueError(f"{_NAME}: AH > 128 is numerically unsafe in upstream PR #4039 (got AH={AH}).")
    if _check_in_dtype(key) != _check_in_dtype(query):
        raise TypeError(f"{_NAME}: query/key dtypes must match")
    if query.device.type != "cuda":
        raise ValueError(f"{_NAME}: unsupported device type {query.device.type!r}")
    idx = _validated_topk(topk_indices, query, AB, ASq, Sk) if sparse_loss else None
    scores = index_scores if index_scores.dtype == torch.float32 and index_scores.is_contiguous() else index_scores.to(torch.float32).contiguous()
    return ops.dsa_indexer_loss(query if query.is_contiguous() else query.contiguous(), key if key.is_contiguous() else key.contiguous(),
                                scores, softmax_scale=float(softmax_scale), out=out, topk_indices=idx)


def dsa_splitk_indexer_loss_tilelang(index_scores: torch.Tensor, topk_indices: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                                     softmax_scale: float, loss_coeff: float, sparse_loss: bool,
                                     pg_collection: object | None = None) -> torch.Tensor:
    """KL(attention || indexer) averaged over positions, times ``loss_coeff``; a zero-sized problem gives 0."""
    if query.ndim == 4 and key.ndim == 4 and tuple(query.shape[1:]) == tuple(key.shape[1:]) and (0 in query.shape or key.shape[0] == 0):
        return torch.zeros((), device=query.device, dtype=torch.float32)
    per_position = dsa_splitk_indexer_loss_per_position(index_scores, topk_indices, query, key, softmax_scale, sparse_loss)
    return per_position.mean() * float(loss_coeff)
