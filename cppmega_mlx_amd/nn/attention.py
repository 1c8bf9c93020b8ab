"""Index producers of the attention block that feed the sparse-MLA kernels.

Mirrors ``causal_sparse_indices`` and ``sparse_indices_from_attention_mask`` of the reference
(``cppmega_mlx/nn/attention.py:251-360``): same names, arguments, validation order and error
types; ``torch.Tensor`` on the GPU in place of ``mx.array``.  Both run a HIP kernel; the device
is the one given (or the mask's).
"""

from __future__ import annotations

import torch

from .. import ops

__all__ = ["causal_sparse_indices", "sparse_indices_from_attention_mask"]


def causal_sparse_indices(
    batch_size: int,
    seq_length: int,
    kv_group: int,
    topk: int,
    *,
    query_offset: int = 0,
    key_length: int | None = None,
    device: torch.device | str = "cuda",
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """Return token-level causal sparse indices shaped ``[B, S, G, topk]`` (int32).

    Reference: ``attention.py:251-284``.  ``out=`` (owner output) avoids the allocation."""
    if batch_size <= 0:
        raise ValueError(f"batch_size must be positive, got {batch_size}")
    if seq_length <= 0:
        raise ValueError(f"seq_length must be positive, got {seq_length}")
    if kv_group <= 0:
        raise ValueError(f"kv_group must be positive, got {kv_group}")
    if topk <= 0:
        raise ValueError(f"topk must be positive, got {topk}")
    if query_offset < 0:
        raise ValueError(f"query_offset must be non-negative, got {query_offset}")
    key_length = seq_length if key_length is None else key_length
    if key_length <= 0:
        raise ValueError(f"key_length must be positive, got {key_length}")
    shape = (batch_size, seq_length, kv_group, topk)
    if out is None:
        out = torch.empty(shape, dtype=torch.int32, device=device)
    elif tuple(out.shape) != shape:
        raise ValueError(f"out must have shape {shape}, got {tuple(out.shape)}")
    return ops.causal_sparse_indices(out, query_offset=query_offset, key_length=key_length)


def sparse_indices_from_attention_mask(
    mask: torch.Tensor,
    *,
    batch_size: int,
    seq_length: int,
    kv_group: int,
    topk: int,
    key_length: int,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """Convert an explicit attention mask to sparse indices: the newest valid keys per
    query / group, ascending, ``-1`` in front (reference: ``attention.py:287-360``).

    The result has ``min(topk, key_length)`` slots per row, as in the reference."""
    if not isinstance(mask, torch.Tensor):
        raise TypeError("attention mask must be a torch.Tensor")
    if batch_size <= 0:
        raise ValueError(f"batch_size must be positive, got {batch_size}")
    if seq_length <= 0:
        raise ValueError(f"seq_length must be positive, got {seq_length}")
    if kv_group <= 0:
        raise ValueError(f"kv_group must be positive, got {kv_group}")
    if topk <= 0:
        raise ValueError(f"topk must be positive, got {topk}")
    if key_length <= 0:
        raise ValueError(f"key_length must be positive, got {key_length}")
    if mask.ndim == 2:
        valid = mask[None, None, :, :]
    elif mask.ndim == 3:
        valid = mask[:, None, :, :]
    elif mask.ndim == 4:
        valid = mask
    else:
        raise ValueError(
            "attention mask must have shape (S,K), (B,S,K), or (B,H,S,K), "
            f"got {tuple(mask.shape)}"
        )
    if tuple(valid.shape[-2:]) != (seq_length, key_length):
        raise ValueError(
            f"attention mask trailing dims must be ({seq_length}, {key_length}), "
            f"got {tuple(valid.shape[-2:])}"
        )
    if valid.shape[0] not in (1, batch_size):
        raise ValueError(
            f"attention mask batch dimension must be 1 or {batch_size}, got {valid.shape[0]}"
        )
    if valid.shape[1] not in (1, kv_group):
        raise ValueError(
            f"Path C sparse masks must be shared across heads or have {kv_group} kv groups, "
            f"got head/group dimension {valid.shape[1]}"
        )
    shape = (batch_size, seq_length, kv_group, min(topk, key_length))
    if out is None:
        out = torch.empty(shape, dtype=torch.int32, device=mask.device)
    elif tuple(out.shape) != shape:
        raise ValueError(f"out must have shape {shape}, got {tuple(out.shape)}")
    return ops.mask_sparse_indices(valid, out, topk=topk)
