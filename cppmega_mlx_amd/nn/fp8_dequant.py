"""Block-128 FP8 checkpoint weights -> bfloat16.

Surface of the reference's ``cppmega_v4/nn/_external/_mlx_lm_fp8_dequant_vendored.py``:
``dequant_block_fp8`` :24-46 and ``sanitize_fp8_weights`` :50-71 (every
``<prefix>.weight_scale_inv`` key replaces its e4m3 ``<prefix>.weight`` by the bfloat16 product;
``activation_scale`` keys are dropped; a state dict without such keys is returned as a copy).
"""

from __future__ import annotations

from typing import Mapping

import torch

from .. import ops

__all__ = ["dequant_block_fp8", "sanitize_fp8_weights"]


def dequant_block_fp8(weight: torch.Tensor, scale_inv: torch.Tensor) -> torch.Tensor:
    """[m, n] e4m3 bytes times float32 ``scale_inv`` [ceil(m/128), ceil(n/128)] -> bfloat16 [m, n]."""
    out = torch.empty(tuple(weight.shape), dtype=torch.bfloat16, device=weight.device)
    return ops.dequant_block_fp8(weight.contiguous(), scale_inv.to(torch.float32).contiguous(), out=out)


def sanitize_fp8_weights(weights: Mapping[str, torch.Tensor]) -> dict[str, torch.Tensor]:
    if not any("weight_scale_inv" in k for k in weights):
        return dict(weights)
    new_weights: dict[str, torch.Tensor] = {}
    for k, v in weights.items():
        if "weight_scale_inv" in k:
            wk = k.replace("_scale_inv", "")
            new_weights[wk] = dequant_block_fp8(weights[wk], v)
        elif "activation_scale" in k:
            continue
        elif k not in new_weights:
            new_weights[k] = v
    return new_weights
