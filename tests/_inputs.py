"""Seeded input builders shared by the GPU parity tests (NumPy side; the torch
tensors are made from these arrays so both paths see identical bits)."""

from __future__ import annotations

import numpy as np
import torch

from oracle import fp8, sparse_mla as om


def to_dev(a: np.ndarray, device) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def bf16_pair(x: np.ndarray, device):
    """float32 array -> (bf16 device tensor, the exact float32 values it holds)."""
    t = to_dev(x.astype(np.float32), device).to(torch.bfloat16)
    return t, t.to(torch.float32).cpu().numpy()


def topk_scores(rng, rows: int, width: int, tie_fraction: float = 0.05) -> np.ndarray:
    """N(0,1) scores with `tie_fraction` of each row overwritten by copies of other
    entries of the same row (exact ties)."""
    s = rng.standard_normal((rows, width)).astype(np.float32)
    n = int(width * tie_fraction)
    if n:
        for r in range(rows):
            dst = rng.integers(0, width, n)
            src = rng.integers(0, width, n)
            s[r, dst] = s[r, src]
    return s


def sparse_indices(rng, B, S, G, Skv, topk, *, causal_offset: int | None = None, replace: bool = False) -> np.ndarray:
    """Per-query indices. causal_offset=None: uniform over [0,Skv). Otherwise query
    i sees positions [0, causal_offset+i] and gets min(topk, visible) distinct
    positions, padded with -1."""
    idx = np.full((B, S, G, topk), -1, dtype=np.int64)
    for b in range(B):
        for s in range(S):
            for g in range(G):
                visible = Skv if causal_offset is None else min(Skv, causal_offset + s + 1)
                n = topk if replace else min(topk, visible)
                idx[b, s, g, :n] = rng.choice(visible, size=n, replace=replace)
    return idx


def latent_cache(rng, B, Skv, G, d_latent, d_rope, device, *, pow2: bool, block: int = 128):
    """FP8 latent KV cache: (codes u8, scale f32 [..,d_latent/block], rope bf16) on
    the device plus the float64 rows [B,Skv,G,d_latent+d_rope] they decode to."""
    lat = rng.standard_normal((B, Skv, G, d_latent)).astype(np.float32)
    codes, scale = fp8.quantize_block(lat, block, pow2=pow2)
    rope_t, rope_f = bf16_pair(rng.standard_normal((B, Skv, G, d_rope)), device) if d_rope else (None, None)
    rows = om.dequant_block_latent(codes, scale, rope_f, block)
    return to_dev(codes, device), to_dev(scale, device), rope_t, rows


def error_report(got: np.ndarray, want: np.ndarray) -> tuple[float, float]:
    """(max abs error, max |want|): the ratio is what the 2e-2 budget applies to."""
    return float(np.abs(got.astype(np.float64) - want).max()), float(np.abs(want).max())
