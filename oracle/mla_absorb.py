"""Absorbed MLA decode and block-128 FP8 weight dequantisation.  TEST INFRASTRUCTURE ONLY.

NumPy float64 restatements of the reference's ``cppmega_v4/nn/mla_absorb.py``
(``absorb_weights`` :39-77, ``absorbed_mla_decode`` :80-138, ``standard_mla_decode`` :141-172)
and of ``dequant_block_fp8`` / ``sanitize_fp8_weights``
(cppmega_v4/nn/_external/_mlx_lm_fp8_dequant_vendored.py:24-71).

Pinned by the identity the reference's own test states
(tests/v4/test_mla_absorb.py:36-50: absorbed == standard on seeded inputs, atol = rtol = 1e-4),
which a transposed weight, a dropped head or a wrong contraction axis breaks; the shapes of
:18-26; the -1e9 mask case of :53-67 against a softmax over the unmasked positions only; and for
the dequantiser a per-element loop over 128 x 128 blocks on shapes that are not multiples of 128
plus the key handling of tests/v4/test_fp8_dequant.py:68-95.
"""

from __future__ import annotations

import numpy as np

from . import fp8


def absorb_weights(w_uk, w_uv, w_o):
    w_uk, w_uv, w_o = (np.asarray(a, dtype=np.float64) for a in (w_uk, w_uv, w_o))
    if w_uk.ndim != 3:
        raise ValueError(f"w_uk must be [H, D_kv, D_k], got {w_uk.shape}")
    if w_uv.ndim != 3 or w_uv.shape[0] != w_uk.shape[0] or w_uv.shape[1] != w_uk.shape[1]:
        raise ValueError(f"w_uv shape {w_uv.shape} inconsistent with w_uk {w_uk.shape}")
    h, d_kv, d_v = w_uv.shape
    if w_o.ndim != 2 or w_o.shape[0] != h * d_v:
        raise ValueError(f"w_o shape {w_o.shape} must be (H*D_v={h * d_v}, D_model)")
    return np.transpose(w_uk, (0, 2, 1)), np.matmul(w_uv, w_o.reshape(h, d_v, w_o.shape[1]))


def _softmax(x):
    m = x.max(axis=-1, keepdims=True)
    e = np.exp(x - m)
    return e / e.sum(axis=-1, keepdims=True)


def absorbed_mla_decode(q, c_kv, w_uk_abs, w_uv_w_o, *, sm_scale=None, mask=None):
    q, c_kv, w_uk_abs, w_uv_w_o = (np.asarray(a, dtype=np.float64) for a in (q, c_kv, w_uk_abs, w_uv_w_o))
    if q.ndim != 4:
        raise ValueError(f"q must be [B, T, H, D_k], got {q.shape}")
    if c_kv.ndim != 3:
        raise ValueError(f"c_kv must be [B, T_kv, D_kv], got {c_kv.shape}")
    h, d_k, d_kv = q.shape[2], q.shape[3], c_kv.shape[-1]
    if w_uk_abs.shape != (h, d_k, d_kv):
        raise ValueError(f"w_uk_abs must be (H={h}, D_k={d_k}, D_kv={d_kv}), got {w_uk_abs.shape}")
    if w_uv_w_o.ndim != 3 or w_uv_w_o.shape[0] != h or w_uv_w_o.shape[1] != d_kv:
        raise ValueError(f"w_uv_w_o must be (H={h}, D_kv={d_kv}, D_model), got {w_uv_w_o.shape}")
    scale = d_k ** -0.5 if sm_scale is None else float(sm_scale)
    q_abs = np.einsum("bthk,hkv->bthv", q, w_uk_abs)
    logits = np.einsum("bthv,bkv->bthk", q_abs, c_kv) * scale
    if mask is not None:
        logits = logits + np.asarray(mask, dtype=np.float64)
    v_abs = np.einsum("bthk,bkv->bthv", _softmax(logits), c_kv)
    return np.einsum("bthv,hvm->btm", v_abs, w_uv_w_o)


def standard_mla_decode(q, c_kv, w_uk, w_uv, w_o, *, sm_scale=None, mask=None):
    q, c_kv, w_uk, w_uv, w_o = (np.asarray(a, dtype=np.float64) for a in (q, c_kv, w_uk, w_uv, w_o))
    scale = q.shape[-1] ** -0.5 if sm_scale is None else float(sm_scale)
    k = np.einsum("bkv,hvd->bkhd", c_kv, w_uk)
    v = np.einsum("bkv,hvd->bkhd", c_kv, w_uv)
    logits = np.einsum("bthk,bnhk->bthn", q, k) * scale
    if mask is not None:
        logits = logits + np.asarray(mask, dtype=np.float64)
    o_h = np.einsum("bthn,bnhv->bthv", _softmax(logits), v)
    b, t, h, d_v = o_h.shape
    return o_h.reshape(b, t, h * d_v) @ w_o


def dequant_block_fp8(weight, scale_inv) -> np.ndarray:
    """float32 values of the bfloat16 result: bf16(dec(byte) * scale of its 128 x 128 block)."""
    weight = np.asarray(weight)
    scale_inv = np.asarray(scale_inv, dtype=np.float32)
    m, n = weight.shape
    if scale_inv.shape != (-(-m // 128), -(-n // 128)):
        raise ValueError(f"scale_inv shape {scale_inv.shape} does not cover a {m} x {n} weight in 128 x 128 blocks")
    full = np.repeat(np.repeat(scale_inv, 128, axis=0), 128, axis=1)[:m, :n]
    return fp8.bf16_round(fp8.e4m3_decode(weight, np.float32) * full)


def sanitize_fp8_weights(weights: dict) -> dict:
    if not any("weight_scale_inv" in k for k in weights):
        return dict(weights)
    out = {}
    for k, v in weights.items():
        if "weight_scale_inv" in k:
            wk = k.replace("_scale_inv", "")
            out[wk] = dequant_block_fp8(weights[wk], v)
        elif "activation_scale" in k:
            continue
        elif k not in out:
            out[k] = v
    return out
