"""FP8 e4m3fn / E8M0 codecs used by the oracle and by the test input generators.

TEST INFRASTRUCTURE ONLY -- the shipped package never imports this module.

Reference anchors:
  * e4m3 bit layout: cppmega_mlx/nn/_tilelang/sparse_mla_fp8.py:177-228 and
    cppmega_v4/_tilelang/fused_fp8_gemm.py:100-121 (sign | 4-bit exponent,
    bias 7 | 3-bit mantissa; exponent 0 is subnormal m/8 * 2**-6; 0x7F and
    0xFF are NaN).
  * E8M0 rule: tests/test_tilelang_sparse_mla_blockscaled.py:332-334.
  * per-token amax scale max(amax/448, 1e-12):
    cppmega_mlx/nn/_tilelang/sparse_mla_fp8.py:123-147.
"""

from __future__ import annotations

import numpy as np

E4M3_MAX = 448.0


def _build_e4m3_table() -> np.ndarray:
    table = np.zeros(256, dtype=np.float64)
    for byte in range(256):
        sign = -1.0 if byte & 0x80 else 1.0
        expo = (byte >> 3) & 0xF
        mant = byte & 0x7
        if expo == 0xF and mant == 0x7:
            value = float("nan")
        elif expo == 0:
            value = sign * (mant / 8.0) * 2.0 ** -6
        else:
            value = sign * (1.0 + mant / 8.0) * 2.0 ** (expo - 7)
        table[byte] = value
    return table


E4M3_TABLE_F64 = _build_e4m3_table()
E4M3_TABLE_F32 = E4M3_TABLE_F64.astype(np.float32)


def e4m3_decode(codes: np.ndarray, dtype=np.float32) -> np.ndarray:
    """uint8 e4m3fn storage -> float (NaN bytes decode to NaN, as mx.from_fp8)."""
    codes = np.asarray(codes)
    if codes.dtype != np.uint8:
        raise TypeError(f"e4m3_decode expects uint8 storage, got {codes.dtype}")
    table = E4M3_TABLE_F64 if dtype == np.float64 else E4M3_TABLE_F32
    return table[codes].astype(dtype, copy=False)


def e8m0_decode(codes: np.ndarray, dtype=np.float32) -> np.ndarray:
    """E8M0 scale byte -> float: 0 and 255 decode to 0, else 2**(b-127)."""
    codes = np.asarray(codes)
    if codes.dtype != np.uint8:
        raise TypeError(f"e8m0_decode expects uint8 storage, got {codes.dtype}")
    as_int = codes.astype(np.int32)
    value = np.ldexp(np.ones(as_int.shape, dtype=np.float64), as_int - 127)
    value = np.where((as_int == 0) | (as_int == 255), 0.0, value)
    return value.astype(dtype)


_POS_GRID = E4M3_TABLE_F64[:0x7F]  # bytes 0x00..0x7E: ascending non-negative values


def e4m3_encode(values: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even onto the e4m3fn grid with saturation at +-448.

    Producer-side helper (input generation).  Nearest grid point; exact
    midpoints go to the code with even mantissa LSB, which for this grid is the
    even byte value.
    """
    x = np.asarray(values, dtype=np.float64)
    if np.isnan(x).any():
        raise ValueError("e4m3_encode: NaN inputs are not supported")
    sign = np.signbit(x)
    mag = np.minimum(np.abs(x), E4M3_MAX)
    hi = np.searchsorted(_POS_GRID, mag, side="left")  # first grid >= mag
    hi = np.clip(hi, 0, len(_POS_GRID) - 1)
    lo = np.clip(hi - 1, 0, len(_POS_GRID) - 1)
    d_hi = np.abs(_POS_GRID[hi] - mag)
    d_lo = np.abs(mag - _POS_GRID[lo])
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & ((lo & 1) == 0))
    code = np.where(pick_lo, lo, hi).astype(np.uint8)
    return (code | (sign.astype(np.uint8) << 7)).astype(np.uint8)


def quantize_per_token(x: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """Per-row (last axis) amax quantiser in float32 arithmetic, as the producer kernel
    states it: scale = max(amax * float32(1/448), 1e-12); code = rne(clamp(x / scale, +-448)).

    Follows cppmega_mlx/nn/_tilelang/sparse_mla_fp8_path_c.py:2683-2709.
    Returns (codes uint8 [..., K], scale float32 [...]).
    """
    x = np.asarray(x, dtype=np.float32)
    amax = np.max(np.abs(x), axis=-1).astype(np.float32)
    scale = np.maximum(amax * np.float32(1.0 / 448.0), np.float32(1e-12)).astype(np.float32)
    norm = np.clip((x / scale[..., None]).astype(np.float32), np.float32(-E4M3_MAX), np.float32(E4M3_MAX))
    return e4m3_encode(norm), scale


def quantize_per_tensor(x: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """One amax scale for the whole tensor, replicated per row: the float-carrier producer
    cppmega_mlx/nn/_tilelang/sparse_mla_fp8.py:123-145 (scale = max(amax/448, 1e-12), float32
    arithmetic), codes round-to-nearest-even with saturation like the per-token producer kernel.
    ``mx.to_fp8`` is not in the tree; pinned by the reference's seeded receipt
    bench/tilelang_ports/sparse_mla_fp8.json ``parity.fp8_vs_bf16.max_abs_err`` =
    0.0030034519731998444 (scripts/bench_tilelang_sparse_mla_fp8.py:105-125,443-444), which this
    reproduces to 1.4e-8 (float32 matmul-order noise of the reference's run)."""
    x = np.asarray(x, dtype=np.float32)
    amax = np.float32(np.max(np.abs(x))) if x.size else np.float32(0)
    scale = np.maximum(amax * np.float32(1.0 / 448.0), np.float32(1e-12)).astype(np.float32)
    norm = np.clip((x / scale).astype(np.float32), np.float32(-E4M3_MAX), np.float32(E4M3_MAX))
    return e4m3_encode(norm), np.full(x.shape[:-1], scale, dtype=np.float32)


def roundtrip_per_tensor(x: np.ndarray) -> np.ndarray:
    """dec(quantize_per_tensor(x)) * scale in float32 (sparse_mla_fp8.py:160-166)."""
    codes, scale = quantize_per_tensor(x)
    return (e4m3_decode(codes) * scale[..., None]).astype(np.float32)


def roundtrip_mxfp8(x: np.ndarray) -> np.ndarray:
    """dec(quantize_mxfp8(x)) * 2^(byte-127) in float32 (sparse_mla_blockscaled.py:90-98)."""
    codes, byte = quantize_mxfp8(x)
    sc = np.repeat(e8m0_decode(byte), 32, axis=-1)
    return (e4m3_decode(codes) * sc).astype(np.float32)


def quantize_block(x: np.ndarray, block: int = 128, pow2: bool = True) -> tuple[np.ndarray, np.ndarray]:
    """Block-scaled quantiser along the last axis (one fp32 scale per `block`).

    scale = 2**ceil(log2(amax/448)) when ``pow2`` (the benchmark's weight and
    KV-cache generator), else amax/448 (the FP8Linear producer,
    cppmega_v4/nn/moe_fp8.py:36-58).  All-zero blocks get scale 1.
    Returns (codes uint8 [..., K], scale float32 [..., K/block]).
    """
    x = np.asarray(x, dtype=np.float32)
    k = x.shape[-1]
    if k % block:
        raise ValueError(f"last dim {k} not divisible by block {block}")
    xb = x.reshape(x.shape[:-1] + (k // block, block)).astype(np.float64)
    amax = np.max(np.abs(xb), axis=-1)
    raw = amax / E4M3_MAX
    if pow2:
        with np.errstate(divide="ignore"):
            scale = np.where(amax > 0, np.exp2(np.ceil(np.log2(np.where(amax > 0, raw, 1.0)))), 1.0)
    else:
        scale = np.where(amax > 0, raw, 1.0)
    scale = scale.astype(np.float32)
    codes = e4m3_encode(xb / scale[..., None].astype(np.float64)).reshape(x.shape)
    return codes, scale


def quantize_mxfp8(x: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """E8M0-per-32 quantiser: ``mx.quantize(mode="mxfp8")`` as the reference calls it
    (cppmega_mlx/nn/_tilelang/sparse_mla_blockscaled.py:75).

    scale byte = 127 + rint(log2(amax/448)) clamped to [1, 254] (the exponent is rounded to
    the NEAREST integer, so up to sqrt(2) of a block's range saturates at +-448); codes =
    rne(clamp(x / 2**(byte-127), +-448)).  MLX's source is not in the tree; the rule is pinned
    by the seeded receipt the reference holds, bench/tilelang_ports/sparse_mla_blockscaled.json
    ``parity.blockscaled_vs_bf16.max_abs_err`` = 0.011328823864459991 (written by
    scripts/bench_tilelang_sparse_mla_fp8.py:105-125,443-445): round reproduces it to 4e-9,
    ceil gives 2.16e-3, floor 1.77e-2, the OCP floor(log2 amax) - 8 rule 2.17e-3.  Left open by
    the receipt: which way an exponent exactly half-way between two integers rounds
    (amax = 448 * 2**(n + 0.5) is not a float, so the case cannot occur).
    """
    x = np.asarray(x, dtype=np.float32)
    k = x.shape[-1]
    if k % 32:
        raise ValueError(f"last dim {k} not divisible by 32")
    xb = x.reshape(x.shape[:-1] + (k // 32, 32)).astype(np.float64)
    amax = np.max(np.abs(xb), axis=-1)
    with np.errstate(divide="ignore"):
        expo = np.where(amax > 0, np.rint(np.log2(np.where(amax > 0, amax / E4M3_MAX, 1.0))), 0.0)
    byte = np.clip(expo + 127, 1, 254).astype(np.uint8)
    scale = np.exp2(byte.astype(np.float64) - 127)
    codes = e4m3_encode(np.clip(xb / scale[..., None], -E4M3_MAX, E4M3_MAX)).reshape(x.shape)
    return codes, byte


def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round float32 to the nearest bfloat16 (ties to even); returns float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    rounding = ((bits >> 16) & 1) + 0x7FFF
    out = (((bits + rounding) >> 16) << 16).astype(np.uint32)
    res = out.view(np.float32).reshape(x.shape)
    return np.where(np.isnan(x), x, res)
