"""The producer-side quantisers against the seeded parity receipts the reference holds.

scripts/bench_tilelang_sparse_mla_fp8.py:105-125 builds its inputs from
``np.random.default_rng(seed)`` (defaults :371-382: batch 1, seq 64, heads 4, kv_group 1,
qk_dim 64, d_v 32, topk 16, scale 0.1, seed 0; indices 0..15 with the upper half -1) and
writes max|fp8_reference - plain| and max|blockscaled_reference - plain| (:443-445,
:814, :923) into bench/tilelang_ports/sparse_mla_fp8.json and
sparse_mla_blockscaled.json.  Those two numbers are the only reference-held results that
depend on ``mx.to_fp8`` / ``mx.quantize(mode="mxfp8")``, so they pin the oracle's quantisers.
"""

import numpy as np
import pytest

from oracle import fp8, sparse_mla as om

FP8_VS_PLAIN = 0.0030034519731998444          # sparse_mla_fp8.json parity.fp8_vs_bf16.max_abs_err
BLOCKSCALED_VS_PLAIN = 0.011328823864459991   # sparse_mla_blockscaled.json parity.blockscaled_vs_bf16.max_abs_err


def receipt_inputs(seed=0, batch=1, seq=64, heads=4, group=1, qk_dim=64, topk=16, scale=0.1):
    rng = np.random.default_rng(seed)
    q = (rng.standard_normal((batch, seq, heads, qk_dim)) * scale).astype(np.float32)
    kv = (rng.standard_normal((batch, seq, group, qk_dim)) * scale).astype(np.float32)
    idx = np.tile(np.arange(topk, dtype=np.int32).reshape(1, 1, 1, topk), (batch, seq, group, 1))
    idx[..., topk // 2:] = -1
    idx[idx >= seq] = -1
    return q, kv, idx


def test_per_tensor_fp8_receipt():
    q, kv, idx = receipt_inputs()
    plain, _ = om.sparse_mla_oracle(q, kv, idx, d_v=32)
    got, _ = om.sparse_mla_oracle(fp8.roundtrip_per_tensor(q), fp8.roundtrip_per_tensor(kv), idx, d_v=32)
    assert abs(np.abs(got - plain).max() - FP8_VS_PLAIN) <= 1e-7


def test_mxfp8_receipt():
    q, kv, idx = receipt_inputs()
    plain, _ = om.sparse_mla_oracle(q, kv, idx, d_v=32)
    got, _ = om.sparse_mla_oracle(fp8.roundtrip_mxfp8(q), fp8.roundtrip_mxfp8(kv), idx, d_v=32)
    assert abs(np.abs(got - plain).max() - BLOCKSCALED_VS_PLAIN) <= 1e-7


@pytest.mark.parametrize("rule", ["ceil", "floor", "ocp"])
def test_receipt_rejects_the_other_exponent_rules(rule):
    """The receipt tells the candidate scale-byte rules apart by a factor of 1.5 or more."""
    q, kv, idx = receipt_inputs()

    def roundtrip(x):
        xb = x.reshape(x.shape[:-1] + (x.shape[-1] // 32, 32)).astype(np.float64)
        amax = np.abs(xb).max(axis=-1)
        if rule == "ocp":
            e = np.floor(np.log2(amax)) - 8
        else:
            e = getattr(np, rule)(np.log2(amax / 448.0))
        sc = np.exp2(e)[..., None]
        codes = fp8.e4m3_encode(np.clip(xb / sc, -448, 448))
        return (fp8.e4m3_decode(codes, np.float64) * sc).reshape(x.shape).astype(np.float32)

    plain, _ = om.sparse_mla_oracle(q, kv, idx, d_v=32)
    got, _ = om.sparse_mla_oracle(roundtrip(q), roundtrip(kv), idx, d_v=32)
    assert abs(np.abs(got - plain).max() - BLOCKSCALED_VS_PLAIN) > 3e-3


def test_mxfp8_exponent_rounds_to_nearest():
    x = np.zeros((4, 32), np.float32)
    x[0, 3] = 448.0                      # log2(1) = 0
    x[1, 3] = 448.0 * 1.40               # log2 = 0.485 -> 0, value saturates
    x[2, 3] = 448.0 * 1.42               # log2 = 0.506 -> 1
    x[3, 3] = 448.0 * 0.70               # log2 = -0.515 -> -1
    codes, byte = fp8.quantize_mxfp8(x)
    assert byte[:, 0].tolist() == [127, 127, 128, 126]
    assert codes[1, 3] == 0x7E           # saturated at 448
