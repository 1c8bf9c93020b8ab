"""The absorb oracle against the identity and cases the reference's tests hold
(tests/v4/test_mla_absorb.py:18-84), and the block-128 dequantiser against a per-element loop and
the key handling of tests/v4/test_fp8_dequant.py:68-110."""

import numpy as np
import pytest

from oracle import fp8, mla_absorb as oa


def _rand(*shape, seed=0):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def test_absorb_weights_shapes_and_errors():
    h, d_kv, d_k, d_v, d_model = 2, 8, 4, 6, 12
    a, f = oa.absorb_weights(_rand(h, d_kv, d_k, seed=1), _rand(h, d_kv, d_v, seed=2), _rand(h * d_v, d_model, seed=3))
    assert a.shape == (h, d_k, d_kv) and f.shape == (h, d_kv, d_model)
    with pytest.raises(ValueError):
        oa.absorb_weights(np.zeros((2, 8)), np.zeros((2, 8, 6)), np.zeros((12, 16)))
    with pytest.raises(ValueError):
        oa.absorb_weights(np.zeros((2, 8, 4)), np.zeros((3, 8, 6)), np.zeros((12, 16)))
    with pytest.raises(ValueError):
        oa.absorb_weights(np.zeros((2, 8, 4)), np.zeros((2, 8, 6)), np.zeros((10, 16)))


def test_absorbed_equals_standard_decode():
    b, t, h, d_k, d_kv, d_v, d_model, t_kv = 1, 2, 2, 4, 8, 6, 12, 5
    q, c_kv = _rand(b, t, h, d_k, seed=10), _rand(b, t_kv, d_kv, seed=11)
    w_uk, w_uv, w_o = _rand(h, d_kv, d_k, seed=12), _rand(h, d_kv, d_v, seed=13), _rand(h * d_v, d_model, seed=14)
    a, f = oa.absorb_weights(w_uk, w_uv, w_o)
    out_abs = oa.absorbed_mla_decode(q, c_kv, a, f)
    out_std = oa.standard_mla_decode(q, c_kv, w_uk, w_uv, w_o)
    np.testing.assert_allclose(out_abs, out_std, atol=1e-10, rtol=1e-10)
    # what the identity rules out: the untransposed key weight, a head dropped from the output sum
    wrong = oa.absorbed_mla_decode(q, c_kv, np.transpose(a, (0, 1, 2))[:, :, ::-1], f)
    assert np.abs(wrong - out_std).max() > 1e-3
    f_drop = f.copy(); f_drop[1] = 0.0
    assert np.abs(oa.absorbed_mla_decode(q, c_kv, a, f_drop) - out_std).max() > 1e-3


def test_masked_position_drops_out_of_the_softmax():
    b, t, h, d_k, d_kv, d_v, d_model, t_kv = 1, 1, 2, 4, 6, 4, 8, 4
    q, c_kv = _rand(b, t, h, d_k, seed=20), _rand(b, t_kv, d_kv, seed=21)
    w_uk, w_uv, w_o = _rand(h, d_kv, d_k, seed=22), _rand(h, d_kv, d_v, seed=23), _rand(h * d_v, d_model, seed=24)
    a, f = oa.absorb_weights(w_uk, w_uv, w_o)
    mask = np.zeros((b, t, h, t_kv)); mask[..., -1] = -1e9
    out = oa.absorbed_mla_decode(q, c_kv, a, f, mask=mask)
    assert out.shape == (b, t, d_model) and not np.isnan(out).any()
    np.testing.assert_allclose(out, oa.absorbed_mla_decode(q, c_kv[:, :-1], a, f), atol=1e-12)
    with pytest.raises(ValueError):
        oa.absorbed_mla_decode(np.zeros((1, 1, d_k)), c_kv, a, f)
    with pytest.raises(ValueError):
        oa.absorbed_mla_decode(q, c_kv, _rand(h, d_k + 1, d_kv), f)


def test_dequant_block_fp8_against_a_per_element_loop():
    rng = np.random.default_rng(5)
    m, n = 200, 300
    codes = rng.integers(0, 256, (m, n)).astype(np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x3A                       # NaN bytes are outside this check
    scale = rng.uniform(0.5, 1.5, (2, 3)).astype(np.float32)
    got = oa.dequant_block_fp8(codes, scale)
    table = fp8.e4m3_decode(np.arange(256, dtype=np.uint8), np.float32)
    for r, c in [(0, 0), (127, 127), (128, 127), (127, 128), (199, 299), (130, 260), (5, 255), (199, 0)]:
        want = fp8.bf16_round(np.float32(table[codes[r, c]]) * scale[r // 128, c // 128])
        assert got[r, c] == want
    assert got.shape == (m, n)
    with pytest.raises(ValueError):
        oa.dequant_block_fp8(codes, scale[:1])


def test_sanitize_replaces_paired_keys_and_drops_activation_scales():
    rng = np.random.default_rng(6)
    wa, sa = rng.integers(0, 120, (64, 64)).astype(np.uint8), np.ones((1, 1), np.float32) * 0.5
    wb, sb = rng.integers(0, 120, (128, 128)).astype(np.uint8), np.ones((1, 1), np.float32) * 2.0
    other = rng.standard_normal((8, 8)).astype(np.float32)
    weights = {"l0.gate_proj.weight": wa, "l0.gate_proj.weight_scale_inv": sa, "l1.gate_proj.weight": wb,
               "l1.gate_proj.weight_scale_inv": sb, "norm.weight": other, "l0.gate_proj.activation_scale": np.ones(1)}
    out = oa.sanitize_fp8_weights(weights)
    assert set(out) == {"l0.gate_proj.weight", "l1.gate_proj.weight", "norm.weight"}
    np.testing.assert_array_equal(out["l0.gate_proj.weight"], oa.dequant_block_fp8(wa, sa))
    np.testing.assert_array_equal(out["l1.gate_proj.weight"], oa.dequant_block_fp8(wb, sb))
    assert out["norm.weight"] is other
    plain = {"a.weight": other}
    assert oa.sanitize_fp8_weights(plain) == plain and oa.sanitize_fp8_weights(plain) is not plain
