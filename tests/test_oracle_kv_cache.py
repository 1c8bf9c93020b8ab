"""Pins oracle/kv_cache.py: the sparse index producers and the block-scaled cache producer."""

import json

import numpy as np
import pytest

from oracle import fp8, kv_cache as okv


@pytest.fixture(scope="module")
def kats(golden_dir):
    return json.loads((golden_dir / "reference_kats.json").read_text())


def test_causal_indices_match_reference_known_answer(kats):
    case = kats["causal_sparse_indices"]
    got = okv.causal_sparse_indices(**case["args"])
    assert got.shape == (2, 5, 2, 3) and got.dtype == np.int32
    assert got[0, :, 0, :].tolist() == case["expected_b0_g0"]
    assert (got == got[:1, :, :1, :]).all()            # broadcast over batch and group


def test_causal_indices_brute_force_with_offset_and_short_key_length():
    got = okv.causal_sparse_indices(1, 6, 1, 5, query_offset=3, key_length=7)
    for s in range(6):
        for j in range(5):
            pos = 3 + s - j
            assert got[0, s, 0, j] == (pos if 0 <= pos < 7 else -1)


def test_mask_indices_match_reference_known_answer(kats):
    case = kats["sparse_indices_from_attention_mask"]
    got = okv.sparse_indices_from_attention_mask(np.array(case["mask"], dtype=np.bool_), **case["args"])
    assert got.shape == (1, 3, 2, 2)
    assert np.sort(got[0, :, 0, :], axis=-1).tolist() == case["expected_sorted_b0_g0"]
    np.testing.assert_array_equal(got[:, :, 0], got[:, :, 1])


def test_mask_indices_brute_force_newest_valid_keys():
    rng = np.random.default_rng(5)
    for K, topk in ((9, 4), (40, 7), (5, 8), (64, 64)):
        mask = rng.random((2, 3, K)) < 0.4
        mask[0, 0] = False                               # a row with nothing valid
        mask[1, 2] = True                                # a row with everything valid
        got = okv.sparse_indices_from_attention_mask(mask, batch_size=2, seq_length=3, kv_group=1, topk=topk, key_length=K)
        n = min(topk, K)
        assert got.shape == (2, 3, 1, n)
        for b in range(2):
            for s in range(3):
                valid = [k for k in range(K) if mask[b, s, k]]
                newest = valid[-n:]
                want = [-1] * (n - len(newest)) + newest      # ascending, right-aligned
                assert got[b, s, 0].tolist() == want


def test_mask_indices_float_masks_use_finiteness():
    m = np.array([[0.0, -np.inf, 1.5, np.inf, np.nan, -2.0]], dtype=np.float32)
    got = okv.sparse_indices_from_attention_mask(m, batch_size=1, seq_length=1, kv_group=1, topk=4, key_length=6)
    assert got[0, 0, 0].tolist() == [-1, 0, 2, 5]


def test_block128_quantiser_closed_forms():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((3, 4, 256)).astype(np.float32) * np.float32(3.0)
    x[0, 0, :128] = 0.0                                   # an all-zero block
    for pow2 in (False, True):
        codes, scale = okv.quantize_block128(x, pow2=pow2)
        assert codes.shape == x.shape and scale.shape == (3, 4, 2)
        dec = fp8.e4m3_decode(codes).reshape(3, 4, 2, 128) * scale[..., None]
        xb = x.reshape(3, 4, 2, 128)
        amax = np.abs(xb).max(-1)
        # the largest element of a block maps to within one e4m3 step of itself; 448 is never exceeded
        assert (np.abs(fp8.e4m3_decode(codes)) <= 448).all()
        assert np.abs(dec - xb).max() <= 2.0 ** -4 * amax.max() + 1e-12
        if pow2:
            nz = amax > 0
            assert (np.log2(scale[nz]) % 1 == 0).all()
            assert (448.0 * scale[nz] >= amax[nz]).all() and (448.0 * scale[nz] / 2 < amax[nz]).all()
            assert (scale[~nz] == 1.0).all() and (codes.reshape(3, 4, 2, 128)[~nz] == 0).all()
        else:
            np.testing.assert_array_equal(scale, np.maximum(amax * np.float32(1 / 448), np.float32(1e-12)))
    # per block it is the per-token producer applied to the block
    codes, scale = okv.quantize_block128(x, pow2=False)
    c2, s2 = fp8.quantize_per_token(x.reshape(3, 4, 2, 128))
    np.testing.assert_array_equal(codes.reshape(3, 4, 2, 128), c2)
    np.testing.assert_array_equal(scale, s2)
    # values on the grid survive exactly with a power-of-two scale
    grid = fp8.e4m3_decode(np.arange(0, 0x7F, dtype=np.uint8)).astype(np.float32)
    row = np.resize(grid, 128)[None] * np.float32(0.25)
    codes, scale = okv.quantize_block128(row, pow2=True)
    np.testing.assert_array_equal(fp8.e4m3_decode(codes) * scale[..., None].repeat(128, -1).reshape(row.shape), row)


def test_append_places_rows_at_positions():
    kv = np.zeros((2, 6, 1, 4), np.uint8)
    sc = np.zeros((2, 6, 1), np.float32)
    new = np.arange(2 * 2 * 4, dtype=np.uint8).reshape(2, 2, 1, 4) + 1
    okv.append(kv, sc, np.array([1, 3]), new, np.ones((2, 2, 1), np.float32))
    assert kv[0, 1:3].tolist() == new[0].tolist() and kv[1, 3:5].tolist() == new[1].tolist()
    assert kv[0, 0].sum() == 0 and kv[0, 3:].sum() == 0 and sc.sum() == 4
