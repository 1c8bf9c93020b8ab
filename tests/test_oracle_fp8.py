"""Pins oracle/fp8.py: the e4m3 / E8M0 codecs every other oracle builds on."""

import json

import numpy as np
import pytest
import torch

from oracle import fp8


@pytest.fixture(scope="module")
def kats(golden_dir):
    return json.loads((golden_dir / "reference_kats.json").read_text())


def test_e4m3_edge_bytes_match_reference_known_answers(kats):
    case = kats["e4m3_edge_bytes"]
    got = fp8.e4m3_decode(np.array(case["bytes"], dtype=np.uint8))
    assert got.tolist() == case["decoded"]
    assert np.isnan(fp8.e4m3_decode(np.array(case["nan_bytes"], dtype=np.uint8))).all()


def test_e4m3_table_matches_torch_decoder_on_all_bytes():
    # torch's float8_e4m3fn decoder is an independent implementation of the same OCP format
    codes = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    got = fp8.e4m3_decode(codes)
    finite = ~np.isnan(want)
    assert finite.sum() == 254
    np.testing.assert_array_equal(got[finite], want[finite])
    assert np.isnan(got[~finite]).all()
    assert np.signbit(got[0x80]) and got[0x80] == 0.0


def test_e4m3_table_structure():
    t = fp8.E4M3_TABLE_F64
    assert t[0x08] == 2.0 ** -6          # smallest normal
    assert t[0x01] == 2.0 ** -9          # smallest subnormal
    assert t[0x38] == 1.0 and t[0x3C] == 1.5
    pos = t[:0x7F]
    assert (np.diff(pos) > 0).all()      # strictly increasing magnitudes
    np.testing.assert_array_equal(t[0x80:0xFF], -pos)


def test_e4m3_on_grid_roundtrip_is_exact(kats):
    vals = np.array(kats["e4m3_on_grid_roundtrip"]["values"], dtype=np.float32)
    np.testing.assert_array_equal(fp8.e4m3_decode(fp8.e4m3_encode(vals)), vals)


def test_e4m3_encode_is_nearest_even_with_saturation():
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.standard_normal(4000) * 30, rng.standard_normal(2000) * 0.01, [1e9, -1e9, 448.0, 464.0, 0.0]])
    codes = fp8.e4m3_encode(x)
    grid = fp8.E4M3_TABLE_F64[~np.isnan(fp8.E4M3_TABLE_F64)]
    clipped = np.clip(x, -448, 448)
    best = np.abs(grid[None, :] - clipped[:, None]).min(axis=1)
    np.testing.assert_allclose(np.abs(fp8.e4m3_decode(codes, np.float64) - clipped), best, rtol=0, atol=0)
    # ties to even, cross-checked against torch's cast on exact midpoints
    mids = (fp8.E4M3_TABLE_F64[1:0x7E] + fp8.E4M3_TABLE_F64[2:0x7F]) / 2
    want = torch.from_numpy(mids.astype(np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    np.testing.assert_array_equal(fp8.e4m3_encode(mids), want)
    assert fp8.e4m3_decode(fp8.e4m3_encode(np.array([1e9])))[0] == 448.0


def test_e8m0_rule(kats):
    case = kats["e8m0_rule"]
    got = fp8.e8m0_decode(np.array(case["bytes"], dtype=np.uint8), np.float64)
    for value, log2 in zip(got, case["decoded_log2"]):
        assert value == (0.0 if log2 is None else 2.0 ** log2)


def test_block_quantiser_roundtrip_error_bound():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((7, 512)).astype(np.float32) * 3
    for pow2 in (True, False):
        codes, scale = fp8.quantize_block(x, 128, pow2=pow2)
        assert codes.shape == x.shape and scale.shape == (7, 4)
        back = fp8.e4m3_decode(codes, np.float64) * np.repeat(scale.astype(np.float64), 128, axis=-1)
        amax = np.abs(x.reshape(7, 4, 128)).max(axis=-1)
        # half an ulp of a 3-bit mantissa relative to the block maximum, doubled for pow2 headroom
        assert (np.abs(back - x).reshape(7, 4, 128).max(axis=-1) <= amax * (2.0 ** -4) * (2 if pow2 else 1) + 1e-12).all()
        if pow2:
            m, _ = np.frexp(scale)
            assert (m == 0.5).all()


def test_bf16_round_matches_torch():
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(10000) * 10).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(fp8.bf16_round(x), want)
