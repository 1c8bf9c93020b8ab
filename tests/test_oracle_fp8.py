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


def test_producer_quantisers_closed_forms():
    """Scales and codes of the producer restatements on inputs whose answer is known in closed form."""
    x = np.zeros((3, 64), dtype=np.float32)
    x[0, :4] = [448.0, -224.0, 1.0, 0.0]          # amax 448 -> scale 1 -> codes are the values' own bytes
    x[1, :2] = [2.0, -1.0]                        # amax 2 -> scale 2/448; 2 -> 448 (0x7E), -1 -> -224 (0xF6)
    codes, scale = fp8.quantize_per_token(x)
    assert scale[0] == np.float32(448.0) * np.float32(1.0 / 448.0)
    assert list(codes[0, :4]) == [0x7E, 0xF6, 0x38, 0x00]
    assert list(codes[1, :2]) == [0x7E, 0xF6]
    assert scale[2] == np.float32(1e-12) and not codes[2].any()      # all-zero row: floor scale, zero bytes
    tcodes, tscale = fp8.quantize_per_tensor(x)
    assert (tscale == tscale.flat[0]).all() and tscale.shape == (3,)
    assert list(tcodes[1, :2]) == [0x40, 0xB8]    # with the tensor amax 448: 2 -> 0x40, -1 -> 0xB8
    # the round trip is a projection: quantising it again changes nothing
    rng = np.random.default_rng(0)
    y = rng.standard_normal((5, 96)).astype(np.float32)
    r = fp8.roundtrip_per_tensor(y)
    np.testing.assert_array_equal(fp8.roundtrip_per_tensor(r), r)
    assert np.abs(r - y).max() <= np.abs(y).max() / 448.0 * 16.0      # half an ulp of the top binade (ulp 32 at 448)
    # MXFP8: the block exponent is log2(amax / 448) rounded to nearest; what exceeds 448 * 2^e saturates
    z = np.zeros((1, 128), dtype=np.float32)
    z[0, 0] = 448.0
    z[0, 32] = 448.0 * 2.0 ** -5
    z[0, 64] = np.nextafter(np.float32(448.0), np.float32(1e9))
    z[0, 96] = 448.0 * 1.5                                            # log2(1.5) = 0.585 -> exponent 1
    mcodes, mbytes = fp8.quantize_mxfp8(z)
    assert list(mbytes[0]) == [127, 122, 127, 128]
    assert mcodes[0, 0] == 0x7E and mcodes[0, 32] == 0x7E and mcodes[0, 64] == 0x7E   # 448.00003 saturates
    assert mcodes[0, 96] == 0x7A                                      # 672 / 2 = 336 -> rne to 320 (1.25 * 2^8)
    rm = fp8.roundtrip_mxfp8(y)
    np.testing.assert_array_equal(fp8.roundtrip_mxfp8(rm), rm)
