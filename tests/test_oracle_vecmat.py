"""Pins oracle/vecmat.py against float64 matmuls over torch's independent e4m3 decoder."""

import numpy as np
import pytest
import torch

from oracle import fp8, vecmat


def _torch_decode(codes):
    return torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float64).numpy()


def test_reference_shaped_vecmat_matches_dequant_matmul():
    rng = np.random.default_rng(0)
    N, K = 37, 64
    w = rng.integers(0, 0x7E, (N, K)).astype(np.uint8) | (rng.integers(0, 2, (N, K)).astype(np.uint8) << 7)
    x = rng.integers(0, 0x7E, K).astype(np.uint8)
    sw = rng.random(N).astype(np.float32) + 0.5
    got = vecmat.fp8_scaled_vecmat_oracle(x, w, scale_x=0.25, scale_w=sw)
    want = (_torch_decode(w) @ _torch_decode(x)) * 0.25 * sw.astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=1e-15)
    got1 = vecmat.fp8_scaled_vecmat_oracle(x, w, scale_x=np.array([0.25]), scale_w=np.array([2.0]))
    np.testing.assert_allclose(got1, (_torch_decode(w) @ _torch_decode(x)) * 0.5, rtol=1e-15)


def test_vecmat_validation():
    w = np.zeros((4, 8), np.uint8)
    with pytest.raises(ValueError, match="expects 1D x and 2D W"):
        vecmat.fp8_scaled_vecmat_oracle(np.zeros((1, 8), np.uint8), w, scale_x=1.0, scale_w=1.0)
    with pytest.raises(ValueError, match="shape mismatch"):
        vecmat.fp8_scaled_vecmat_oracle(np.zeros(12, np.uint8), w, scale_x=1.0, scale_w=1.0)
    with pytest.raises(ValueError, match="multiple of 4"):
        vecmat.fp8_scaled_vecmat_oracle(np.zeros(6, np.uint8), np.zeros((4, 6), np.uint8), scale_x=1.0, scale_w=1.0)
    with pytest.raises(ValueError, match="scale_w"):
        vecmat.fp8_scaled_vecmat_oracle(np.zeros(8, np.uint8), w, scale_x=1.0, scale_w=np.ones(3))


def test_block128_gemm_grid_and_row_block_scales_agree():
    rng = np.random.default_rng(1)
    N, K, M = 200, 384, 3
    w = rng.integers(0, 0x7E, (N, K)).astype(np.uint8)
    grid = rng.random((2, 3)).astype(np.float32) + 0.5
    a = rng.standard_normal((M, K))
    got = vecmat.fused_fp8_gemm_oracle(w, grid, a)
    dense = _torch_decode(w) * np.repeat(np.repeat(grid.astype(np.float64), 128, 0)[:N], 128, 1)
    np.testing.assert_allclose(got, a @ dense.T, rtol=1e-14)
    rows = np.repeat(grid, 128, 0)[:N]
    np.testing.assert_array_equal(vecmat.fused_fp8_gemm_oracle(w, rows, a), got)
    with pytest.raises(ValueError, match="scale shape"):
        vecmat.fused_fp8_gemm_oracle(w, grid[:1], a)


def test_linearity_in_the_activation():
    rng = np.random.default_rng(2)
    w, sc = fp8.quantize_block(rng.standard_normal((16, 256)).astype(np.float32))
    a, b = rng.standard_normal((2, 256))
    f = lambda v: vecmat.fused_fp8_gemm_oracle(w, sc, v)
    np.testing.assert_allclose(f(2 * a - 3 * b), 2 * f(a) - 3 * f(b), atol=1e-10)
