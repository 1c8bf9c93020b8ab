"""The float32 torch restatement bench.py times on the host (oracle/torch_cpu.py) against the
float64 NumPy oracle."""

import numpy as np
import torch

from oracle import fp8, sparse_mla as om, topk as ot, torch_cpu, vecmat as ov
from tests._inputs import sparse_indices


def test_sparse_mla_fallback_matches_the_oracle():
    rng = np.random.default_rng(3)
    B, S, H, G, Skv, topk, D, d_v = 2, 5, 8, 2, 40, 12, 32, 24
    q = rng.standard_normal((B, S, H, D)).astype(np.float32)
    kv = rng.standard_normal((B, Skv, G, D)).astype(np.float32)
    idx = sparse_indices(rng, B, S, G, Skv, topk, causal_offset=3)
    idx[0, 0] = -1                                              # an all-invalid row
    want, want_lse = om.sparse_mla_oracle(q, kv, idx, d_v=d_v)
    got, got_lse = torch_cpu.sparse_mla_fallback(torch.from_numpy(q), torch.from_numpy(kv), torch.from_numpy(idx.astype(np.int64)),
                                                 d_v=d_v, chunk=2)
    np.testing.assert_allclose(got.numpy(), want, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(got_lse.numpy(), want_lse, rtol=1e-5, atol=1e-6)
    assert not got[0, 0].any() and not got_lse[0, 0].any()


def test_topk_fallback_matches_the_oracle():
    rng = np.random.default_rng(4)
    s = rng.standard_normal((9, 64)).astype(np.float32)
    s[:, ::7] = s[:, 1:2]                                       # exact ties
    ends = rng.integers(0, 65, size=9).astype(np.int32)
    want = ot.topk_selector_oracle(s, 16, ends=ends)
    got = torch_cpu.topk_fallback(torch.from_numpy(s), 16, ends=torch.from_numpy(ends)).numpy()
    np.testing.assert_array_equal(got, want)


def test_fused_fp8_gemm_fallback_matches_the_oracle():
    rng = np.random.default_rng(5)
    codes, scale = fp8.quantize_block(rng.standard_normal((24, 256)).astype(np.float32), 128, pow2=False)
    x = rng.standard_normal((3, 256)).astype(np.float32)
    want = ov.fused_fp8_gemm_oracle(codes, scale, x)
    got = torch_cpu.fused_fp8_gemm_fallback(torch.from_numpy(fp8.e4m3_decode(codes)), torch.from_numpy(scale), torch.from_numpy(x))
    np.testing.assert_allclose(got.numpy(), want, rtol=2e-5, atol=1e-4)
