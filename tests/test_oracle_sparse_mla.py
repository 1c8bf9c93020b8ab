"""Pins oracle/sparse_mla.py: loop formulation, closed forms and the invariants the reference tests hold."""

import numpy as np
import pytest
import torch

from oracle import fp8, sparse_mla as om


def _inputs(seed, B=2, S=3, H=4, G=2, Skv=24, topk=8, D=16):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((B, S, H, D))
    kv = rng.standard_normal((B, Skv, G, D))
    idx = rng.integers(0, Skv, (B, S, G, topk))
    return rng, q, kv, idx


@pytest.mark.parametrize("d_v", [16, 12, 4])
def test_batched_oracle_matches_scalar_loop(d_v):
    rng, q, kv, idx = _inputs(1)
    idx[rng.random(idx.shape) < 0.3] = -1
    out, lse = om.sparse_mla_oracle(q, kv, idx, d_v=d_v)
    out2, lse2 = om.sparse_mla_loop_oracle(q, kv, idx, sm_scale=16 ** -0.5, d_v=d_v)
    np.testing.assert_allclose(out, out2, rtol=0, atol=1e-12)
    np.testing.assert_allclose(lse, lse2, rtol=0, atol=1e-12)


def test_full_width_case_reduces_to_torch_softmax_attention():
    _, q, kv, idx = _inputs(2, G=1, H=3)
    out, lse = om.sparse_mla_oracle(q, kv, idx, sm_scale=0.37)
    tq, tkv = torch.from_numpy(q), torch.from_numpy(kv)
    for b in range(q.shape[0]):
        for s in range(q.shape[1]):
            rows = tkv[b, torch.from_numpy(idx[b, s, 0]), 0]            # [topk, D]
            logits = (tq[b, s] @ rows.T) * 0.37                          # [H, topk]
            want = torch.softmax(logits, dim=-1) @ rows
            np.testing.assert_allclose(out[b, s], want.numpy(), atol=1e-12)
            np.testing.assert_allclose(lse[b, s], torch.logsumexp(logits, dim=-1).numpy(), atol=1e-12)


def test_all_invalid_row_gives_exact_zeros_and_zero_lse():
    _, q, kv, idx = _inputs(3)
    idx[0, 1] = -1
    out, lse = om.sparse_mla_oracle(q, kv, idx, d_v=8)
    assert not np.isnan(out).any()
    assert (out[0, 1] == 0).all() and (lse[0, 1] == 0).all()
    assert np.abs(out[0, 0]).max() > 0


def test_out_of_range_index_is_skipped_like_minus_one():
    _, q, kv, idx = _inputs(4)
    a = idx.copy(); a[..., 0] = -1
    b = idx.copy(); b[..., 0] = kv.shape[1] + 5
    np.testing.assert_array_equal(om.sparse_mla_oracle(q, kv, a)[0], om.sparse_mla_oracle(q, kv, b)[0])


def test_permutation_invariance_and_duplicate_weight():
    rng, q, kv, idx = _inputs(5, G=1, H=2)
    out, lse = om.sparse_mla_oracle(q, kv, idx)
    perm = rng.permutation(idx.shape[-1])
    out_p, lse_p = om.sparse_mla_oracle(q, kv, idx[..., perm])
    np.testing.assert_allclose(out, out_p, atol=1e-12)
    np.testing.assert_allclose(lse, lse_p, atol=1e-12)
    # a row listed twice carries twice the weight: {a, a, b} == softmax with logit(a)+ln2
    two = np.array([[[[3, 3, 7]]]]); one = np.array([[[[3, 7]]]])
    o2, _ = om.sparse_mla_oracle(q[:1, :1], kv[:1], two)
    rows = kv[0, [3, 7], 0]
    logits = (q[0, 0] @ rows.T) * (q.shape[-1] ** -0.5) + np.array([np.log(2.0), 0.0])
    w = np.exp(logits - logits.max(-1, keepdims=True)); w /= w.sum(-1, keepdims=True)
    np.testing.assert_allclose(o2[0, 0], w @ rows, atol=1e-12)
    assert not np.allclose(o2, om.sparse_mla_oracle(q[:1, :1], kv[:1], one)[0])


def test_sinks_are_one_extra_logit_with_a_zero_value_row():
    rng, q, kv, idx = _inputs(6, G=1, H=3)
    sinks = rng.standard_normal(3)
    out, lse = om.sparse_mla_oracle(q, kv, idx, sinks=sinks)
    plain, plain_lse = om.sparse_mla_oracle(q, kv, idx)
    # closed form: out = plain * Z/(Z+e^sink), lse = log(Z + e^sink), with Z = e^plain_lse
    z = np.exp(plain_lse)
    np.testing.assert_allclose(lse, np.log(z + np.exp(sinks)[None, None, :]), atol=1e-12)
    np.testing.assert_allclose(out, plain * (z / (z + np.exp(sinks)[None, None, :]))[..., None], atol=1e-12)
    idx2 = idx.copy(); idx2[:] = -1
    out0, lse0 = om.sparse_mla_oracle(q, kv, idx2, sinks=sinks)
    assert (out0 == 0).all()
    np.testing.assert_allclose(lse0, np.broadcast_to(sinks, lse0.shape), atol=1e-12)


def test_dequantisers_apply_scale_per_block():
    rng = np.random.default_rng(7)
    codes = rng.integers(0, 0x7E, (2, 3, 64)).astype(np.uint8)
    e8 = rng.integers(120, 134, (2, 3, 2)).astype(np.uint8)
    got = om.dequant_e8m0(codes, e8)
    for kb in range(2):   # same per-block structure as the reference-held oracle loop
        want = fp8.e4m3_decode(codes[..., kb * 32:(kb + 1) * 32], np.float64) * (2.0 ** (e8[..., kb].astype(int) - 127))[..., None]
        np.testing.assert_array_equal(got[..., kb * 32:(kb + 1) * 32], want)
    tok = rng.random((2, 3)).astype(np.float32)
    np.testing.assert_array_equal(om.dequant_per_token(codes, tok), fp8.e4m3_decode(codes, np.float64) * tok.astype(np.float64)[..., None])
    lat_codes = rng.integers(0, 0x7E, (2, 3, 256)).astype(np.uint8)
    sc = rng.random((2, 3, 2)).astype(np.float32)
    rope = rng.standard_normal((2, 3, 8))
    full = om.dequant_block_latent(lat_codes, sc, rope)
    assert full.shape == (2, 3, 264)
    np.testing.assert_array_equal(full[..., 256:], rope)
    np.testing.assert_array_equal(full[..., 128:256], fp8.e4m3_decode(lat_codes[..., 128:], np.float64) * sc[..., 1:2].astype(np.float64))


def test_shape_validation_messages():
    _, q, kv, idx = _inputs(8)
    with pytest.raises(ValueError, match="q must be 4D"):
        om.sparse_mla_oracle(q[0], kv, idx)
    with pytest.raises(ValueError, match="d_v must be in"):
        om.sparse_mla_oracle(q, kv, idx, d_v=17)
    with pytest.raises(ValueError, match="not divisible by kv_group"):
        om.sparse_mla_oracle(q[:, :, :3], kv, idx)


def _bwd_case(rng, B=1, S=2, H=4, G=2, Skv=9, topk=5, D=6, d_v=4):
    q = rng.standard_normal((B, S, H, D))
    kv = rng.standard_normal((B, Skv, G, D))
    idx = rng.integers(0, Skv, (B, S, G, topk))
    idx[0, 0, 0, 1] = idx[0, 0, 0, 0]          # a repeated key
    idx[0, 1, 1, 2] = -1                       # a skipped slot
    idx[0, 1, 0, 3] = Skv + 2                  # out of range: skipped as well
    d_out = rng.standard_normal((B, S, H, d_v))
    return q, kv, idx, d_out, d_v


def test_backward_oracle_matches_finite_differences_of_the_forward_oracle():
    rng = np.random.default_rng(31)
    q, kv, idx, d_out, d_v = _bwd_case(rng)
    dq, dkv = om.sparse_mla_bwd_oracle(q, kv, idx, d_out, sm_scale=0.37, d_v=d_v)

    def loss(q_, kv_):
        out, _ = om.sparse_mla_oracle(q_, kv_, idx, sm_scale=0.37, d_v=d_v)
        return float((out * d_out).sum())

    eps = 1e-6
    for arr, grad in ((q, dq), (kv, dkv)):
        num = np.zeros_like(arr)
        it = np.nditer(arr, flags=["multi_index"])
        for _ in it:
            i = it.multi_index
            hi, lo = arr.copy(), arr.copy()
            hi[i] += eps
            lo[i] -= eps
            num[i] = (loss(hi, kv) - loss(lo, kv)) / (2 * eps) if arr is q else (loss(q, hi) - loss(q, lo)) / (2 * eps)
        np.testing.assert_allclose(grad, num, atol=1e-7, rtol=1e-6)
    # rows nobody selected get no gradient; a fully skipped query row gives none either
    assert (dkv[0, [i for i in range(9) if i not in set(idx[idx >= 0].ravel().tolist())]] == 0).all()
    idx2 = idx.copy(); idx2[0, 0] = -1
    dq2, _ = om.sparse_mla_bwd_oracle(q, kv, idx2, d_out, sm_scale=0.37, d_v=d_v)
    assert (dq2[0, 0] == 0).all()


def test_backward_oracle_matches_torch_autograd_through_dense_attention():
    rng = np.random.default_rng(32)
    B, S, H, G, Skv, topk, D, d_v = 2, 3, 4, 2, 7, 4, 8, 8
    q = rng.standard_normal((B, S, H, D)); kv = rng.standard_normal((B, Skv, G, D))
    idx = np.stack([np.stack([np.stack([rng.choice(Skv, topk, replace=False) for _ in range(G)]) for _ in range(S)]) for _ in range(B)])
    d_out = rng.standard_normal((B, S, H, d_v))
    dq, dkv = om.sparse_mla_bwd_oracle(q, kv, idx, d_out, d_v=d_v)
    qt = torch.tensor(q, requires_grad=True); kt = torch.tensor(kv, requires_grad=True)
    mask = torch.full((B, S, G, Skv), float("-inf"), dtype=torch.float64)
    mask.scatter_(3, torch.tensor(idx), 0.0)
    kh = kt.repeat_interleave(H // G, dim=2)                                   # [B, Skv, H, D]
    logits = torch.einsum("bshd,bkhd->bshk", qt, kh) * D ** -0.5 + mask.repeat_interleave(H // G, dim=2)
    out = torch.einsum("bshk,bkhd->bshd", torch.softmax(logits, dim=-1), kh[..., :d_v])
    (out * torch.tensor(d_out)).sum().backward()
    np.testing.assert_allclose(dq, qt.grad.numpy(), atol=1e-12, rtol=1e-10)
    np.testing.assert_allclose(dkv, kt.grad.numpy(), atol=1e-12, rtol=1e-10)
