"""DSA indexer KL loss: the HIP kernel against the float64 oracle, and the wrapper's contract
(reference: cppmega_mlx/nn/_tilelang/dsa_splitk_indexer_loss.py:1327-1570).

Tolerance: the kernel accumulates in float32 (dot products, exp, log); against the float64 oracle
on the same (already rounded) inputs the per-position loss agrees to 2e-5 absolute + 2e-4 relative.
"""

import numpy as np
import pytest
import torch

from cppmega_mlx_amd.nn._tilelang.dsa_splitk_indexer_loss import (
    dsa_splitk_indexer_loss_per_position,
    dsa_splitk_indexer_loss_tilelang,
    dsa_splitk_path_c_status,
    tilelang_supports,
)
from oracle import dsa_loss as od

DTYPES = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def _case(seed, ASq, AB, AH, AD, Sk, topk, dtype):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((ASq, AB, AH, AD), generator=g).to(dtype)
    k = torch.randn((Sk, AB, AH, AD), generator=g).to(dtype)
    idx = torch.randn((AB, ASq, Sk), generator=g) * 2.0
    top = torch.stack([torch.stack([torch.randperm(Sk, generator=g)[:topk] for _ in range(ASq)]) for _ in range(AB)])
    return q, k, idx, top


def _want(q, k, idx, top, scale, sparse):
    mask = od.sparse_index_mask(top.numpy(), k.shape[0]) if sparse else None
    return od.dsa_indexer_loss_per_position(idx.numpy(), q.float().numpy(), k.float().numpy(), softmax_scale=scale, index_mask=mask)


def test_cpu_side_checks_need_no_device():
    q = torch.zeros((4, 2, 3, 8)); k = torch.zeros((6, 2, 3, 8)); idx = torch.zeros((2, 4, 6)); top = torch.zeros((2, 4, 2), dtype=torch.int64)
    with pytest.raises(ValueError, match="query/key shape mismatch"):
        dsa_splitk_indexer_loss_tilelang(idx, top, q, k[:, :, :2], 1.0, 1.0, False)
    zero = dsa_splitk_indexer_loss_tilelang(idx[:, :0], top[:, :0], q[:0], k, 1.0, 1.0, True)
    assert zero.shape == () and zero.dtype == torch.float32 and float(zero) == 0.0
    assert float(dsa_splitk_indexer_loss_tilelang(idx[:, :, :0], top, q, k[:0], 1.0, 1.0, False)) == 0.0
    with pytest.raises(ValueError, match="AH > 128"):
        dsa_splitk_indexer_loss_tilelang(torch.zeros((1, 2, 2)), None, torch.zeros((2, 1, 129, 4)), torch.zeros((2, 1, 129, 4)), 1.0, 1.0, False)
    with pytest.raises(TypeError, match="dtypes must match"):
        dsa_splitk_indexer_loss_tilelang(idx, top, q, k.half(), 1.0, 1.0, False)
    with pytest.raises(TypeError, match="unsupported Q/K dtype"):
        dsa_splitk_indexer_loss_tilelang(idx, top, q.double(), k.double(), 1.0, 1.0, False)
    with pytest.raises(ValueError, match="unsupported device type"):
        dsa_splitk_indexer_loss_tilelang(idx, top, q, k, 1.0, 1.0, False)
    assert tilelang_supports(None) is False and tilelang_supports("cpu") is False
    assert isinstance(dsa_splitk_path_c_status().reason, str)


@pytest.mark.gpu
@pytest.mark.parametrize("sparse", [False, True])
@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("shape", [(5, 1, 2, 8, 5, 3), (33, 2, 4, 64, 33, 7), (17, 3, 3, 20, 40, 9), (40, 1, 8, 128, 24, 24), (300, 1, 2, 32, 300, 64)])
def test_per_position_loss_matches_the_oracle(shape, dt, sparse):
    ASq, AB, AH, AD, Sk, topk = shape
    q, k, idx, top = _case(11 + ASq, ASq, AB, AH, AD, Sk, topk, DTYPES[dt])
    scale = AD ** -0.5
    got = dsa_splitk_indexer_loss_per_position(idx.cuda(), top.cuda(), q.cuda(), k.cuda(), scale, sparse).cpu().numpy()
    want = _want(q, k, idx, top, scale, sparse)
    assert np.isfinite(got).all()
    np.testing.assert_allclose(got, want, atol=2e-5, rtol=2e-4)


@pytest.mark.gpu
def test_closed_forms_on_the_device():
    ASq, AB, AH, AD, Sk = 9, 2, 3, 16, 12
    z = lambda *s: torch.zeros(s, device="cuda")
    got = dsa_splitk_indexer_loss_per_position(z(AB, ASq, Sk), None, z(ASq, AB, AH, AD), z(Sk, AB, AH, AD), 0.5, False).cpu().numpy()
    want = np.log(Sk) - np.log(np.arange(1, ASq + 1))
    np.testing.assert_allclose(got, np.broadcast_to(want, (AB, ASq)), atol=1e-5)


@pytest.mark.gpu
def test_wrapper_contract_on_the_device():
    ASq, AB, AH, AD, Sk, topk = 24, 2, 4, 32, 24, 6
    q, k, idx, top = _case(5, ASq, AB, AH, AD, Sk, topk, torch.bfloat16)
    qd, kd, idxd, topd = q.cuda(), k.cuda(), idx.cuda(), top.cuda()
    for sparse in (False, True):
        got = dsa_splitk_indexer_loss_tilelang(idxd, topd, qd, kd, 0.2, 0.37, sparse)
        assert got.shape == () and got.dtype == torch.float32
        want = _want(q, k, idx, top, 0.2, sparse).mean() * 0.37
        assert abs(float(got) - want) < 2e-5 + 2e-4 * abs(want)
    # int32 lists, non-contiguous inputs and non-float32 index scores are taken as the reference takes them
    a = dsa_splitk_indexer_loss_tilelang(idxd, topd.int(), qd, kd, 0.2, 1.0, True)
    b = dsa_splitk_indexer_loss_tilelang(idxd.double(), topd, qd.transpose(0, 1).contiguous().transpose(0, 1), kd, 0.2, 1.0, True)
    c = dsa_splitk_indexer_loss_tilelang(idxd, topd, qd, kd, 0.2, 1.0, True)
    assert float(a) == float(c) == float(b)
    # duplicates in a list select the key once
    dup = topd.clone(); dup[..., 1] = dup[..., 0]
    want_dup = _want(q, k, idx, dup.cpu(), 0.2, True).mean()
    assert abs(float(dsa_splitk_indexer_loss_tilelang(idxd, dup, qd, kd, 0.2, 1.0, True)) - want_dup) < 1e-4
    with pytest.raises(ValueError, match="out of range"):
        bad = topd.clone(); bad[0, 0, 0] = Sk
        dsa_splitk_indexer_loss_tilelang(idxd, bad, qd, kd, 0.2, 1.0, True)
    with pytest.raises(ValueError, match="out of range"):
        bad = topd.clone(); bad[1, 3, 2] = -1
        dsa_splitk_indexer_loss_tilelang(idxd, bad, qd, kd, 0.2, 1.0, True)
    with pytest.raises(ValueError, match="TOPK"):
        dsa_splitk_indexer_loss_tilelang(idxd, topd[:, :, :0], qd, kd, 0.2, 1.0, True)
    with pytest.raises(ValueError, match="must have shape"):
        dsa_splitk_indexer_loss_tilelang(idxd, topd[:, :-1], qd, kd, 0.2, 1.0, True)
    with pytest.raises(TypeError, match="int32 or int64"):
        dsa_splitk_indexer_loss_tilelang(idxd, topd.float(), qd, kd, 0.2, 1.0, True)
    with pytest.raises(ValueError, match="device"):
        dsa_splitk_indexer_loss_tilelang(idxd, top, qd, kd, 0.2, 1.0, True)
    assert tilelang_supports("cuda") and dsa_splitk_path_c_status().available


@pytest.mark.gpu
def test_long_rows_use_the_large_lds_window():
    ASq, AB, AH, AD, Sk, topk = 6, 1, 2, 64, 9000, 512
    q, k, idx, top = _case(9, ASq, AB, AH, AD, Sk, topk, torch.bfloat16)
    # query positions near the end of a long context: rows see thousands of keys
    qpos = Sk - ASq
    qfull = torch.zeros((Sk, AB, AH, AD), dtype=torch.bfloat16); qfull[qpos:] = q
    idxfull = torch.zeros((AB, Sk, Sk)); idxfull[:, qpos:] = idx
    topfull = torch.zeros((AB, Sk, topk), dtype=torch.int64); topfull[:, qpos:] = top
    got = dsa_splitk_indexer_loss_per_position(idxfull.cuda(), topfull.cuda(), qfull.cuda(), k.cuda(), 0.125, True)[:, qpos:].cpu().numpy()
    mask = od.sparse_index_mask(top.numpy(), Sk)
    want = np.zeros((AB, ASq))
    for i in range(ASq):                       # query position qpos + i sees keys 0 .. qpos + i
        for b in range(AB):
            want[b, i] = od.row_loss(idx.double().numpy()[b, i], q.double().numpy()[i, b], k.double().numpy()[:, b], qpos + i + 1, 0.125, mask[b, i])
    np.testing.assert_allclose(got, want, atol=2e-5, rtol=2e-4)


@pytest.mark.gpu
def test_bench_size_properties():
    """At the size the bench times (4096 positions, 8 heads of 64): the closed form for zero rows and a uniform index,
    and non-negativity / finiteness of the divergence for random rows, dense and sparse."""
    ASq = Sk = 4096
    AB, AH, AD, topk = 1, 8, 64, 1024
    z = lambda *s: torch.zeros(s, device="cuda", dtype=torch.bfloat16)
    got = dsa_splitk_indexer_loss_per_position(torch.zeros((AB, ASq, Sk), device="cuda"), None, z(ASq, AB, AH, AD), z(Sk, AB, AH, AD),
                                               0.125, False).cpu().numpy()
    want = np.log(Sk) - np.log(np.arange(1, ASq + 1))
    np.testing.assert_allclose(got[0], want, atol=2e-5, rtol=2e-4)
    g = torch.Generator(device="cuda").manual_seed(3)
    q = torch.randn((ASq, AB, AH, AD), generator=g, device="cuda").to(torch.bfloat16)
    k = torch.randn((Sk, AB, AH, AD), generator=g, device="cuda").to(torch.bfloat16)
    idx = torch.randn((AB, ASq, Sk), generator=g, device="cuda")
    top = torch.topk(idx, topk, dim=-1).indices
    for sparse in (False, True):
        loss = dsa_splitk_indexer_loss_per_position(idx, top, q, k, AD ** -0.5, sparse)
        assert torch.isfinite(loss).all() and (loss >= -1e-4).all()       # a divergence of p against a sub-normalised q
    # a few rows against the float64 oracle row function
    mask = None
    for sq in (0, 17, 2047, 4095):
        w = od.row_loss(idx[0, sq].double().cpu().numpy(), q[sq, 0].double().cpu().numpy(), k[:, 0].double().cpu().numpy(), sq + 1,
                        AD ** -0.5, mask)
        d = float(dsa_splitk_indexer_loss_per_position(idx, top, q, k, AD ** -0.5, False)[0, sq])
        assert abs(d - w) <= 2e-5 + 2e-4 * abs(w), (sq, d, w)
