"""GPU parity: the float-carrier sparse-MLA backward (through the C ABI) vs the float64 oracle.

dkv is accumulated with float32 atomic adds, so results agree to rounding, not bit for bit:
float32 carriers are held to 1e-4 of each gradient's scale, half carriers to 2e-2 for dq (one
rounding of the result) and 1e-2 for the float32 dkv (inputs are already rounded; the oracle
sees the same values)."""

import numpy as np
import pytest
import torch

from cppmega_mlx_amd import ops
from cppmega_mlx_amd.nn._tilelang import sparse_mla_path_c as pc
from oracle import sparse_mla as om
from tests._inputs import error_report, sparse_indices, to_dev

pytestmark = pytest.mark.gpu

CASES = [
    dict(B=1, S=4, H=4, G=1, Skv=32, topk=8, D=64, d_v=64),
    dict(B=2, S=5, H=8, G=2, Skv=64, topk=16, D=64, d_v=48),
    dict(B=1, S=3, H=6, G=3, Skv=300, topk=100, D=128, d_v=32),
    dict(B=1, S=2, H=16, G=1, Skv=256, topk=64, D=576, d_v=512),       # the tiny bf16 configuration's widths
    dict(B=1, S=2, H=2, G=1, Skv=50, topk=37, D=20, d_v=7),
]


@pytest.mark.parametrize("shape", CASES, ids=lambda c: "B%dS%dH%dG%dT%dk%dD%ddv%d" % tuple(c.values()))
@pytest.mark.parametrize("carrier", [torch.float32, torch.bfloat16, torch.float16])
def test_backward_matches_oracle(device, shape, carrier):
    B, S, H, G, Skv, topk, D, d_v = shape.values()
    rng = np.random.default_rng(B * 100 + S * 10 + D)
    qt = to_dev(rng.standard_normal((B, S, H, D)).astype(np.float32), device).to(carrier)
    kt = to_dev(rng.standard_normal((B, Skv, G, D)).astype(np.float32), device).to(carrier)
    dt = to_dev(rng.standard_normal((B, S, H, d_v)).astype(np.float32), device).to(carrier)
    idx = sparse_indices(rng, B, S, G, Skv, topk, replace=True)      # repeated keys accumulate
    idx[rng.random(idx.shape) < 0.2] = -1
    idx[0, 1] = -1                                                   # a query with nothing to attend to
    idx[0, 0, 0, 0] = Skv + 5                                        # out of range: skipped
    want_dq, want_dkv = om.sparse_mla_bwd_oracle(qt.double().cpu().numpy(), kt.double().cpu().numpy(), idx,
                                                 dt.double().cpu().numpy(), sm_scale=D ** -0.5, d_v=d_v)
    dq = torch.full((B, S, H, D), 9.0, dtype=carrier, device=device)
    dkv = torch.full((B, Skv, G, D), 9.0, dtype=torch.float32, device=device)
    got = ops.sparse_mla_backward(qt, kt, dt, to_dev(idx.astype(np.int32), device), sm_scale=D ** -0.5, d_v=d_v, dq=dq, dkv=dkv)
    torch.cuda.synchronize()
    assert got[0] is dq and got[1] is dkv
    half = carrier != torch.float32
    err, ref = error_report(dq.float().cpu().numpy(), want_dq)
    assert err <= (2e-2 if half else 1e-4) * ref, (err, ref)
    err, ref = error_report(dkv.cpu().numpy(), want_dkv)
    assert err <= 1e-4 * ref, (err, ref)
    assert (dq[0, 1] == 0).all()
    # accumulate on top of existing contents when asked not to clear
    ops.sparse_mla_backward(qt, kt, dt, to_dev(idx, device), sm_scale=torch.tensor([D ** -0.5], device=device), d_v=d_v, dq=dq, dkv=dkv,
                            clear_dkv=False)
    torch.cuda.synchronize()
    err, ref = error_report(dkv.cpu().numpy(), 2 * want_dkv)
    assert err <= 2e-4 * ref


MATRIX_CORE_CASES = [
    dict(B=1, S=3, H=16, G=1, Skv=256, topk=100, D=576, d_v=512),      # one chunk of 16 heads, a partial last tile
    dict(B=1, S=2, H=40, G=1, Skv=300, topk=70, D=576, d_v=512),       # chunks of 32 heads, the second one with 8
    dict(B=2, S=3, H=24, G=2, Skv=200, topk=130, D=128, d_v=64),       # 12 heads per group, three tiles
    dict(B=1, S=4, H=64, G=1, Skv=64, topk=33, D=64, d_v=64),          # d_v == d_qk
    dict(B=1, S=2, H=1, G=1, Skv=40, topk=5, D=96, d_v=32),            # a single head
    dict(B=1, S=2, H=128, G=1, Skv=512, topk=256, D=576, d_v=512),     # the production head count
]


@pytest.mark.parametrize("shape", MATRIX_CORE_CASES, ids=lambda c: "B%dS%dH%dG%dT%dk%dD%ddv%d" % tuple(c.values()))
@pytest.mark.parametrize("index_dtype", [np.int32, np.int64])
@pytest.mark.parametrize("carrier", [torch.bfloat16, torch.float16])
def test_bfloat16_backward_on_the_matrix_cores(device, shape, index_dtype, carrier):
    """bfloat16 (or float16: the reference kernel's own carrier) q / kv / d_out take the matrix-core kernel; with
    float32 dq both gradients are held to 1e-4 of their scale (P and dS enter the second products as hi + lo planes)."""
    B, S, H, G, Skv, topk, D, d_v = shape.values()
    rng = np.random.default_rng(B * 1000 + H * 10 + topk)
    qt = to_dev(rng.standard_normal((B, S, H, D)).astype(np.float32), device).to(carrier)
    kt = to_dev(rng.standard_normal((B, Skv, G, D)).astype(np.float32), device).to(carrier)
    dt = to_dev(rng.standard_normal((B, S, H, d_v)).astype(np.float32), device).to(carrier)
    idx = sparse_indices(rng, B, S, G, Skv, topk, replace=True)
    idx[rng.random(idx.shape) < 0.15] = -1
    idx[0, 1] = -1
    idx[0, 0, 0, 0] = Skv + 5
    sm = 1.7 * D ** -0.5
    want_dq, want_dkv = om.sparse_mla_bwd_oracle(qt.double().cpu().numpy(), kt.double().cpu().numpy(), idx,
                                                 dt.double().cpu().numpy(), sm_scale=sm, d_v=d_v)
    dq = torch.full((B, S, H, D), 9.0, dtype=torch.float32, device=device)
    dkv = torch.full((B, Skv, G, D), 9.0, dtype=torch.float32, device=device)
    ops.sparse_mla_backward(qt, kt, dt, to_dev(idx.astype(index_dtype), device), sm_scale=sm, d_v=d_v, dq=dq, dkv=dkv)
    torch.cuda.synchronize()
    for got, want in ((dq, want_dq), (dkv, want_dkv)):
        err, ref = error_report(got.cpu().numpy(), want)
        assert err <= 1e-4 * ref, (err, ref)
    assert (dq[0, 1] == 0).all()
    # dq in the carrier: one rounding of the same values
    dq16 = torch.empty((B, S, H, D), dtype=carrier, device=device)
    ops.sparse_mla_backward(qt, kt, dt, to_dev(idx.astype(index_dtype), device), sm_scale=torch.tensor([sm], device=device), d_v=d_v,
                            dq=dq16, dkv=dkv)
    torch.cuda.synchronize()
    assert torch.equal(dq16, dq.to(carrier))


@pytest.mark.parametrize("shape", [
    dict(B=2, S=3, H=8, G=2, Skv=120, topk=70, D=64, d_v=32),
    dict(B=1, S=2, H=48, G=1, Skv=300, topk=45, D=576, d_v=512),
    dict(B=1, S=3, H=16, G=1, Skv=200, topk=130, D=128, d_v=128),
], ids=lambda c: "B%dS%dH%dG%dT%dk%dD%ddv%d" % tuple(c.values()))
@pytest.mark.parametrize("cotangent", [torch.bfloat16, torch.float16])
def test_per_token_fp8_backward_on_the_matrix_cores(device, shape, cotangent):
    """e4m3 q / kv with per-token scales and a bfloat16 cotangent take the matrix-core kernel: the code
    values are exact in bfloat16 and the scales are applied in fp32, so the 1e-4 bar of the fp32 kernel holds."""
    from cppmega_mlx_amd.nn._tilelang import sparse_mla_fp8_path_c as f8
    from oracle import fp8

    B, S, H, G, Skv, topk, D, d_v = shape.values()
    rng = np.random.default_rng(H * 100 + topk)
    qc, qs = fp8.quantize_per_token((rng.standard_normal((B * S * H, D)) * rng.uniform(0.2, 3.0, (B * S * H, 1))).astype(np.float32))
    kc, ks = fp8.quantize_per_token((rng.standard_normal((B * Skv * G, D)) * rng.uniform(0.2, 3.0, (B * Skv * G, 1))).astype(np.float32))
    qc, qs, kc, ks = qc.reshape(B, S, H, D), qs.reshape(B, S, H), kc.reshape(B, Skv, G, D), ks.reshape(B, Skv, G)
    d_out = to_dev(rng.standard_normal((B, S, H, d_v)).astype(np.float32), device).to(cotangent)
    idx = sparse_indices(rng, B, S, G, Skv, topk, replace=True)
    idx[rng.random(idx.shape) < 0.15] = -1
    idx[0, 1] = -1
    idx[0, 0, 0, :2] = Skv + 1
    sm = 0.9 * D ** -0.5
    want_dq, want_dkv = om.sparse_mla_bwd_oracle(om.dequant_per_token(qc, qs), om.dequant_per_token(kc, ks), idx,
                                                 d_out.double().cpu().numpy(), sm_scale=sm, d_v=d_v)
    dq, dkv = f8.sparse_mla_fp8_bwd_path_c(to_dev(qc, device), to_dev(qs, device), to_dev(kc, device), to_dev(ks, device), d_out,
                                           to_dev(idx.astype(np.int32), device), sm_scale=sm, d_v=d_v)
    torch.cuda.synchronize()
    for got, want in ((dq, want_dq), (dkv, want_dkv)):
        assert got.dtype == torch.float32
        err, ref = error_report(got.cpu().numpy(), want)
        assert err <= 1e-4 * ref, (err, ref)
    assert (dq[0, 1] == 0).all()


def test_public_backward_entry_points_and_autograd(device):
    rng = np.random.default_rng(8)
    B, S, H, G, Skv, topk, D = 2, 4, 4, 2, 48, 12, 64
    q = to_dev(rng.standard_normal((B, S, H, D)).astype(np.float32), device)
    kv = to_dev(rng.standard_normal((B, Skv, G, D)).astype(np.float32), device)
    d_out = to_dev(rng.standard_normal((B, S, H, D)).astype(np.float32), device)
    idx = sparse_indices(rng, B, S, G, Skv, topk)
    idx[..., -2:] = -1
    it = to_dev(idx, device)
    want_dq, want_dkv = om.sparse_mla_bwd_oracle(q.cpu().numpy(), kv.cpu().numpy(), idx, d_out.cpu().numpy())
    dq, dkv = pc.sparse_mla_bwd_path_c(q, kv, d_out, it)
    torch.cuda.synchronize()
    assert dq.dtype == torch.float32 and dkv.dtype == torch.float32
    np.testing.assert_allclose(dq.cpu().numpy(), want_dq, atol=1e-4 * np.abs(want_dq).max())
    np.testing.assert_allclose(dkv.cpu().numpy(), want_dkv, atol=1e-4 * np.abs(want_dkv).max())
    qa, ka = q.clone().requires_grad_(True), kv.clone().requires_grad_(True)
    out = pc.sparse_mla_path_c_metal_apply(qa, ka, it)
    (out * d_out).sum().backward()
    torch.cuda.synchronize()
    np.testing.assert_allclose(qa.grad.cpu().numpy(), want_dq, atol=1e-4 * np.abs(want_dq).max())
    np.testing.assert_allclose(ka.grad.cpu().numpy(), want_dkv, atol=1e-4 * np.abs(want_dkv).max())
    with pytest.raises(pc.SparseMLAPathCDirectError):
        pc._sparse_mla_bwd_path_c_direct(q, kv.half(), d_out, it, sm_scale_buf=torch.tensor([0.1], device=device))
    with pytest.raises(ValueError):
        ops.sparse_mla_backward(q, kv, d_out, it, sm_scale=0.1, d_v=D, dq=torch.empty_like(q), dkv=torch.empty_like(kv).half())


def test_per_token_fp8_backward_over_prepared_buffers(device):
    """fp8_sparse_mla_bwd_kernel's contract: gradients with respect to the dequantised q and kv."""
    from cppmega_mlx_amd.nn._tilelang import sparse_mla_fp8_path_c as f8
    from oracle import fp8

    rng = np.random.default_rng(12)
    B, S, H, G, Skv, topk, D, d_v = 2, 5, 4, 2, 40, 16, 64, 32
    qc, qs = fp8.quantize_per_token(rng.standard_normal((B * S * H, D)).astype(np.float32))
    kc, ks = fp8.quantize_per_token(rng.standard_normal((B * Skv * G, D)).astype(np.float32))
    qc, qs, kc, ks = qc.reshape(B, S, H, D), qs.reshape(B, S, H), kc.reshape(B, Skv, G, D), ks.reshape(B, Skv, G)
    d_out = rng.standard_normal((B, S, H, d_v)).astype(np.float32)
    idx = sparse_indices(rng, B, S, G, Skv, topk, replace=True)
    idx[0, 2] = -1
    idx[1, 0, 0, :3] = Skv + 1
    want_dq, want_dkv = om.sparse_mla_bwd_oracle(om.dequant_per_token(qc, qs), om.dequant_per_token(kc, ks), idx, d_out,
                                                 sm_scale=0.2, d_v=d_v)
    args = (to_dev(qc, device), to_dev(qs, device), to_dev(kc, device), to_dev(ks, device))
    for dtype in (torch.float32, torch.float16):
        dq, dkv = f8.sparse_mla_fp8_bwd_path_c(*args, to_dev(d_out, device).to(dtype), to_dev(idx.astype(np.int32), device),
                                               sm_scale=0.2, d_v=d_v)
        torch.cuda.synchronize()
        tol = 1e-4 if dtype == torch.float32 else 2e-3
        for got, want in ((dq, want_dq), (dkv, want_dkv)):
            assert got.dtype == torch.float32
            err, ref = error_report(got.cpu().numpy(), want)
            assert err <= tol * ref, (err, ref)
    dq_buf = torch.zeros((B, S, H, D), dtype=torch.float32, device=device)
    dkv_buf = torch.full((B, Skv, G, D), 3.0, dtype=torch.float32, device=device)
    got = f8.sparse_mla_fp8_bwd_path_c(*args, to_dev(d_out, device), to_dev(idx, device), sm_scale=0.2, d_v=d_v,
                                       dq_buffer=dq_buf, dkv_buffer=dkv_buf)
    torch.cuda.synchronize()
    assert got[0] is dq_buf and got[1] is dkv_buf
    err, ref = error_report(dkv_buf.cpu().numpy(), want_dkv)
    assert err <= 1e-4 * ref
    with pytest.raises(ValueError):
        f8.sparse_mla_fp8_bwd_path_c(*args, to_dev(d_out, device)[..., :8].contiguous(), to_dev(idx, device), sm_scale=0.2, d_v=d_v)
    # the differentiable owner wrapper: forward over the prepared buffers, gradients to the float producers
    qf = to_dev(om.dequant_per_token(qc, qs).astype(np.float32), device).requires_grad_(True)
    kf = to_dev(om.dequant_per_token(kc, ks).astype(np.float32), device).to(torch.bfloat16).requires_grad_(True)
    out = f8.sparse_mla_fp8_path_c_apply_prepared_float(qf, kf, *args, to_dev(idx.astype(np.int32), device), sm_scale=0.2, d_v=d_v)
    assert out.dtype == torch.float32 and tuple(out.shape) == (B, S, H, d_v)
    (out * to_dev(d_out, device)).sum().backward()
    torch.cuda.synchronize()
    assert qf.grad.dtype == torch.float32 and kf.grad.dtype == torch.bfloat16
    err, ref = error_report(qf.grad.cpu().numpy(), want_dq)
    assert err <= 1e-4 * ref
    err, ref = error_report(kf.grad.float().cpu().numpy(), want_dkv)
    assert err <= 1e-2 * ref                                    # one rounding to bfloat16
    with pytest.raises(RuntimeError, match="sinks backward"):
        o2 = f8.sparse_mla_fp8_path_c_apply_prepared_float(qf, kf, *args, to_dev(idx.astype(np.int32), device), sm_scale=0.2, d_v=d_v,
                                                           sinks=torch.zeros(H, device=device))
        o2.sum().backward()
    with pytest.raises(RuntimeError, match="requires prepared FP8 buffers"):
        f8.sparse_mla_fp8_path_c_apply_from_float(qf, kf, to_dev(idx, device), sm_scale=0.2)


def test_bench_size_invariants_of_the_backward(device):
    """At the size the bench times: the columns of dkv sum to the cotangents of the queries that had a valid key on the
    first d_v channels (every softmax row sums to 1) and to zero on the rest (every dS row sums to 0); the gradients
    are linear in d_out."""
    B, S, H, D, d_v, Skv, topk = 1, 1024, 16, 576, 512, 4096, 256
    gen = torch.Generator(device=device).manual_seed(5)
    q = torch.randn((B, S, H, D), generator=gen, device=device).to(torch.bfloat16)
    kv = (torch.randn((B, Skv, 1, D), generator=gen, device=device) * 0.5).to(torch.bfloat16)
    d_out = torch.randn((B, S, H, d_v), generator=gen, device=device).to(torch.bfloat16)
    idx = torch.stack([torch.randperm(Skv, generator=gen, device=device)[:topk] for _ in range(S)]).to(torch.int32).view(B, S, 1, topk).clone()
    idx[0, 5] = -1                                            # one query without keys
    dq = torch.empty((B, S, H, D), dtype=torch.float32, device=device)
    dkv = torch.empty((B, Skv, 1, D), dtype=torch.float32, device=device)
    ops.sparse_mla_backward(q, kv, d_out, idx, sm_scale=D ** -0.5, d_v=d_v, dq=dq, dkv=dkv)
    torch.cuda.synchronize()
    cols = dkv.double().sum(dim=(0, 1, 2)).cpu().numpy()
    live = torch.ones(S, dtype=torch.bool, device=device); live[5] = False
    want = d_out[0, live].double().sum(dim=(0, 1)).cpu().numpy()
    scale = float(np.abs(dkv.cpu().numpy()).sum(axis=(0, 1, 2)).max())      # what the column sums are sums of
    assert np.abs(cols[:d_v] - want).max() <= 1e-5 * scale
    assert np.abs(cols[d_v:]).max() <= 1e-5 * scale
    assert (dq[0, 5] == 0).all()
    dq2 = torch.empty_like(dq); dkv2 = torch.empty_like(dkv)
    ops.sparse_mla_backward(q, kv, d_out * 2, idx, sm_scale=D ** -0.5, d_v=d_v, dq=dq2, dkv=dkv2)
    torch.cuda.synchronize()
    assert torch.equal(dq2, dq * 2)                            # doubling is exact in every step of dq
    assert float((dkv2 - 2 * dkv).abs().max()) <= 1e-5 * float(dkv.abs().max())   # atomic order only


def test_training_entry_points_replay_from_a_hip_graph(device):
    """The backward (with its dkv clear, a fill kernel) and the indexer loss captured once; each replay, with the
    inputs rewritten and eager launches in between, must reproduce the eager result for the contents at that moment."""
    from cppmega_mlx_amd.nn._tilelang.dsa_splitk_indexer_loss import dsa_splitk_indexer_loss_per_position

    gen = torch.Generator(device=device).manual_seed(21)
    B, S, H, D, d_v, Skv, topk = 1, 12, 16, 128, 64, 96, 40
    q = torch.randn((B, S, H, D), generator=gen, device=device).to(torch.bfloat16)
    kv = torch.randn((B, Skv, 1, D), generator=gen, device=device).to(torch.bfloat16)
    d_out = torch.randn((B, S, H, d_v), generator=gen, device=device).to(torch.bfloat16)
    idx = torch.stack([torch.randperm(Skv, generator=gen, device=device)[:topk] for _ in range(S)]).to(torch.int32).view(B, S, 1, topk)
    sm = torch.tensor([D ** -0.5], dtype=torch.float32, device=device)
    ASq = Sk = 48
    lq = torch.randn((ASq, 1, 4, 64), generator=gen, device=device).to(torch.bfloat16)
    lk = torch.randn((Sk, 1, 4, 64), generator=gen, device=device).to(torch.bfloat16)
    lidx = torch.randn((1, ASq, Sk), generator=gen, device=device)
    ltop = torch.topk(lidx, 8, dim=-1).indices.to(torch.int32).contiguous()

    def buffers():
        return dict(dq=torch.zeros((B, S, H, D), dtype=torch.float32, device=device),
                    dkv=torch.zeros((B, Skv, 1, D), dtype=torch.float32, device=device),
                    loss=torch.zeros((1, ASq), dtype=torch.float32, device=device))

    def launch(o):
        ops.sparse_mla_backward(q, kv, d_out, idx, sm_scale=sm, d_v=d_v, dq=o["dq"], dkv=o["dkv"])
        ops.dsa_indexer_loss(lq, lk, lidx, softmax_scale=0.125, out=o["loss"], topk_indices=ltop)

    captured, eager = buffers(), buffers()
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        launch(captured)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        launch(captured)
    for step in range(3):
        sm.fill_(D ** -0.5 * (1 + step))
        d_out.mul_(-1.5)
        lidx.add_(0.25 * step * torch.arange(Sk, device=device, dtype=torch.float32))
        for t in captured.values():
            t.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        launch(eager)
        torch.cuda.synchronize()
        assert torch.equal(captured["dq"], eager["dq"]) and torch.equal(captured["loss"], eager["loss"]), step
        assert float((captured["dkv"] - eager["dkv"]).abs().max()) <= 1e-5 * float(eager["dkv"].abs().max())   # atomic order
        want_dq, want_dkv = om.sparse_mla_bwd_oracle(q.double().cpu().numpy(), kv.double().cpu().numpy(), idx.cpu().numpy(),
                                                     d_out.double().cpu().numpy(), sm_scale=float(sm), d_v=d_v)
        err, ref = error_report(captured["dq"].cpu().numpy(), want_dq)
        assert err <= 1e-4 * ref
        err, ref = error_report(captured["dkv"].cpu().numpy(), want_dkv)
        assert err <= 1e-4 * ref
    want_loss = dsa_splitk_indexer_loss_per_position(lidx, ltop, lq, lk, 0.125, True)
    assert torch.equal(captured["loss"], want_loss)
