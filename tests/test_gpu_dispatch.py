"""GPU parity through the kernel boundary: the four kernels as ``dispatch_lower`` hands them out.

The reference compiles a PrimFunc and calls the artifact with device buffers in PrimFunc
parameter order plus caller-owned ``out=`` buffers (cppmega_mlx/nn/_tilelang/_engine_dispatch.py
:242-304, _mlx_runtime.py:147-215).  These tests take the same route: flat buffers in the
reference's order, the scale and the sink switch as device buffers, owner outputs returned as
the same objects, results against the oracle, and the launches replayed from a HIP graph.
"""

import numpy as np
import pytest
import torch

from cppmega_mlx_amd.nn._tilelang import _engine_dispatch as ed
from oracle import fp8, sparse_mla as om, topk as otk, vecmat as ovm
from tests._inputs import sparse_indices, to_dev, topk_scores

pytestmark = pytest.mark.gpu


def _mla_case(rng, device, *, blockscaled: bool):
    """Prepared buffers of one sparse-MLA call, flat as the reference's kernels take them, and the
    real numbers they decode to."""
    B, S, H, G, Skv, topk, K, dv = 2, 5, 8, 2, 96, 24, 64, 32
    qf = rng.standard_normal((B, S, H, K)).astype(np.float32)
    kf = rng.standard_normal((B, Skv, G, K)).astype(np.float32)
    if blockscaled:
        qc, qs = fp8.quantize_mxfp8(qf)
        kc, ks = fp8.quantize_mxfp8(kf)
        q_real, k_real = om.dequant_e8m0(qc, qs), om.dequant_e8m0(kc, ks)
    else:
        qc, qs = fp8.quantize_per_token(qf.reshape(-1, K))
        kc, ks = fp8.quantize_per_token(kf.reshape(-1, K))
        qc, qs, kc, ks = qc.reshape(B, S, H, K), qs.reshape(B, S, H), kc.reshape(B, Skv, G, K), ks.reshape(B, Skv, G)
        q_real, k_real = om.dequant_per_token(qc, qs), om.dequant_per_token(kc, ks)
    idx = sparse_indices(rng, B, S, G, Skv, topk, causal_offset=40)
    idx[:, :, :, -3:] = -1
    shape = dict(B=B, S=S, H=H, G=G, Skv=Skv, topk=topk, K=K, d_v=dv)
    bufs = dict(q_fp8=to_dev(qc, device).reshape(-1), q_scale=to_dev(qs, device).reshape(-1),
                kv_fp8=to_dev(kc, device).reshape(-1), kv_scale=to_dev(ks, device).reshape(-1),
                indices=to_dev(idx.astype(np.int32), device).reshape(-1))
    return shape, bufs, q_real, k_real, idx


def _check_mla(out, lse, want_out, want_lse):
    got = out.float().cpu().numpy().reshape(want_out.shape)
    assert np.abs(got - want_out).max() <= 2e-2 * np.abs(want_out).max()
    assert np.abs(lse.cpu().numpy().reshape(want_lse.shape) - want_lse).max() <= 1e-3


def test_topk_kernel_from_dispatch_lower(device):
    rng = np.random.default_rng(41)
    rows, width, k = 9, 777, 16
    scores = topk_scores(rng, rows, width)
    starts = rng.integers(0, 50, rows).astype(np.int32)
    ends = rng.integers(400, width + 1, rows).astype(np.int32)
    kernel = ed.dispatch_lower(ed.topk_spec(k), "gfx950")
    assert kernel._tilelang_engine_target == "gfx950" and kernel.result_indices == (1,)
    owner = torch.full((rows, k), -7, dtype=torch.int32, device=device)
    got = kernel(to_dev(ends, device), to_dev(scores, device), to_dev(starts, device), out=owner)
    torch.cuda.synchronize()
    assert got is owner
    want = otk.topk_selector_oracle(scores, k, starts=starts, ends=ends, order="value")
    np.testing.assert_array_equal(owner.cpu().numpy(), want)
    # full-ABI form: every parameter in PrimFunc order, the owner among them
    owner2 = torch.zeros_like(owner)
    assert kernel(to_dev(ends, device), owner2, to_dev(scores, device), to_dev(starts, device)) is owner2
    torch.cuda.synchronize()
    assert torch.equal(owner2, owner)


def test_vecmat_kernel_from_dispatch_lower(device):
    rng = np.random.default_rng(42)
    N, K = 300, 512
    w = fp8.e4m3_encode(rng.standard_normal((N, K)).astype(np.float32))
    x = fp8.e4m3_encode(rng.standard_normal(K).astype(np.float32))
    sx = np.array([0.37], dtype=np.float32)
    kernel = ed.dispatch_lower(ed.vecmat_spec(), "hip")
    for sw in (np.array([1.9], dtype=np.float32), rng.uniform(0.5, 2.0, N).astype(np.float32)):
        owner = torch.zeros((1, N), dtype=torch.float32, device=device)
        got = kernel(to_dev(x, device).reshape(1, K), to_dev(sx, device), to_dev(w, device), to_dev(sw, device), out=owner)
        torch.cuda.synchronize()
        assert got is owner
        want = ovm.fp8_scaled_vecmat_oracle(x, w, scale_x=sx, scale_w=sw)
        np.testing.assert_allclose(owner.cpu().numpy().reshape(-1), want, rtol=2e-5, atol=1e-5 * np.abs(want).max())


def test_blockscaled_mla_kernel_from_dispatch_lower(device):
    rng = np.random.default_rng(43)
    shape, bufs, q_real, k_real, idx = _mla_case(rng, device, blockscaled=True)
    B, S, H, dv = shape["B"], shape["S"], shape["H"], shape["d_v"]
    kernel = ed.dispatch_lower(ed.blockscaled_mla_spec(**shape), "gfx950")
    assert kernel.result_indices == (6, 7)
    sm = torch.tensor([0.11], dtype=torch.float32, device=device)
    out = torch.zeros(B * S * H * dv, dtype=torch.bfloat16, device=device)
    lse = torch.zeros(B * S * H, dtype=torch.float32, device=device)
    got = kernel(bufs["q_fp8"], bufs["q_scale"], bufs["kv_fp8"], bufs["kv_scale"], bufs["indices"], sm, out=(out, lse))
    torch.cuda.synchronize()
    assert got[0] is out and got[1] is lse
    _check_mla(out, lse, *om.sparse_mla_oracle(q_real, k_real, idx, sm_scale=0.11, d_v=dv))
    # the scale is read on the device: a new value in the same buffer, no new kernel object
    sm.fill_(0.05)
    kernel(bufs["q_fp8"], bufs["q_scale"], bufs["kv_fp8"], bufs["kv_scale"], bufs["indices"], sm, out=(out, lse))
    torch.cuda.synchronize()
    _check_mla(out, lse, *om.sparse_mla_oracle(q_real, k_real, idx, sm_scale=0.05, d_v=dv))


def test_fp8_mla_kernel_from_dispatch_lower_reads_the_sink_switch_on_the_device(device):
    rng = np.random.default_rng(44)
    shape, bufs, q_real, k_real, idx = _mla_case(rng, device, blockscaled=False)
    B, S, H, dv = shape["B"], shape["S"], shape["H"], shape["d_v"]
    kernel = ed.dispatch_lower(ed.fp8_mla_spec(**shape), "gfx950")
    assert kernel.result_indices == (8, 9)
    sinks = rng.standard_normal(H).astype(np.float32)
    sm = torch.tensor([0.125], dtype=torch.float32, device=device)
    has = torch.zeros(1, dtype=torch.int32, device=device)
    out = torch.zeros(B * S * H * dv, dtype=torch.float32, device=device)
    lse = torch.zeros(B * S * H, dtype=torch.float32, device=device)
    args = (bufs["q_fp8"], bufs["q_scale"], bufs["kv_fp8"], bufs["kv_scale"], bufs["indices"], sm, to_dev(sinks, device), has)
    for flag, want_sinks in ((0, None), (1, sinks), (0, None)):
        has.fill_(flag)
        kernel(*args, out=(out, lse))
        torch.cuda.synchronize()
        _check_mla(out, lse, *om.sparse_mla_oracle(q_real, k_real, idx, sm_scale=0.125, d_v=dv, sinks=want_sinks))


def test_dispatched_kernels_replay_from_a_hip_graph(device):
    """All four kernels captured once; every replay, with eager launches and buffer updates in
    between, must equal the eager result for the buffers' contents at that moment."""
    rng = np.random.default_rng(45)
    shape, bufs, q_real, k_real, idx = _mla_case(rng, device, blockscaled=False)
    bshape, bbufs, bq_real, bk_real, bidx = _mla_case(rng, device, blockscaled=True)
    B, S, H, dv = shape["B"], shape["S"], shape["H"], shape["d_v"]
    rows, width, k, N, K = 6, 3000, 32, 256, 1024
    scores = to_dev(topk_scores(rng, rows, width), device)
    ends = to_dev(rng.integers(width // 2, width + 1, rows).astype(np.int32), device)
    starts = torch.zeros(rows, dtype=torch.int32, device=device)
    w = to_dev(fp8.e4m3_encode(rng.standard_normal((N, K)).astype(np.float32)), device)
    x = to_dev(fp8.e4m3_encode(rng.standard_normal(K).astype(np.float32)), device).reshape(1, K)
    sx = torch.tensor([0.5], dtype=torch.float32, device=device)
    sw = to_dev(rng.uniform(0.5, 2.0, N).astype(np.float32), device)
    sinks = to_dev(rng.standard_normal(H).astype(np.float32), device)
    sm = torch.tensor([0.125], dtype=torch.float32, device=device)
    has = torch.ones(1, dtype=torch.int32, device=device)

    k_topk = ed.dispatch_lower(ed.topk_spec(k), "gfx950")
    k_vec = ed.dispatch_lower(ed.vecmat_spec(), "gfx950")
    k_fp8 = ed.dispatch_lower(ed.fp8_mla_spec(**shape), "gfx950")
    k_bs = ed.dispatch_lower(ed.blockscaled_mla_spec(**bshape), "gfx950")

    def buffers():
        return dict(idx=torch.zeros((rows, k), dtype=torch.int32, device=device),
                    c=torch.zeros((1, N), dtype=torch.float32, device=device),
                    out=torch.zeros(B * S * H * dv, dtype=torch.float32, device=device),
                    lse=torch.zeros(B * S * H, dtype=torch.float32, device=device),
                    bout=torch.zeros(B * S * H * dv, dtype=torch.float32, device=device),
                    blse=torch.zeros(B * S * H, dtype=torch.float32, device=device))

    def launch(o):
        k_topk(ends, scores, starts, out=o["idx"])
        k_vec(x, sx, w, sw, out=o["c"])
        k_fp8(bufs["q_fp8"], bufs["q_scale"], bufs["kv_fp8"], bufs["kv_scale"], bufs["indices"], sm, sinks, has,
              out=(o["out"], o["lse"]))
        k_bs(bbufs["q_fp8"], bbufs["q_scale"], bbufs["kv_fp8"], bbufs["kv_scale"], bbufs["indices"], sm,
             out=(o["bout"], o["blse"]))

    captured, eager = buffers(), buffers()
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        launch(captured)                                     # warm-up on the capture stream
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        launch(captured)
    for step, (scale, flag) in enumerate(((0.125, 1), (0.07, 0), (0.2, 1), (0.125, 1))):
        sm.fill_(scale)
        has.fill_(flag)
        scores.mul_(-1.0 if step else 1.0)                   # new top-k answer every replay after the first
        sx.fill_(0.5 + step)
        for t in captured.values():
            t.fill_(-3)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        launch(eager)                                        # the program's own eager work between replays
        torch.cuda.synchronize()
        for name in captured:
            assert torch.equal(captured[name], eager[name]), (step, name)
        want_out, want_lse = om.sparse_mla_oracle(q_real, k_real, idx, sm_scale=scale, d_v=dv,
                                                  sinks=sinks.cpu().numpy() if flag else None)
        _check_mla(captured["out"], captured["lse"], want_out, want_lse)
        np.testing.assert_array_equal(
            captured["idx"].cpu().numpy(),
            otk.topk_selector_oracle(scores.cpu().numpy(), k, starts=starts.cpu().numpy(), ends=ends.cpu().numpy(), order="value"))
