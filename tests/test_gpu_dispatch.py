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


def test_float_carrier_mla_kernels_from_dispatch_lower(device):
    """The float-carrier forward in the reference's order kernel(indices, kv, lse, out, q, sm_scale_buf) with
    out_idx=[2, 3] (sparse_mla_path_c.py:2291-2299, 3068, 3282-3288) and the backward kernel(d_out, dkv, dq,
    indices, kv, q, sm_scale_buf) with out_idx=[1, 2] (:2670-2678, 3159), float16 carriers as in the reference."""
    rng = np.random.default_rng(46)
    B, S, H, G, Skv, topk, K, dv = 2, 3, 8, 2, 80, 20, 64, 32
    shape = dict(B=B, S=S, H=H, G=G, Skv=Skv, topk=topk, K=K, d_v=dv)
    q16 = rng.standard_normal((B, S, H, K)).astype(np.float16)
    kv16 = rng.standard_normal((B, Skv, G, K)).astype(np.float16)
    idx = sparse_indices(rng, B, S, G, Skv, topk, causal_offset=30)
    idx[:, :, :, -2:] = -1
    q, kv, ind = to_dev(q16, device).reshape(-1), to_dev(kv16, device).reshape(-1), to_dev(idx.astype(np.int32), device).reshape(-1)
    sm = torch.tensor([0.2], dtype=torch.float32, device=device)
    fwd = ed.dispatch_lower(ed.float_mla_spec(**shape), "gfx950")
    assert fwd.result_indices == (2, 3)
    lse = torch.zeros(B * S * H, dtype=torch.float32, device=device)
    out = torch.zeros(B * S * H * dv, dtype=torch.float16, device=device)
    got = fwd(ind, kv, q, sm, out=(lse, out))
    torch.cuda.synchronize()
    assert got[0] is lse and got[1] is out
    want_out, want_lse = om.sparse_mla_oracle(q16.astype(np.float64), kv16.astype(np.float64), idx, sm_scale=0.2, d_v=dv)
    _check_mla(out, lse, want_out, want_lse)

    bwd = ed.dispatch_lower(ed.float_mla_bwd_spec(**shape), "gfx950")
    assert bwd.result_indices == (1, 2)
    d_out16 = rng.standard_normal((B, S, H, dv)).astype(np.float16)
    dkv = torch.full((B * Skv * G * K,), 7.0, dtype=torch.float32, device=device)      # cleared by the call
    dq = torch.zeros(B * S * H * K, dtype=torch.float16, device=device)
    got = bwd(to_dev(d_out16, device).reshape(-1), ind, kv, q, sm, out=(dkv, dq))
    torch.cuda.synchronize()
    assert got[0] is dkv and got[1] is dq
    want_dq, want_dkv = om.sparse_mla_bwd_oracle(q16.astype(np.float64), kv16.astype(np.float64), idx, d_out16.astype(np.float64),
                                                 sm_scale=0.2, d_v=dv)
    assert np.abs(dq.float().cpu().numpy().reshape(want_dq.shape) - want_dq).max() <= 2e-2 * np.abs(want_dq).max()
    assert np.abs(dkv.cpu().numpy().reshape(want_dkv.shape) - want_dkv).max() <= 1e-3 * np.abs(want_dkv).max()


def test_latent_cache_mla_kernel_from_dispatch_lower_and_graph_replay(device):
    """The latent-cache layout (bfloat16 q, e4m3 latent + float32 scales per 128 channels + bfloat16 rope tail)
    through dispatch_lower on the 64-head kernel with key splits, eager and replayed from a HIP graph with the
    scale buffer rewritten in between."""
    from tests._inputs import bf16_pair, latent_cache
    rng = np.random.default_rng(47)
    B, S, H, G, Skv, topk = 2, 1, 128, 1, 3000, 1024
    shape = dict(B=B, S=S, H=H, G=G, Skv=Skv, topk=topk, K=512, R=64, d_v=512, scale_block=128)
    q, qf = bf16_pair(rng.standard_normal((B, S, H, 576)), device)
    codes, scale, rope, rows = latent_cache(rng, B, Skv, G, 512, 64, device, pow2=False)
    idx = sparse_indices(rng, B, S, G, Skv, topk)
    ind = to_dev(idx.astype(np.int32), device)
    kernel = ed.dispatch_lower(ed.latent_mla_spec(**shape), "gfx950")
    assert kernel.result_indices == (8, 9)
    sm = torch.tensor([576 ** -0.5], dtype=torch.float32, device=device)
    out = torch.zeros(B * S * H * 512, dtype=torch.bfloat16, device=device)
    lse = torch.zeros(B * S * H, dtype=torch.float32, device=device)
    args = (q.reshape(-1), codes.reshape(-1), scale.reshape(-1), rope.reshape(-1), ind.reshape(-1), sm, None, None)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        assert kernel(*args, out=(out, lse))[0] is out
    stream.synchronize()
    _check_mla(out, lse, *om.sparse_mla_oracle(qf, rows, idx, sm_scale=576 ** -0.5, d_v=512))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        kernel(*args, out=(out, lse))
    for scale_value in (0.03, 576 ** -0.5, 0.05):
        sm.fill_(scale_value)
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        _check_mla(out, lse, *om.sparse_mla_oracle(qf, rows, idx, sm_scale=scale_value, d_v=512))


def test_bare_e4m3_conversions(device):
    """fp8_to_half / half_to_fp8 (cppmega_mlx/nn/_tilelang/fp8_msl_kernels.py:65-81): every byte decodes to the
    oracle's table value; float16 inputs round to nearest even and saturate at +-448; a decode of an encode is
    the identity on the non-NaN codes."""
    from cppmega_mlx_amd.nn._tilelang import fp8_msl_kernels as fk
    codes = np.arange(256, dtype=np.uint8)
    got = fk.fp8_to_half(to_dev(codes, device))
    torch.cuda.synchronize()
    want = fp8.e4m3_decode(codes).astype(np.float32)
    got_np = got.float().cpu().numpy()
    ok = ~np.isnan(want)
    assert got.dtype == torch.float16 and np.array_equal(got_np[ok], want[ok]) and np.isnan(got_np[~ok]).all()
    rng = np.random.default_rng(48)
    x = np.concatenate([rng.standard_normal(4000) * 3, rng.standard_normal(500) * 300, fp8.e4m3_decode(codes[ok]),
                        [0.0, -0.0, 448.0, 449.0, -1000.0, 2.0 ** -10, 2.0 ** -9 * 1.5, 0.0009765625 * 3]]).astype(np.float16)
    enc = fk.half_to_fp8(to_dev(x, device))
    torch.cuda.synchronize()
    assert enc.dtype == torch.uint8
    np.testing.assert_array_equal(enc.cpu().numpy(), fp8.e4m3_encode(x.astype(np.float64)))
    back = fk.half_to_fp8(fk.fp8_to_half(to_dev(codes[ok], device)))
    torch.cuda.synchronize()
    keep = codes[ok] != 0x80                                    # -0 encodes as it is; compare values for it
    np.testing.assert_array_equal(back.cpu().numpy()[keep], codes[ok][keep])
    assert fk.fp8_to_half(torch.zeros((0, 4), dtype=torch.uint8, device=device)).shape == (0, 4)
    with pytest.raises(TypeError):
        fk.half_to_fp8(torch.zeros(4, dtype=torch.float32, device=device))
