"""GPU parity: the per-head projections of the absorbed MLA decode, the block-128 FP8 weight
dequantiser, the reference's absorbed == standard identity, and one whole decode-layer step
(append -> indices -> absorb -> sparse MLA over the FP8 cache -> un-absorb -> FP8 out-projection)
against the oracle chain.

Tolerances: float32 operands enter the matrix cores as bf16 hi + lo pairs, so a product carries
about 2^-16 relative error: 1e-4 of the output scale for float32 results (the reference's own
atol = rtol = 1e-4), 2e-2 of the output scale once bfloat16 tensors are involved."""

import numpy as np
import pytest
import torch

from cppmega_mlx_amd import _lib, ops
from cppmega_mlx_amd.inference import SparseFP8KVCache, SparseFP8KVCacheConfig
from cppmega_mlx_amd.nn import fp8_dequant as fd, mla_absorb as ma
from cppmega_mlx_amd.nn._tilelang.fused_fp8_gemm import fused_fp8_gemm
from cppmega_mlx_amd.nn.attention import causal_sparse_indices
from oracle import fp8, kv_cache as okv, mla_absorb as oa, sparse_mla as om, vecmat as ovm
from tests._inputs import bf16_pair, error_report, to_dev

pytestmark = pytest.mark.gpu


def _rand(*shape, seed=0):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("w_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(1, 3, 70, 100), (33, 2, 64, 128), (70, 1, 130, 1100), (32, 4, 512, 128)])
def test_head_gemm_matches_einsum(device, x_dtype, w_dtype, shape):
    M, G, N, K = shape
    rng = np.random.default_rng(M + N + K)
    xt = to_dev(rng.standard_normal((M, G, K)).astype(np.float32), device).to(x_dtype)
    wt = to_dev(rng.standard_normal((G, N, K)).astype(np.float32), device).to(w_dtype)
    want = np.einsum("mgk,gnk->mgn", xt.double().cpu().numpy(), wt.double().cpu().numpy())
    out = torch.zeros((M, G, N), dtype=torch.float32, device=device)
    assert ops.head_gemm(xt, wt, out=out) is out
    torch.cuda.synchronize()
    err, ref = error_report(out.cpu().numpy(), want)
    assert err <= 1e-4 * ref
    # strided operands: x rows inside wider rows, the result inside wider rows
    wide_x = torch.zeros((M, G, K + 24), dtype=x_dtype, device=device); wide_x[..., 8:8 + K] = xt
    wide_y = torch.full((M, G, N + 10), 5.0, dtype=torch.bfloat16, device=device)
    ops.head_gemm(wide_x[..., 8:8 + K], wt, out=wide_y[..., :N])
    torch.cuda.synchronize()
    err, ref = error_report(wide_y[..., :N].float().cpu().numpy(), want)
    assert err <= 2e-2 * ref and (wide_y[..., N:] == 5.0).all()


def test_head_gemm_is_exact_on_integers_and_rejects_bad_arguments(device):
    rng = np.random.default_rng(3)
    x = rng.integers(-4, 5, (20, 2, 96)).astype(np.float32)
    w = rng.integers(-4, 5, (2, 40, 96)).astype(np.float32)
    out = torch.zeros((20, 2, 40), dtype=torch.float32, device=device)
    ops.head_gemm(to_dev(x, device), to_dev(w, device).to(torch.bfloat16), out=out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), np.einsum("mgk,gnk->mgn", x, w))
    with pytest.raises(ValueError):
        ops.head_gemm(to_dev(x, device), to_dev(w, device)[:, :, :90], out=out)
    with pytest.raises(ValueError):
        ops.head_gemm(to_dev(x, device), to_dev(w, device).transpose(1, 2).contiguous().transpose(1, 2), out=out)
    with pytest.raises(TypeError):
        ops.head_gemm(to_dev(x, device).half(), to_dev(w, device), out=out)
    with pytest.raises(_lib.NativeCallError):
        ops.head_gemm(torch.from_numpy(x), to_dev(w, device), out=out)


def test_absorb_weights_shapes_and_errors(device):
    h, d_kv, d_k, d_v, d_model = 2, 8, 4, 6, 12
    w_uk, w_uv, w_o = (to_dev(a, device) for a in (_rand(h, d_kv, d_k, seed=1), _rand(h, d_kv, d_v, seed=2), _rand(h * d_v, d_model, seed=3)))
    a, f = ma.absorb_weights(w_uk, w_uv, w_o)
    torch.cuda.synchronize()
    assert tuple(a.shape) == (h, d_k, d_kv) and tuple(f.shape) == (h, d_kv, d_model)
    want_a, want_f = oa.absorb_weights(w_uk.cpu().numpy(), w_uv.cpu().numpy(), w_o.cpu().numpy())
    np.testing.assert_array_equal(a.cpu().numpy(), want_a.astype(np.float32))
    np.testing.assert_allclose(f.cpu().numpy(), want_f, atol=1e-4, rtol=1e-4)
    z = lambda *s: torch.zeros(s, device=device)
    with pytest.raises(ValueError):
        ma.absorb_weights(z(2, 8), z(2, 8, 6), z(12, 16))
    with pytest.raises(ValueError):
        ma.absorb_weights(z(2, 8, 4), z(3, 8, 6), z(12, 16))
    with pytest.raises(ValueError):
        ma.absorb_weights(z(2, 8, 4), z(2, 8, 6), z(10, 16))


@pytest.mark.parametrize("dims", [(1, 2, 2, 4, 8, 6, 12, 5), (2, 1, 8, 128, 512, 128, 256, 70)])
def test_absorbed_equals_standard_decode(device, dims):
    """tests/v4/test_mla_absorb.py:36-50 (same seeds and sizes in the first case), then head sizes of the real model."""
    b, t, h, d_k, d_kv, d_v, d_model, t_kv = dims
    scale = 1.0 if d_kv <= 8 else d_kv ** -0.5
    q, c_kv = _rand(b, t, h, d_k, seed=10), _rand(b, t_kv, d_kv, seed=11)
    w_uk, w_uv, w_o = _rand(h, d_kv, d_k, seed=12) * scale, _rand(h, d_kv, d_v, seed=13) * scale, _rand(h * d_v, d_model, seed=14) * (h * d_v) ** -0.5
    qt, ct, ukt, uvt, ot = (to_dev(a, device) for a in (q, c_kv, w_uk, w_uv, w_o))
    a, f = ma.absorb_weights(ukt, uvt, ot)
    out_abs = ma.absorbed_mla_decode(qt, ct, a, f)
    out_std = ma.standard_mla_decode(qt, ct, ukt, uvt, ot)
    torch.cuda.synchronize()
    assert tuple(out_abs.shape) == (b, t, d_model)
    want = oa.standard_mla_decode(q, c_kv, w_uk, w_uv, w_o)
    np.testing.assert_allclose(out_abs.cpu().numpy(), want, atol=1e-4, rtol=1e-4)
    np.testing.assert_allclose(out_abs.cpu().numpy(), out_std.cpu().numpy(), atol=1e-4, rtol=1e-4)
    # weights in another memory order give the same result (re-laid out on the call)
    out_again = ma.absorbed_mla_decode(qt, ct, a.contiguous(), f.contiguous())
    torch.cuda.synchronize()
    assert torch.equal(out_again, out_abs)


def test_absorbed_decode_with_mask_and_bad_shapes(device):
    b, t, h, d_k, d_kv, d_v, d_model, t_kv = 1, 1, 2, 4, 6, 4, 8, 4
    q, c_kv = _rand(b, t, h, d_k, seed=20), _rand(b, t_kv, d_kv, seed=21)
    w_uk, w_uv, w_o = _rand(h, d_kv, d_k, seed=22), _rand(h, d_kv, d_v, seed=23), _rand(h * d_v, d_model, seed=24)
    qt, ct = to_dev(q, device), to_dev(c_kv, device)
    a, f = ma.absorb_weights(to_dev(w_uk, device), to_dev(w_uv, device), to_dev(w_o, device))
    mask = np.zeros((b, t, h, t_kv), dtype=np.float32); mask[..., -1] = -1e9
    out = ma.absorbed_mla_decode(qt, ct, a, f, mask=to_dev(mask, device))
    torch.cuda.synchronize()
    want_a, want_f = oa.absorb_weights(w_uk, w_uv, w_o)
    np.testing.assert_allclose(out.cpu().numpy(), oa.absorbed_mla_decode(q, c_kv, want_a, want_f, mask=mask), atol=1e-4, rtol=1e-4)
    with pytest.raises(ValueError):
        ma.absorbed_mla_decode(torch.zeros((1, 1, d_k), device=device), ct, a, f)
    with pytest.raises(ValueError):
        ma.absorbed_mla_decode(qt, ct, torch.zeros((h, d_k + 1, d_kv), device=device), f)


def test_dequant_block_fp8_and_sanitize(device):
    rng = np.random.default_rng(5)
    m, n = 200, 300
    codes = rng.integers(0, 256, (m, n)).astype(np.uint8)
    scale = rng.uniform(0.5, 1.5, (2, 3)).astype(np.float32)
    got = fd.dequant_block_fp8(to_dev(codes, device), to_dev(scale, device))
    torch.cuda.synchronize()
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (m, n)
    want = oa.dequant_block_fp8(codes, scale)
    nan = (codes & 0x7F) == 0x7F
    g = got.float().cpu().numpy()
    assert np.isnan(g[nan]).all() and nan.any()
    np.testing.assert_array_equal(g[~nan], want[~nan])
    out32 = torch.zeros((m, n), dtype=torch.float32, device=device)
    ops.dequant_block_fp8(to_dev(codes, device), to_dev(scale, device), out=out32)
    torch.cuda.synchronize()
    table = fp8.e4m3_decode(codes, np.float32)
    full = np.repeat(np.repeat(scale, 128, 0), 128, 1)[:m, :n]
    np.testing.assert_array_equal(out32.cpu().numpy()[~nan], (table * full)[~nan])
    wa, sa = to_dev(rng.integers(0, 120, (64, 64)).astype(np.uint8), device), to_dev(np.full((1, 1), 0.5, np.float32), device)
    other = torch.zeros((8, 8), device=device)
    weights = {"l0.proj.weight": wa, "l0.proj.weight_scale_inv": sa, "norm.weight": other, "l0.proj.activation_scale": torch.ones(1, device=device)}
    clean = fd.sanitize_fp8_weights(weights)
    torch.cuda.synchronize()
    assert set(clean) == {"l0.proj.weight", "norm.weight"} and clean["norm.weight"] is other
    np.testing.assert_array_equal(clean["l0.proj.weight"].float().cpu().numpy(), oa.dequant_block_fp8(wa.cpu().numpy(), sa.cpu().numpy()))
    assert fd.sanitize_fp8_weights({"a.weight": other}) == {"a.weight": other}
    with pytest.raises(TypeError):
        ops.dequant_block_fp8(other, to_dev(scale, device), out=out32)


def test_decode_layer_step_end_to_end(device):
    """One decode step of an MLA layer on the kernels of this library, stage by stage as a serving
    loop would run it, against the same chain in float64 (bfloat16 rounding applied where a stage
    hands a bfloat16 tensor to the next):
      append the new token's latent + rope row to the FP8 cache -> causal window indices ->
      q_abs = q_nope . W_UK^T written into the [.., 576] query rows beside q_rope ->
      sparse MLA over the cache -> per-head W_UV -> FP8 block-128 W_O projection."""
    rng = np.random.default_rng(42)
    B, H, D_k, D_kv, R, D_v, D_model, T, topk = 3, 128, 128, 512, 64, 128, 512, 301, 128
    sm_scale = (D_k + R) ** -0.5
    cfg = SparseFP8KVCacheConfig(num_layers=1, batch_size=B, num_kv_heads=1, head_dim=D_kv, max_seq_len=320, rope_dim=R,
                                 scale_block=128, pow2_scales=False)
    cache = SparseFP8KVCache(cfg, device)
    lat_t, lat_f = bf16_pair(rng.standard_normal((B, T, 1, D_kv)), device)
    rope_t, rope_f = bf16_pair(rng.standard_normal((B, T, 1, R)), device)
    cache.append_latent(0, lat_t[:, :T - 1].contiguous(), rope_t[:, :T - 1].contiguous())          # the prompt
    kv, sc, rp = cache.append_latent(0, lat_t[:, T - 1:].contiguous(), rope_t[:, T - 1:].contiguous())   # this step's token
    idx = causal_sparse_indices(B, 1, 1, topk, query_offset=T - 1, key_length=T, device=device)

    w_uk_t, w_uk = bf16_pair(rng.standard_normal((H, D_kv, D_k)) * D_k ** -0.5, device)
    w_uv_t, w_uv = bf16_pair(rng.standard_normal((H, D_kv, D_v)) * D_kv ** -0.5, device)
    w_o_f = (rng.standard_normal((D_model, H * D_v)) * (H * D_v) ** -0.5).astype(np.float32)
    w_o_codes, w_o_scale = fp8.quantize_block(w_o_f, 128, pow2=False)                               # [D_model, H*D_v] e4m3, scale per (row, 128 k)
    q_nope_t, q_nope = bf16_pair(rng.standard_normal((B, 1, H, D_k)), device)
    q_rope_t, q_rope = bf16_pair(rng.standard_normal((B, 1, H, R)), device)

    q_full = torch.empty((B, 1, H, D_kv + R), dtype=torch.bfloat16, device=device)
    q_full[..., D_kv:] = q_rope_t
    ma.absorb_query(q_nope_t, w_uk_t.transpose(1, 2), out=q_full[..., :D_kv])
    o_lat = torch.empty((B, 1, H, D_kv), dtype=torch.bfloat16, device=device)
    ops.sparse_mla_forward(q_full, kv, idx, sm_scale=sm_scale, d_v=D_kv, out=o_lat,
                           kv_spec=ops.QuantSpec(_lib.SCALE_F32_BLOCK, sc, 128), kv_rope=rp)
    o_heads = torch.empty((B, H, D_v), dtype=torch.bfloat16, device=device)
    ops.head_gemm(o_lat.view(B, H, D_kv), w_uv_t.transpose(1, 2).contiguous(), out=o_heads)          # W[h][d][v] = w_uv[h][v][d]
    y = fused_fp8_gemm(to_dev(w_o_codes, device), to_dev(w_o_scale, device), o_heads.view(B, H * D_v))
    torch.cuda.synchronize()
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (B, D_model)

    # the same chain in float64
    codes, scale = okv.quantize_block128(lat_f, pow2=False)
    rows = om.dequant_block_latent(codes, scale, rope_f, 128)                                       # [B, T, 1, 576]
    q_abs = fp8.bf16_round(np.einsum("bthk,hvk->bthv", q_nope, w_uk).astype(np.float32))
    q_cat = np.concatenate([q_abs, q_rope], axis=-1)
    want_lat, _ = om.sparse_mla_oracle(q_cat, rows, idx.cpu().numpy().astype(np.int64), sm_scale=sm_scale, d_v=D_kv)
    err, ref = error_report(o_lat.float().cpu().numpy(), want_lat)
    assert err <= 2e-2 * ref
    err, ref = error_report(q_full[..., :D_kv].float().cpu().numpy(), np.einsum("bthk,hvk->bthv", q_nope, w_uk))
    assert err <= 1e-2 * ref
    o_h = fp8.bf16_round(np.einsum("bthv,hvd->bthd", fp8.bf16_round(want_lat.astype(np.float32)).astype(np.float64), w_uv).astype(np.float32))
    want_y = ovm.fused_fp8_gemm_oracle(w_o_codes, w_o_scale, o_h.reshape(B, H * D_v))
    err, ref = error_report(y.float().cpu().numpy(), want_y)
    assert err <= 2e-2 * ref, (err, ref)
