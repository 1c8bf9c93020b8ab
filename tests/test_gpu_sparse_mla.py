"""GPU parity: sparse-MLA forward (through the C ABI) vs the float64 oracle.

Tolerance (stated by the task): max-abs error <= 2e-2 relative to the output
scale max|oracle| for bf16/fp16 outputs; the reference's own block-scaled
budget atol 2e-2 / rtol 5e-2 is checked as well.  fp32 outputs of the fp32
kernel are held to 1e-4 of the output scale.  lse (fp32) to 1e-3 absolute for
the fp32-arithmetic kernel and 5e-3 for the bf16 MFMA kernel, whose scores carry
the bf16 rounding of the dequantised keys (|score| * 2^-9)."""

import numpy as np
import pytest
import torch

from cppmega_mlx_amd import ops
from cppmega_mlx_amd.nn import sparse_mla as mla
from cppmega_mlx_amd.nn._tilelang import (
    sparse_mla_blockscaled_path_c as bs,
    sparse_mla_fp8_path_c as f8,
    sparse_mla_path_c as pc,
)
from oracle import fp8, sparse_mla as om
from tests._inputs import bf16_pair, error_report, latent_cache, sparse_indices, to_dev

pytestmark = pytest.mark.gpu

REL_TOL = 2e-2
LSE_TOL = 1e-3
LSE_TOL_MFMA = 5e-3


def _assert_close(out_t, lse_t, want_out, want_lse, *, rel=REL_TOL, lse_tol=LSE_TOL):
    got = out_t.float().cpu().numpy()
    assert not np.isnan(got).any()
    err, ref = error_report(got, want_out)
    assert err <= rel * ref, f"max-abs {err:.3e} vs output scale {ref:.3e}"
    if rel == REL_TOL:
        np.testing.assert_allclose(got, want_out, atol=2e-2, rtol=5e-2)
    if lse_t is not None:
        assert np.abs(lse_t.cpu().numpy() - want_lse).max() <= lse_tol


# shapes of the reference's own parity grid (tests/test_tilelang_sparse_mla.py:164-186) plus wider ones
SMOKE = [
    dict(B=1, S=4, H=4, G=1, Skv=32, topk=8, D=64, d_v=64),
    dict(B=2, S=8, H=8, G=2, Skv=64, topk=16, D=64, d_v=64),
    dict(B=1, S=5, H=4, G=2, Skv=40, topk=16, D=64, d_v=48),      # tail_dim 16
    dict(B=1, S=3, H=6, G=3, Skv=300, topk=100, D=128, d_v=32),
]


@pytest.mark.parametrize("shape", SMOKE)
@pytest.mark.parametrize("carrier", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("kernel", ["scalar", "auto"])
def test_float_carriers(device, shape, carrier, kernel):
    rng = np.random.default_rng(hash((shape["Skv"], shape["D"], str(carrier))) % 2 ** 31)
    B, S, H, G, Skv, topk, D, d_v = (shape[k] for k in ("B", "S", "H", "G", "Skv", "topk", "D", "d_v"))
    q = to_dev(rng.standard_normal((B, S, H, D)).astype(np.float32), device).to(carrier)
    kv = to_dev(rng.standard_normal((B, Skv, G, D)).astype(np.float32), device).to(carrier)
    idx = sparse_indices(rng, B, S, G, Skv, topk, replace=True)      # the reference samples with replacement
    idx[rng.random(idx.shape) < 0.2] = -1
    idx[0, 1] = -1                                                   # an all-invalid query
    want_out, want_lse = om.sparse_mla_oracle(q.float().cpu().numpy(), kv.float().cpu().numpy(), idx, d_v=d_v)
    out = torch.zeros((B, S, H, d_v), dtype=carrier, device=device)
    lse = torch.zeros((B, S, H), dtype=torch.float32, device=device)
    ops.sparse_mla_forward(q, kv, to_dev(idx.astype(np.int32), device), sm_scale=D ** -0.5, d_v=d_v, out=out, lse=lse,
                           kernel=kernel)
    torch.cuda.synchronize()
    _assert_close(out, lse, want_out, want_lse, rel=1e-4 if carrier == torch.float32 else REL_TOL)
    assert (out[0, 1] == 0).all() and (lse[0, 1] == 0).all()


def test_public_float_entry_points_and_int64_indices(device):
    rng = np.random.default_rng(11)
    B, S, H, G, Skv, topk, D = 2, 4, 4, 2, 48, 12, 64
    q, qf = bf16_pair(rng.standard_normal((B, S, H, D)), device)
    kv, kvf = bf16_pair(rng.standard_normal((B, Skv, G, D)), device)
    idx = sparse_indices(rng, B, S, G, Skv, topk)
    idx[..., -3:] = -1
    want_out, want_lse = om.sparse_mla_oracle(qf, kvf, idx, sm_scale=0.2, d_v=32)
    i64 = to_dev(idx, device)
    for fn in (mla.sparse_mla_attention_reference, mla.sparse_mla_attention, pc.sparse_mla_path_c_apply):
        out, lse = fn(q, kv, i64, sm_scale=0.2, d_v=32, return_lse=True)
        torch.cuda.synchronize()
        assert out.dtype == torch.bfloat16 and tuple(out.shape) == (B, S, H, 32)
        _assert_close(out, lse, want_out, want_lse)
    out = torch.zeros((B, S, H, 32), dtype=torch.float32, device=device)
    lse = torch.zeros((B, S, H), dtype=torch.float32, device=device)
    o, l = pc.sparse_mla_fwd_path_c(q, kv, i64, sm_scale_buf=torch.tensor([0.2], device=device), out=out, lse=lse, d_v=32)
    torch.cuda.synchronize()
    assert o is out and l is lse
    _assert_close(out, lse, want_out, want_lse)


@pytest.mark.parametrize("shape", SMOKE[:3])
def test_e8m0_block_scaled_prepared_buffers(device, shape):
    rng = np.random.default_rng(21 + shape["Skv"])
    B, S, H, G, Skv, topk, D, d_v = (shape[k] for k in ("B", "S", "H", "G", "Skv", "topk", "D", "d_v"))
    qc, qb = fp8.quantize_mxfp8(rng.standard_normal((B, S, H, D)).astype(np.float32) * 0.1)
    kc, kb = fp8.quantize_mxfp8(rng.standard_normal((B, Skv, G, D)).astype(np.float32) * 0.1)
    kb[0, 0, 0, 0] = 0                                               # E8M0 byte 0 decodes to 0
    idx = sparse_indices(rng, B, S, G, Skv, topk, replace=True)
    idx[..., -2:] = -1
    idx[0, 0, 0, 0] = Skv + 3                                        # out-of-range index is skipped too
    want_out, want_lse = om.sparse_mla_oracle(om.dequant_e8m0(qc, qb), om.dequant_e8m0(kc, kb), idx, d_v=d_v)
    out = torch.zeros((B, S, H, d_v), dtype=torch.float16, device=device)
    lse = torch.zeros((B, S, H), dtype=torch.float32, device=device)
    o, l = bs.sparse_mla_blockscaled_path_c_apply(
        to_dev(qc, device), to_dev(qb, device), to_dev(kc, device), to_dev(kb, device), to_dev(idx.astype(np.int32), device),
        sm_scale=D ** -0.5, d_v=d_v, return_lse=True, out=out, lse=lse)
    torch.cuda.synchronize()
    assert o is out and l is lse
    _assert_close(out, lse, want_out, want_lse)
    alloc = bs.sparse_mla_blockscaled_path_c_apply(
        to_dev(qc, device), to_dev(qb, device), to_dev(kc, device), to_dev(kb, device), to_dev(idx, device),
        sm_scale=D ** -0.5, d_v=d_v, force_path_c=True)
    torch.cuda.synchronize()
    assert alloc.dtype == torch.float16
    _assert_close(alloc, None, want_out, want_lse)


@pytest.mark.parametrize("with_sinks", [False, True])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_per_token_fp8_prepared_buffers_with_sinks(device, with_sinks, out_dtype):
    rng = np.random.default_rng(31)
    B, S, H, G, Skv, topk, D, d_v = 1, 6, 4, 2, 40, 16, 64, 32
    qc, qs = fp8.quantize_per_token(rng.standard_normal((B, S, H, D)).astype(np.float32))
    kc, ks = fp8.quantize_per_token(rng.standard_normal((B, Skv, G, D)).astype(np.float32))
    idx = sparse_indices(rng, B, S, G, Skv, topk, replace=True)
    idx[0, 2] = -1
    sinks = rng.standard_normal(H).astype(np.float32) if with_sinks else None
    want_out, want_lse = om.sparse_mla_oracle(om.dequant_per_token(qc, qs), om.dequant_per_token(kc, ks), idx, d_v=d_v,
                                              sinks=sinks)
    out, lse = f8.sparse_mla_fp8_path_c_apply(
        to_dev(qc, device), to_dev(qs, device), to_dev(kc, device), to_dev(ks, device), to_dev(idx.astype(np.int32), device),
        sm_scale=D ** -0.5, d_v=d_v, sinks=None if sinks is None else to_dev(sinks, device), return_lse=True,
        output_dtype=out_dtype)
    torch.cuda.synchronize()
    assert out.dtype == out_dtype
    _assert_close(out, lse, want_out, want_lse, rel=1e-4 if out_dtype == torch.float32 else REL_TOL)
    if with_sinks:                                                   # all-invalid row: out 0, lse = sink
        assert (out[0, 2] == 0).all()
        np.testing.assert_allclose(lse[0, 2].cpu().numpy(), sinks, atol=1e-6)


@pytest.mark.parametrize("shape", [
    dict(B=1, S=4, H=16, G=1, Skv=256, topk=64),
    dict(B=2, S=3, H=40, G=1, Skv=700, topk=333),             # a partial head group, ragged tiles
    dict(B=1, S=2, H=64, G=2, Skv=5000, topk=2048),           # two KV groups, key splits + combine
    dict(B=1, S=3, H=128, G=1, Skv=3000, topk=1000),          # 4 head groups share one key stream
    dict(B=2, S=2, H=144, G=2, Skv=900, topk=130),            # 72 heads per KV group: a wavefront without heads
    dict(B=1, S=2, H=160, G=1, Skv=9000, topk=4096),          # two workgroups per query, key splits
    dict(B=1, S=2, H=64, G=1, Skv=100, topk=7),               # less than one tile
], ids=["h16", "h40_ragged", "g2_splits", "h128", "h144_g2", "h160_splits", "h64_tiny"])
@pytest.mark.parametrize("with_sinks", [False, True], ids=["plain", "sinks"])
def test_mfma_kernel_per_token_fp8_rows(device, shape, with_sinks):
    """Per-token FP8 prepared buffers at the attention shape (rows of 576 codes, d_v 512; reference:
    cppmega_mlx/nn/_tilelang/sparse_mla_fp8_path_c.py:1701-3004) on the matrix cores: codes enter the
    products exactly, the scales multiply the scores, so the result is held to the fp32 kernel's lse bound."""
    rng = np.random.default_rng(shape["H"] * 11 + shape["topk"] + with_sinks)
    B, S, H, G, Skv, topk = (shape[k] for k in ("B", "S", "H", "G", "Skv", "topk"))
    qc, qs = fp8.quantize_per_token(rng.standard_normal((B, S, H, 576)).astype(np.float32) * 3.0)
    kc, ks = fp8.quantize_per_token(rng.standard_normal((B, Skv, G, 576)).astype(np.float32) * 0.5)
    idx = sparse_indices(rng, B, S, G, Skv, topk, replace=True)
    idx[rng.random(idx.shape) < 0.15] = -1
    idx[0, 1] = -1
    sinks = rng.standard_normal(H).astype(np.float32) if with_sinks else None
    want_out, want_lse = om.sparse_mla_oracle(om.dequant_per_token(qc, qs), om.dequant_per_token(kc, ks), idx,
                                              sm_scale=576 ** -0.5, d_v=512, sinks=sinks)
    out = torch.zeros((B, S, H, 512), dtype=torch.bfloat16, device=device)
    lse = torch.zeros((B, S, H), dtype=torch.float32, device=device)
    got = f8.sparse_mla_fp8_path_c_apply_direct(
        to_dev(qc, device), to_dev(qs, device), to_dev(kc, device), to_dev(ks, device), to_dev(idx.astype(np.int32), device),
        sm_scale=576 ** -0.5, d_v=512, out=out, lse=lse, sinks=None if sinks is None else to_dev(sinks, device), kernel="mfma")
    torch.cuda.synchronize()
    assert got[0] is out and got[1] is lse
    _assert_close(out, lse, want_out, want_lse, lse_tol=LSE_TOL)
    if with_sinks:
        assert (out[0, 1] == 0).all()
        np.testing.assert_allclose(lse[0, 1].cpu().numpy(), sinks, atol=1e-6)
    else:
        assert (out[0, 1] == 0).all() and (lse[0, 1] == 0).all()


@pytest.mark.parametrize("shape", [
    dict(B=1, S=4, H=16, G=1, Skv=255, topk=64),              # an odd number of rows: the last row's scale bytes end the buffer
    dict(B=2, S=3, H=40, G=1, Skv=700, topk=333),
    dict(B=1, S=2, H=64, G=2, Skv=5000, topk=2048),
    dict(B=1, S=3, H=128, G=1, Skv=3000, topk=1000),
    dict(B=2, S=2, H=144, G=2, Skv=901, topk=130),
    dict(B=1, S=2, H=64, G=1, Skv=100, topk=7),
], ids=["h16_odd_rows", "h40_ragged", "g2_splits", "h128", "h144_g2", "h64_tiny"])
def test_mfma_kernel_e8m0_rows(device, shape):
    """E8M0-per-32 prepared buffers at the attention shape (rows of 576 codes + 18 scale bytes, d_v 512;
    reference: cppmega_mlx/nn/_tilelang/sparse_mla_blockscaled_path_c.py:943-1504) on the matrix cores.
    A power of two times an e4m3 code is a bfloat16: the operands enter the products exactly."""
    rng = np.random.default_rng(shape["H"] * 13 + shape["topk"])
    B, S, H, G, Skv, topk = (shape[k] for k in ("B", "S", "H", "G", "Skv", "topk"))
    qc, qb = fp8.quantize_mxfp8(rng.standard_normal((B, S, H, 576)).astype(np.float32) * 2.0)
    kc, kb = fp8.quantize_mxfp8(rng.standard_normal((B, Skv, G, 576)).astype(np.float32) *
                                np.exp2(rng.integers(-6, 3, size=(B, Skv, G, 1))).astype(np.float32))
    kb[0, 0, 0, 0] = 0                                               # E8M0 byte 0 decodes to 0
    kb[0, 1, 0, 17] = 255                                            # ... and so does 255
    idx = sparse_indices(rng, B, S, G, Skv, topk, replace=True)
    idx[rng.random(idx.shape) < 0.15] = -1
    idx[0, 1] = -1
    idx[0, 0, 0, :4] = [0, 1, Skv - 1, Skv + 3]                      # the patched rows, the last row, one out of range
    want_out, want_lse = om.sparse_mla_oracle(om.dequant_e8m0(qc, qb), om.dequant_e8m0(kc, kb), idx,
                                              sm_scale=576 ** -0.5, d_v=512)
    out = torch.zeros((B, S, H, 512), dtype=torch.bfloat16, device=device)
    lse = torch.zeros((B, S, H), dtype=torch.float32, device=device)
    got = bs.sparse_mla_blockscaled_path_c_apply_direct(
        to_dev(qc, device), to_dev(qb, device), to_dev(kc, device), to_dev(kb, device), to_dev(idx.astype(np.int32), device),
        sm_scale=576 ** -0.5, d_v=512, out=out, lse=lse, kernel="mfma")
    torch.cuda.synchronize()
    assert got[0] is out and got[1] is lse
    _assert_close(out, lse, want_out, want_lse, lse_tol=LSE_TOL)
    assert (out[0, 1] == 0).all() and (lse[0, 1] == 0).all()


def _latent_case(device, rng, *, B, S, H, Skv, topk, pow2, causal_offset=None, d_latent=512, d_rope=64):
    q, qf = bf16_pair(rng.standard_normal((B, S, H, d_latent + d_rope)), device)
    codes, scale, rope, rows = latent_cache(rng, B, Skv, 1, d_latent, d_rope, device, pow2=pow2)
    idx = sparse_indices(rng, B, S, 1, Skv, topk, causal_offset=causal_offset)
    return q, qf, codes, scale, rope, rows, idx


@pytest.mark.parametrize("kernel", ["scalar", "auto"])
@pytest.mark.parametrize("pow2", [True, False])
def test_latent_cache_layout_small(device, kernel, pow2):
    rng = np.random.default_rng(41 + pow2)
    B, S, H, Skv, topk = 2, 3, 16, 200, 70
    q, qf, codes, scale, rope, rows, idx = _latent_case(device, rng, B=B, S=S, H=H, Skv=Skv, topk=topk, pow2=pow2,
                                                        causal_offset=40)
    want_out, want_lse = om.sparse_mla_oracle(qf, rows, idx, sm_scale=576 ** -0.5, d_v=512)
    out = torch.zeros((B, S, H, 512), dtype=torch.bfloat16, device=device)
    lse = torch.zeros((B, S, H), dtype=torch.float32, device=device)
    bs.sparse_mla_blockscaled_path_c_apply(q, None, codes, scale, to_dev(idx.astype(np.int32), device),
                                           sm_scale=576 ** -0.5, d_v=512, out=out, lse=lse, kv_rope=rope, kernel=kernel)
    torch.cuda.synchronize()
    _assert_close(out, lse, want_out, want_lse, lse_tol=LSE_TOL if kernel == "scalar" else LSE_TOL_MFMA)


# (B, S, H, G, Skv, topk, pow2 scales, causal offset, sinks): cases that exercise the MFMA kernel's
# head groups, key splits, ragged last tiles, masked tiles and the sink/lse epilogues
MFMA_CASES = [
    (1, 1, 32, 1, 64, 16, True, None, False),          # one tile, one wavefront busy
    (1, 2, 32, 1, 300, 64, True, None, False),         # one tile per wavefront
    (2, 3, 128, 1, 500, 200, True, 50, False),         # four head groups, ragged tiles, causal padding
    (2, 3, 128, 1, 500, 200, False, 50, True),         # general fp32 scales + sinks
    (1, 2, 64, 2, 400, 130, True, None, False),        # two KV groups
    (1, 2, 48, 1, 256, 100, False, None, True),        # head count not a multiple of 32
    (4, 1, 128, 1, 4096, 2048, True, None, False),     # decode shape at reduced batch: key splits + combine
    (2, 1, 128, 1, 4096, 2048, False, None, True),     # key splits with sinks and general scales
    (1, 1, 128, 1, 36000, 34000, True, None, False),   # more keys than 16 splits of the shared-tile kernel hold
    (1, 3, 96, 1, 700, 300, False, 100, False),        # a second head chunk of 32 heads only
]


@pytest.mark.parametrize("case", MFMA_CASES)
def test_mfma_kernel_latent_cache(device, case):
    B, S, H, G, Skv, topk, pow2, causal, with_sinks = case
    rng = np.random.default_rng(hash(case) % 2 ** 31)
    q, qf = bf16_pair(rng.standard_normal((B, S, H, 576)), device)
    codes, scale, rope, rows = latent_cache(rng, B, Skv, G, 512, 64, device, pow2=pow2)
    idx = sparse_indices(rng, B, S, G, Skv, topk, causal_offset=causal)
    sinks = rng.standard_normal(H).astype(np.float32) if with_sinks else None
    want_out, want_lse = om.sparse_mla_oracle(qf, rows, idx, sm_scale=576 ** -0.5, d_v=512, sinks=sinks)
    out = torch.zeros((B, S, H, 512), dtype=torch.bfloat16, device=device)
    lse = torch.zeros((B, S, H), dtype=torch.float32, device=device)
    from cppmega_mlx_amd import _lib
    ops.sparse_mla_forward(q, codes, to_dev(idx.astype(np.int32), device), sm_scale=576 ** -0.5, d_v=512, out=out, lse=lse,
                           kv_spec=ops.QuantSpec(_lib.SCALE_F32_BLOCK, scale, 128), kv_rope=rope,
                           sinks=None if sinks is None else to_dev(sinks, device), kernel="mfma")
    torch.cuda.synchronize()
    _assert_close(out, lse, want_out, want_lse, lse_tol=LSE_TOL_MFMA)


def test_mfma_kernel_matches_scalar_kernel_bf16_cache(device):
    """bf16 KV rows (no quantisation): both kernels see identical inputs."""
    rng = np.random.default_rng(77)
    B, S, H, Skv, topk = 1, 4, 16, 256, 64
    q, qf = bf16_pair(rng.standard_normal((B, S, H, 576)), device)
    kv, kvf = bf16_pair(rng.standard_normal((B, Skv, 1, 576)), device)
    idx = sparse_indices(rng, B, S, 1, Skv, topk, causal_offset=0)
    want_out, want_lse = om.sparse_mla_oracle(qf, kvf, idx, sm_scale=576 ** -0.5, d_v=512)
    for kernel in ("scalar", "mfma"):
        out = torch.zeros((B, S, H, 512), dtype=torch.bfloat16, device=device)
        lse = torch.zeros((B, S, H), dtype=torch.float32, device=device)
        ops.sparse_mla_forward(q, kv, to_dev(idx.astype(np.int32), device), sm_scale=576 ** -0.5, d_v=512, out=out, lse=lse,
                               kernel=kernel)
        torch.cuda.synchronize()
        _assert_close(out, lse, want_out, want_lse, lse_tol=LSE_TOL if kernel == "scalar" else LSE_TOL_MFMA)


@pytest.mark.parametrize("shape", [
    dict(B=1, S=4, H=16, G=1, Skv=256, topk=64),
    dict(B=2, S=3, H=40, G=1, Skv=700, topk=333),             # a partial head group, ragged tiles
    dict(B=1, S=2, H=64, G=2, Skv=5000, topk=2048),           # two KV groups, key splits + combine
    dict(B=1, S=3, H=128, G=1, Skv=3000, topk=1000),          # 4 head groups share one key stream
    dict(B=2, S=2, H=144, G=2, Skv=900, topk=130),            # 72 heads per KV group: 32 + 32 + 8, a wavefront without heads
    dict(B=1, S=2, H=160, G=1, Skv=9000, topk=4096),          # 5 head groups: two workgroups per query, key splits
    dict(B=1, S=2, H=64, G=1, Skv=100, topk=7),               # less than one tile
], ids=["h16", "h40_ragged", "g2_splits", "h128_shared", "h144_g2_shared", "h160_shared_splits", "h64_tiny"])
@pytest.mark.parametrize("rope_tail", [False, True], ids=["packed576", "latent_plus_rope"])
def test_mfma_kernel_float16_rows(device, shape, rope_tail):
    """float16 queries and rows of 576 (the carrier the reference's float Path C kernels compute in,
    cppmega_mlx/nn/_tilelang/sparse_mla_path_c.py) on the float16 matrix instructions."""
    rng = np.random.default_rng(shape["H"] * 7 + shape["topk"] + rope_tail)
    B, S, H, G, Skv, topk = (shape[k] for k in ("B", "S", "H", "G", "Skv", "topk"))
    q = to_dev(rng.standard_normal((B, S, H, 576)).astype(np.float32), device).to(torch.float16)
    kv = to_dev(rng.standard_normal((B, Skv, G, 576)).astype(np.float32), device).to(torch.float16)
    idx = sparse_indices(rng, B, S, G, Skv, topk, replace=True)
    idx[rng.random(idx.shape) < 0.15] = -1
    idx[0, 1] = -1
    want_out, want_lse = om.sparse_mla_oracle(q.float().cpu().numpy(), kv.float().cpu().numpy(), idx,
                                              sm_scale=576 ** -0.5, d_v=512)
    kw = {}
    rows = kv
    if rope_tail:
        rows = kv[..., :512].contiguous()
        kw["kv_rope"] = kv[..., 512:].contiguous()
    out = torch.zeros((B, S, H, 512), dtype=torch.float16, device=device)
    lse = torch.zeros((B, S, H), dtype=torch.float32, device=device)
    ops.sparse_mla_forward(q, rows, to_dev(idx.astype(np.int32), device), sm_scale=576 ** -0.5, d_v=512, out=out,
                           lse=lse, kernel="mfma", **kw)
    torch.cuda.synchronize()
    _assert_close(out, lse, want_out, want_lse, lse_tol=LSE_TOL_MFMA)
    assert (out[0, 1] == 0).all() and (lse[0, 1] == 0).all()


def test_shared_key_stream_int64_indices_and_cache_views(device):
    """128 heads on bf16 rows of 576: int64 indices, and the rows passed as the live prefix of a larger
    cache buffer (batch pitch = capacity), as `update_and_fetch` hands them out."""
    rng = np.random.default_rng(4242)
    B, S, H, cap, Skv, topk = 2, 3, 128, 600, 500, 200
    q, qf = bf16_pair(rng.standard_normal((B, S, H, 576)), device)
    buf, buf_f = bf16_pair(rng.standard_normal((B, cap, 1, 576)), device)
    kv = buf[:, :Skv]
    idx = sparse_indices(rng, B, S, 1, Skv, topk, replace=True)
    idx[rng.random(idx.shape) < 0.1] = -1
    idx[1, 0, 0, :3] = [Skv, Skv + 50, cap - 1]                      # beyond the live length: skipped, though inside the buffer
    want_out, want_lse = om.sparse_mla_oracle(qf, buf_f[:, :Skv], idx, sm_scale=576 ** -0.5, d_v=512)
    out = torch.zeros((B, S, H, 512), dtype=torch.bfloat16, device=device)
    lse = torch.zeros((B, S, H), dtype=torch.float32, device=device)
    ops.sparse_mla_forward(q, kv, to_dev(idx.astype(np.int64), device), sm_scale=576 ** -0.5, d_v=512, out=out, lse=lse,
                           kernel="mfma")
    torch.cuda.synchronize()
    _assert_close(out, lse, want_out, want_lse, lse_tol=LSE_TOL_MFMA)


@pytest.mark.parametrize("pow2", [True, False], ids=["pow2_scales", "general_scales"])
def test_decode_full_config_sampled_batches(device, pow2):
    """B=32, S_q=1, H=128, topk=2048 over a 65536-token FP8 cache (the headline
    workload) with power-of-two and with general amax/448 block scales: every batch
    runs on the GPU, five of them are checked against the oracle, and the rest
    through properties: permuting a query's selected keys leaves its output
    unchanged (to accumulation order), and appending masked (-1) slots changes
    nothing."""
    from cppmega_mlx_amd import _lib
    B, H, Skv, topk = 32, 128, 65536, 2048
    gen = torch.Generator(device=device).manual_seed(5)
    codes = torch.empty((B, Skv, 1, 512), dtype=torch.uint8, device=device)
    scale = torch.empty((B, Skv, 1, 4), dtype=torch.float32, device=device)
    rope = torch.empty((B, Skv, 1, 64), dtype=torch.bfloat16, device=device)
    for b in range(B):
        lat = torch.randn((Skv, 1, 4, 128), generator=gen, device=device)
        sc = lat.abs().amax(dim=-1) / 448.0
        if pow2:
            sc = torch.exp2(torch.ceil(torch.log2(sc)))
        codes[b] = (lat / sc[..., None]).to(torch.float8_e4m3fn).view(torch.uint8).reshape(Skv, 1, 512)
        scale[b] = sc
        rope[b] = torch.randn((Skv, 1, 64), generator=gen, device=device).to(torch.bfloat16)
    q = torch.randn((B, 1, H, 576), generator=gen, device=device).to(torch.bfloat16)
    idx = torch.stack([torch.randperm(Skv, generator=gen, device=device)[:topk] for _ in range(B)]).to(torch.int32)
    idx = idx.reshape(B, 1, 1, topk).contiguous()
    spec = ops.QuantSpec(_lib.SCALE_F32_BLOCK, scale, 128)

    def run(indices):
        out = torch.zeros((B, 1, H, 512), dtype=torch.bfloat16, device=device)
        lse = torch.zeros((B, 1, H), dtype=torch.float32, device=device)
        ops.sparse_mla_forward(q, codes, indices, sm_scale=576 ** -0.5, d_v=512, out=out, lse=lse, kv_spec=spec, kv_rope=rope)
        torch.cuda.synchronize()
        return out.float().cpu().numpy(), lse.cpu().numpy()

    got_out, got_lse = run(idx)
    assert ops.sparse_mla_selected_kernel(q, codes, idx, d_v=512, kv_spec=spec, kv_rope=rope) == "mfma"
    for b in (0, 7, 13, 22, 31):
        sel = idx[b, 0, 0].cpu().numpy().astype(np.int64)
        rows = om.dequant_block_latent(codes[b, sel].cpu().numpy(), scale[b, sel].cpu().numpy(),
                                       rope[b, sel].float().cpu().numpy(), 128)[None]
        local = np.arange(topk, dtype=np.int64).reshape(1, 1, 1, topk)
        want_out, want_lse = om.sparse_mla_oracle(q[b:b + 1].float().cpu().numpy(), rows, local, sm_scale=576 ** -0.5, d_v=512)
        err, ref = error_report(got_out[b:b + 1], want_out)
        assert err <= REL_TOL * ref, f"batch {b}: max-abs {err:.3e} vs output scale {ref:.3e}"
        assert np.abs(got_lse[b:b + 1] - want_lse).max() <= LSE_TOL_MFMA
    perm = torch.randperm(topk, generator=gen, device=device)
    out_p, lse_p = run(idx[..., perm].contiguous())
    scale_ref = np.abs(got_out).max()
    assert np.abs(out_p - got_out).max() <= REL_TOL * scale_ref
    assert np.abs(lse_p - got_lse).max() <= 1e-4
    padded = torch.cat([idx, torch.full((B, 1, 1, 64), -1, dtype=torch.int32, device=device)], dim=-1).contiguous()
    out_m, lse_m = run(padded)
    assert np.abs(out_m - got_out).max() <= REL_TOL * scale_ref
    assert np.abs(lse_m - got_lse).max() <= 1e-4


@pytest.mark.parametrize("pow2", [True, False], ids=["pow2_scales", "general_scales"])
def test_prefill_full_config_sampled_queries(device, pow2):
    """B=1, S=8192, H=128, topk=2048 with causal top-k indices over an 8192-token FP8 cache: the
    whole chunk runs on the GPU (indices from the GPU selector), sampled queries -- heavily
    padded early ones, the 2047/2048 boundary, the last -- are checked against the oracle, and
    every query with no visible key beyond itself must reproduce its own value row.  Block scales
    are powers of two (2^ceil(log2(amax/448))) or general fp32 values (amax/448)."""
    from cppmega_mlx_amd import _lib
    from cppmega_mlx_amd.nn._tilelang import topk_selector as tk
    S, H, topk = 8192, 128, 2048
    gen = torch.Generator(device=device).manual_seed(17)
    lat = torch.randn((S, 1, 4, 128), generator=gen, device=device)
    amax = lat.abs().amax(dim=-1)
    sc = torch.exp2(torch.ceil(torch.log2(amax / 448.0))) if pow2 else amax / 448.0
    codes = (lat / sc[..., None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).reshape(1, S, 1, 512)
    scale = sc.reshape(1, S, 1, 4).contiguous()
    rope = torch.randn((1, S, 1, 64), generator=gen, device=device).to(torch.bfloat16)
    q = torch.randn((1, S, H, 576), generator=gen, device=device).to(torch.bfloat16)
    ends = torch.arange(1, S + 1, device=device, dtype=torch.int32)
    idx = torch.empty((S, topk), dtype=torch.int32, device=device)
    tk.topk_selector_tilelang_direct(torch.randn((S, S), generator=gen, device=device), topk, out=idx, ends=ends, order="index")
    idx = idx.view(1, S, 1, topk)
    spec = ops.QuantSpec(_lib.SCALE_F32_BLOCK, scale, 128)
    out = torch.zeros((1, S, H, 512), dtype=torch.bfloat16, device=device)
    lse = torch.zeros((1, S, H), dtype=torch.float32, device=device)
    ops.sparse_mla_forward(q, codes, idx, sm_scale=576 ** -0.5, d_v=512, out=out, lse=lse, kv_spec=spec, kv_rope=rope)
    torch.cuda.synchronize()
    assert ops.sparse_mla_selected_kernel(q, codes, idx, d_v=512, kv_spec=spec, kv_rope=rope) == "mfma"
    idx_np = idx.cpu().numpy().astype(np.int64)
    assert ((idx_np[0, :, 0, :] >= 0).sum(axis=-1) == np.minimum(np.arange(1, S + 1), topk)).all()
    rows_all = om.dequant_block_latent(codes.cpu().numpy(), scale.cpu().numpy(), rope.float().cpu().numpy(), 128)
    for s in (0, 1, 31, 33, 700, 2046, 2047, 2048, 5000, S - 1):
        want_out, want_lse = om.sparse_mla_oracle(q[:, s:s + 1].float().cpu().numpy(), rows_all, idx_np[:, s:s + 1],
                                                  sm_scale=576 ** -0.5, d_v=512)
        err, ref = error_report(out[:, s:s + 1].float().cpu().numpy(), want_out)
        assert err <= REL_TOL * ref, f"query {s}: max-abs {err:.3e} vs output scale {ref:.3e}"
        assert np.abs(lse[:, s:s + 1].cpu().numpy() - want_lse).max() <= LSE_TOL_MFMA, f"query {s}"
    # query 0 sees only key 0: softmax over one key is 1, the output is that key's value row for every head
    v0 = rows_all[0, 0, 0, :512]
    got0 = out[0, 0].float().cpu().numpy()
    assert np.abs(got0 - v0[None, :]).max() <= 2.0 ** -8 * np.abs(v0).max() + 1e-6     # bf16 rounding of the output
    assert not torch.isnan(out.float()).any()


def test_tiny_bf16_config(device):
    """B=1, S_q=64, H=16, d_qk=576, d_v=512, Skv=256, topk=64, causal sampling, both windows."""
    for off in (0, 192):
        rng = np.random.default_rng(64 + off)
        q, qf = bf16_pair(rng.standard_normal((1, 64, 16, 576)), device)
        kv, kvf = bf16_pair(rng.standard_normal((1, 256, 1, 576)), device)
        idx = sparse_indices(rng, 1, 64, 1, 256, 64, causal_offset=off)
        want_out, want_lse = om.sparse_mla_oracle(qf, kvf, idx, sm_scale=576 ** -0.5, d_v=512)
        out, lse = mla.sparse_mla_attention(q, kv, to_dev(idx.astype(np.int32), device), sm_scale=576 ** -0.5, d_v=512,
                                            return_lse=True)
        torch.cuda.synchronize()
        _assert_close(out, lse, want_out, want_lse, lse_tol=LSE_TOL_MFMA)
        if off == 0:
            assert (idx[0, 0, 0] >= 0).sum() == 1                    # first query sees one key: out == that V row
            np.testing.assert_allclose(out[0, 0].float().cpu().numpy(), np.broadcast_to(kvf[0, idx[0, 0, 0, 0], 0, :512], (16, 512)),
                                       atol=2e-2, rtol=1e-2)


def test_score_only_entry_points(device):
    """QK-only seams: per-token FP8 indexed scores, the (1, N) FP8 reducer and the E8M0 reducer."""
    rng = np.random.default_rng(91)
    B, S, H, G, Skv, topk, D = 2, 3, 8, 2, 50, 20, 64
    qc, qs = fp8.quantize_per_token(rng.standard_normal((B, S, H, D)).astype(np.float32))
    kc, ks = fp8.quantize_per_token(rng.standard_normal((B, Skv, G, D)).astype(np.float32))
    idx = sparse_indices(rng, B, S, G, Skv, topk, replace=True)
    idx[..., -3:] = -1
    idx[0, 0, 0, 0] = Skv + 5
    want = om.sparse_mla_scores_oracle(om.dequant_per_token(qc, qs), om.dequant_per_token(kc, ks), idx, sm_scale=0.125)
    got = f8.fp8_sparse_mla_indexed_qk_reduce_path_c(to_dev(qc, device), to_dev(qs, device), to_dev(kc, device),
                                                     to_dev(ks, device), to_dev(idx.astype(np.int32), device), sm_scale=0.125)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    bad = want == om.INVALID_SCORE_SENTINEL
    assert (got[bad] == om.INVALID_SCORE_SENTINEL).all()
    np.testing.assert_allclose(got[~bad], want[~bad], rtol=1e-5, atol=1e-5)

    N, K = 37, 128
    a, a_s = fp8.quantize_per_token(rng.standard_normal((1, K)).astype(np.float32))
    bm, b_s = fp8.quantize_per_token(rng.standard_normal((N, K)).astype(np.float32))
    want2 = (fp8.e4m3_decode(bm).astype(np.float64) @ fp8.e4m3_decode(a[0]).astype(np.float64)) * float(a_s[0]) * b_s.astype(np.float64)
    got2 = f8.fp8_sparse_mla_qk_reduce_path_c(to_dev(a, device), to_dev(a_s.reshape(1), device), to_dev(bm, device), to_dev(b_s, device))
    torch.cuda.synchronize()
    assert tuple(got2.shape) == (1, N)
    np.testing.assert_allclose(got2.cpu().numpy()[0], want2, rtol=1e-5, atol=1e-5)

    ac, ab = fp8.quantize_mxfp8(rng.standard_normal((1, K)).astype(np.float32))
    bc, bb = fp8.quantize_mxfp8(rng.standard_normal((N, K)).astype(np.float32))
    want3 = om.dequant_e8m0(bc, bb).astype(np.float64) @ om.dequant_e8m0(ac, ab)[0].astype(np.float64)
    got3 = bs.blockscaled_sparse_mla_qk_reduce_path_c(to_dev(ac, device), to_dev(ab.reshape(-1), device), to_dev(bc, device), to_dev(bb, device))
    torch.cuda.synchronize()
    np.testing.assert_allclose(got3.cpu().numpy()[0], want3, rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError):
        f8.fp8_sparse_mla_qk_reduce_path_c(to_dev(a, device), to_dev(a_s.reshape(1), device), to_dev(bm[:, :64].copy(), device), to_dev(b_s, device))
    with pytest.raises(TypeError):
        bs.blockscaled_sparse_mla_qk_reduce_path_c(to_dev(ac, device), to_dev(ab.reshape(-1).astype(np.float32), device), to_dev(bc, device), to_dev(bb, device))
