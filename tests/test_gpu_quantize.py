"""GPU parity: FP8 producers (through the C ABI) vs the NumPy oracle, bit for bit, and the
float-carrier attention wrappers built on them."""

import numpy as np
import pytest
import torch

from cppmega_mlx_amd import ops
from cppmega_mlx_amd.nn._tilelang import sparse_mla_blockscaled as fbs, sparse_mla_fp8 as ff8
from oracle import fp8, sparse_mla as om
from tests._inputs import sparse_indices, to_dev

pytestmark = pytest.mark.gpu

CARRIERS = [torch.float32, torch.bfloat16, torch.float16]


def _values(rng, rows, k):
    x = rng.standard_normal((rows, k)).astype(np.float32)
    x[0] = 0.0                                          # an all-zero row
    x[1, :8] = [448.0, -448.0, 1e-30, -1e-30, 0.0, 3.0, 2.5, 0.0234375]
    x[2] *= 1e-6
    x[3] *= 1e3                                        # (finite in float16 too)
    # exact ties of the e4m3 grid once divided by the row scale: amax 448 -> scale 1
    x[4] = 0.0
    x[4, :10] = [448.0, 17.0, 18.0, 19.0, 21.0, 0.0009765625, 0.0029296875, 1.0625, 1.1875, -15.5]
    return x


@pytest.mark.parametrize("carrier", CARRIERS)
def test_per_token_and_per_tensor_match_oracle(device, carrier):
    rng = np.random.default_rng(5)
    rows, k = 37, 192
    xt = to_dev(_values(rng, rows, k), device).to(carrier)
    xf = xt.float().cpu().numpy()
    for mode, quant in (("per_token", fp8.quantize_per_token), ("per_tensor", fp8.quantize_per_tensor)):
        want_codes, want_scale = quant(xf)
        codes = torch.zeros((rows, k), dtype=torch.uint8, device=device)
        scale = torch.zeros((rows,), dtype=torch.float32, device=device)
        rec = torch.zeros((rows, k), dtype=carrier, device=device)
        ops.fp8_quantize(xt, mode, codes=codes, scale=scale, recovered=rec)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(scale.cpu().numpy(), want_scale)
        np.testing.assert_array_equal(codes.cpu().numpy(), want_codes)
        want_rec = to_dev((fp8.e4m3_decode(want_codes) * want_scale[:, None]).astype(np.float32), device).to(carrier)
        assert torch.equal(rec, want_rec)
        back = torch.zeros((rows, k), dtype=carrier, device=device)
        ops.fp8_dequantize(codes, scale, out=back)
        torch.cuda.synchronize()
        assert torch.equal(back, want_rec)


@pytest.mark.parametrize("carrier", CARRIERS)
def test_mxfp8_matches_oracle(device, carrier):
    rng = np.random.default_rng(6)
    rows, k = 21, 160
    x = _values(rng, rows, k)
    x[5, :32] = 448.0 * 2.0 ** -3                        # amax exactly 448 * 2^e
    x[5, 32:64] = np.nextafter(np.float32(448.0 * 2.0 ** -3), np.float32(1e9))
    # either side of the exponent's rounding point amax = 448 * 2^(e + 1/2)
    half = np.float32(448.0 * 2.0 ** -2.5)
    x[6, :32] = np.nextafter(half, np.float32(0)); x[6, 32:64] = half; x[6, 64:96] = np.nextafter(half, np.float32(1e9))
    xt = to_dev(x, device).to(carrier)
    xf = xt.float().cpu().numpy()
    want_codes, want_bytes = fp8.quantize_mxfp8(xf)
    codes = torch.zeros((rows, k), dtype=torch.uint8, device=device)
    scale = torch.zeros((rows, k // 32), dtype=torch.uint8, device=device)
    rec = torch.zeros((rows, k), dtype=carrier, device=device)
    ops.fp8_quantize(xt, "mxfp8", codes=codes, scale=scale, recovered=rec)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(scale.cpu().numpy(), want_bytes)
    np.testing.assert_array_equal(codes.cpu().numpy(), want_codes)
    want_rec = to_dev(fp8.roundtrip_mxfp8(xf), device).to(carrier)
    assert torch.equal(rec, want_rec)
    packed, bytes_ = fbs._quantize_mxfp8(xt)
    assert packed.dtype == torch.int32 and tuple(packed.shape) == (rows, k // 4)
    assert torch.equal(fbs._unpack_mxfp8_to_uint8(packed, k), codes) and torch.equal(bytes_, scale)
    assert torch.equal(fbs._dequantize_mxfp8(packed, bytes_, out_dtype=carrier), want_rec)
    with pytest.raises(ValueError):
        fbs._quantize_mxfp8(xt[:, :40].contiguous())


def test_float_carrier_attention_wrappers(device):
    rng = np.random.default_rng(7)
    B, S, H, G, Skv, topk, D, d_v = 2, 4, 8, 2, 60, 16, 64, 32
    q = to_dev(rng.standard_normal((B, S, H, D)).astype(np.float32), device).to(torch.bfloat16)
    kv = to_dev(rng.standard_normal((B, Skv, G, D)).astype(np.float32), device).to(torch.bfloat16)
    idx = sparse_indices(rng, B, S, G, Skv, topk, replace=True)
    idx[..., -2:] = -1
    it = to_dev(idx.astype(np.int32), device)
    qf, kf = q.float().cpu().numpy(), kv.float().cpu().numpy()

    def carrier(a):                                      # the round trip lands in bf16, like q.dtype in the reference
        return to_dev(a, device).to(torch.bfloat16).float().cpu().numpy()

    for fn, rt in ((ff8.sparse_mla_fp8_apply, fp8.roundtrip_per_tensor), (fbs.sparse_mla_blockscaled_apply, fp8.roundtrip_mxfp8)):
        want_out, want_lse = om.sparse_mla_oracle(carrier(rt(qf)), carrier(rt(kf)), idx, d_v=d_v)
        out, lse = fn(q, kv, it, d_v=d_v, return_lse=True)
        torch.cuda.synchronize()
        assert out.dtype == torch.bfloat16 and tuple(out.shape) == (B, S, H, d_v)
        got = out.float().cpu().numpy()
        assert np.abs(got - want_out).max() <= 2e-2 * np.abs(want_out).max()
        assert np.abs(lse.cpu().numpy() - want_lse).max() <= 1e-3
        with pytest.raises(RuntimeError):
            fn(q, kv, it, d_v=d_v, force_metal=True)
    codes, scale = ff8._to_fp8_with_per_tensor_scale(q)
    assert codes.dtype == torch.uint8 and tuple(scale.shape) == (B, S, H)
    want_codes, want_scale = fp8.quantize_per_tensor(qf)
    np.testing.assert_array_equal(codes.cpu().numpy(), want_codes)
    np.testing.assert_array_equal(scale.cpu().numpy(), want_scale)
    rec = ff8._from_fp8_with_scale(codes, scale, dtype=torch.float32)
    np.testing.assert_array_equal(rec.cpu().numpy(), fp8.roundtrip_per_tensor(qf))


def test_reference_parity_receipts_on_the_gpu(device):
    """The reference's two seeded receipts (scripts/bench_tilelang_sparse_mla_fp8.py:105-125, 443-445;
    bench/tilelang_ports/sparse_mla_fp8.json and sparse_mla_blockscaled.json, ``parity``) through the
    float-carrier entry points: max|quantised - plain| on float32 carriers."""
    from cppmega_mlx_amd.nn.sparse_mla import sparse_mla_attention_reference
    from tests.test_oracle_reference_receipts import BLOCKSCALED_VS_PLAIN, FP8_VS_PLAIN, receipt_inputs

    q, kv, idx = receipt_inputs()
    qt, kt, it = to_dev(q, device), to_dev(kv, device), to_dev(idx, device)
    plain = sparse_mla_attention_reference(qt, kt, it, d_v=32)
    fp8_out = ff8.sparse_mla_fp8_apply(qt, kt, it, d_v=32)
    bs_out = fbs.sparse_mla_blockscaled_apply(qt, kt, it, d_v=32)
    fp8_ref = ff8.sparse_mla_fp8_reference(qt, kt, it, d_v=32)
    bs_ref = fbs.sparse_mla_blockscaled_reference(qt, kt, it, d_v=32)
    torch.cuda.synchronize()
    assert plain.dtype == torch.float32
    for got, want in ((fp8_out, FP8_VS_PLAIN), (fp8_ref, FP8_VS_PLAIN), (bs_out, BLOCKSCALED_VS_PLAIN), (bs_ref, BLOCKSCALED_VS_PLAIN)):
        assert abs(float((got - plain).abs().max()) - want) <= 1e-6
