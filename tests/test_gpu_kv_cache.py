"""GPU parity: cache append (with the fused FP8 producer) and the sparse index producers,
bit-exact against oracle/kv_cache.py, and the producer tied to its consumer (append, then
decode over the cache)."""

import json

import numpy as np
import pytest
import torch

from cppmega_mlx_amd import ops, _lib
from cppmega_mlx_amd.inference import SparseFP8KVCache, SparseFP8KVCacheConfig
from cppmega_mlx_amd.nn.attention import causal_sparse_indices, sparse_indices_from_attention_mask
from oracle import fp8, kv_cache as okv, sparse_mla as om
from tests._inputs import bf16_pair, error_report, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def kats(golden_dir):
    return json.loads((golden_dir / "reference_kats.json").read_text())


# ---- index producers ------------------------------------------------------------------------

def test_causal_indices_reference_known_answer(device, kats):
    case = kats["causal_sparse_indices"]
    got = causal_sparse_indices(**case["args"], device=device)
    assert got.dtype == torch.int32 and tuple(got.shape) == (2, 5, 2, 3)
    assert got[0, :, 0, :].cpu().tolist() == case["expected_b0_g0"]


@pytest.mark.parametrize("args", [
    dict(batch_size=1, seq_length=1, kv_group=1, topk=2048, query_offset=65535, key_length=65536),   # a decode step
    dict(batch_size=2, seq_length=300, kv_group=2, topk=37, query_offset=0, key_length=None),
    dict(batch_size=1, seq_length=64, kv_group=1, topk=128, query_offset=10, key_length=50),          # key_length cuts the window
])
def test_causal_indices_match_oracle(device, args):
    want = okv.causal_sparse_indices(**args)
    got = causal_sparse_indices(**args, device=device)
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    out64 = torch.empty(want.shape, dtype=torch.int64, device=device)
    ops.causal_sparse_indices(out64, query_offset=args["query_offset"], key_length=args["key_length"] or args["seq_length"])
    np.testing.assert_array_equal(out64.cpu().numpy(), want.astype(np.int64))


def test_causal_indices_argument_errors(device):
    for bad in (dict(batch_size=0), dict(seq_length=0), dict(kv_group=0), dict(topk=0), dict(query_offset=-1), dict(key_length=0)):
        args = dict(batch_size=1, seq_length=2, kv_group=1, topk=2, query_offset=0, key_length=2)
        args.update(bad)
        with pytest.raises(ValueError):
            causal_sparse_indices(**args, device=device)


def test_mask_indices_reference_known_answer(device, kats):
    case = kats["sparse_indices_from_attention_mask"]
    mask = to_dev(np.array(case["mask"], dtype=np.bool_), device)
    got = sparse_indices_from_attention_mask(mask, **case["args"])
    assert tuple(got.shape) == (1, 3, 2, 2)
    assert np.sort(got[0, :, 0, :].cpu().numpy(), axis=-1).tolist() == case["expected_sorted_b0_g0"]


@pytest.mark.parametrize("shape,K,topk,dtype", [
    ((7,), 100, 16, np.bool_),                # (S,K) shared by batch and groups; K not a multiple of 16
    ((2, 5), 1000, 64, np.bool_),             # (B,S,K)
    ((2, 3, 4), 257, 300, np.bool_),          # (B,G,S,K), topk > K
    ((2, 1, 4), 4096, 2048, np.bool_),        # (B,1,S,K) group broadcast, more than one 1024-key step
    ((2, 1, 4), 4096, 1500, np.bool_),        # the window starts inside an all-valid 1024-key step
    ((3,), 77, 10, np.float32),
    ((2, 2), 130, 33, np.float16),
])
def test_mask_indices_match_oracle(device, shape, K, topk, dtype):
    rng = np.random.default_rng(K * 7 + topk)
    valid = rng.random(shape + (K,)) < 0.3
    if valid.ndim >= 2:
        valid[(0,) * (valid.ndim - 1)] = False        # a row with nothing valid
        valid[(-1,) * (valid.ndim - 1)] = True        # a row with everything valid
        if K >= 4096:                                 # a causal row: whole steps valid, then a ragged one, then nothing
            valid[(0,) * (valid.ndim - 2) + (1,)] = np.arange(K) < 2500
    if dtype == np.bool_:
        mask = valid
        t = to_dev(mask, device)
    else:
        mask = np.where(valid, rng.standard_normal(valid.shape), -np.inf).astype(dtype)
        t = to_dev(mask, device)
    B = shape[0] if len(shape) >= 2 else 2
    G = shape[1] if len(shape) == 3 and shape[1] > 1 else 2
    S = shape[-1]
    want = okv.sparse_indices_from_attention_mask(mask, batch_size=B, seq_length=S, kv_group=G, topk=topk, key_length=K)
    got = sparse_indices_from_attention_mask(t, batch_size=B, seq_length=S, kv_group=G, topk=topk, key_length=K)
    np.testing.assert_array_equal(got.cpu().numpy(), want)


def test_mask_indices_unaligned_rows_and_bf16(device):
    rng = np.random.default_rng(3)
    valid = rng.random((4, 51)) < 0.5                    # 51-byte rows: most rows start off 16-byte alignment
    want = okv.sparse_indices_from_attention_mask(valid, batch_size=1, seq_length=4, kv_group=1, topk=9, key_length=51)
    got = sparse_indices_from_attention_mask(to_dev(valid, device), batch_size=1, seq_length=4, kv_group=1, topk=9, key_length=51)
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    fm = torch.where(to_dev(valid, device), torch.zeros((), device=device), torch.full((), float("-inf"), device=device)).to(torch.bfloat16)
    got = sparse_indices_from_attention_mask(fm, batch_size=1, seq_length=4, kv_group=1, topk=9, key_length=51)
    np.testing.assert_array_equal(got.cpu().numpy(), want)


def test_mask_indices_argument_errors(device):
    m = torch.ones((3, 4), dtype=torch.bool, device=device)
    kw = dict(batch_size=1, seq_length=3, kv_group=1, topk=2, key_length=4)
    with pytest.raises(TypeError):
        sparse_indices_from_attention_mask(np.ones((3, 4), bool), **kw)
    with pytest.raises(ValueError):
        sparse_indices_from_attention_mask(m[None, None, None], **kw)                 # 5-D
    with pytest.raises(ValueError):
        sparse_indices_from_attention_mask(m, **{**kw, "key_length": 5})
    with pytest.raises(ValueError):
        sparse_indices_from_attention_mask(m.expand(3, 3, 4), **kw)                   # batch 3 vs 1
    with pytest.raises(ValueError):
        sparse_indices_from_attention_mask(m.expand(1, 3, 3, 4), **kw)                # 3 groups vs 1


# ---- cache append ---------------------------------------------------------------------------

def test_prepared_append_matches_reference_semantics(device):
    rng = np.random.default_rng(1)
    cfg = SparseFP8KVCacheConfig(num_layers=2, batch_size=2, num_kv_heads=2, head_dim=256, max_seq_len=12)
    cache = SparseFP8KVCache(cfg, device)
    ref_kv = np.zeros((2, 12, 2, 256), np.uint8)
    ref_sc = np.zeros((2, 12, 2), np.float32)
    pos = 0
    for S in (5, 1, 1, 4):
        kv = rng.integers(0, 256, (2, S, 2, 256), dtype=np.uint8)
        sc = rng.random((2, S, 2)).astype(np.float32)
        okv.append(ref_kv, ref_sc, pos, kv, sc)
        pos += S
        got_kv, got_sc = cache.update_and_fetch_sparse_fp8(1, to_dev(kv, device), to_dev(sc, device))
        assert tuple(got_kv.shape) == (2, pos, 2, 256) and tuple(got_sc.shape) == (2, pos, 2)
        assert got_kv.data_ptr() == cache.sparse_fp8_layers[1].kv.data_ptr()      # references to the cache's buffers
        np.testing.assert_array_equal(got_kv.cpu().numpy(), ref_kv[:, :pos])
        np.testing.assert_array_equal(got_sc.cpu().numpy(), ref_sc[:, :pos])
    assert cache.layer_position(1) == 11 and cache.layer_position(0) == 0
    with pytest.raises(RuntimeError):
        cache.update_and_fetch_sparse_fp8(1, torch.zeros((2, 2, 2, 256), dtype=torch.uint8, device=device),
                                          torch.zeros((2, 2, 2), dtype=torch.float32, device=device))
    with pytest.raises(ValueError):
        cache.update_and_fetch_sparse_fp8(0, torch.zeros((2, 1, 2, 256), dtype=torch.int8, device=device),
                                          torch.zeros((2, 1, 2), dtype=torch.float32, device=device))
    with pytest.raises(ValueError):
        cache.update_and_fetch_sparse_fp8(0, torch.zeros((3, 1, 2, 256), dtype=torch.uint8, device=device),
                                          torch.zeros((3, 1, 2), dtype=torch.float32, device=device))
    with pytest.raises(IndexError):
        cache.update_and_fetch_sparse_fp8(2, torch.zeros((2, 1, 2, 256), dtype=torch.uint8, device=device),
                                          torch.zeros((2, 1, 2), dtype=torch.float32, device=device))
    assert cache.trim(3) == 0                                                       # layer 0 is empty


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_per_row_producer_append_bit_exact(device, dtype):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((2, 3, 1, 512)) * rng.uniform(0.01, 30, (2, 3, 1, 1))).astype(np.float32)
    x[0, 1] = 0.0
    t = to_dev(x, device).to(dtype)
    xf = t.float().cpu().numpy()
    want_codes, want_scale = fp8.quantize_per_token(xf)
    kv = torch.zeros((2, 8, 1, 512), dtype=torch.uint8, device=device)
    sc = torch.zeros((2, 8, 1), dtype=torch.float32, device=device)
    positions = to_dev(np.array([4, 0], dtype=np.int32), device)
    ops.kv_cache_append(t, kv_cache=kv, scale_cache=sc, position=positions)
    for b, p in enumerate((4, 0)):
        np.testing.assert_array_equal(kv[b, p:p + 3].cpu().numpy(), want_codes[b])
        np.testing.assert_array_equal(sc[b, p:p + 3].cpu().numpy(), want_scale[b])
    assert int(kv[0, :4].sum()) == 0 and int(kv[1, 3:].sum()) == 0


@pytest.mark.parametrize("pow2", [False, True])
@pytest.mark.parametrize("D", [512, 128, 1152])
def test_block128_producer_append_bit_exact(device, pow2, D):
    rng = np.random.default_rng(D + int(pow2))
    B, S, G = 2, 5, 2
    x = (rng.standard_normal((B, S, G, D)) * rng.uniform(0.001, 100, (B, S, G, 1))).astype(np.float32)
    x[1, 2, 0, :128] = 0.0
    rope = rng.standard_normal((B, S, G, 64)).astype(np.float32)
    t, xf = bf16_pair(x, device)
    rt = to_dev(rope, device)
    want_codes, want_scale = okv.quantize_block128(xf, pow2=pow2)
    cfg = SparseFP8KVCacheConfig(num_layers=1, batch_size=B, num_kv_heads=G, head_dim=D, max_seq_len=9, rope_dim=64,
                                 scale_block=128, pow2_scales=pow2)
    cache = SparseFP8KVCache(cfg, device)
    cache.append_latent(0, t[:, :2].contiguous(), rt[:, :2].contiguous())
    kv, sc, rp = cache.append_latent(0, t[:, 2:].contiguous(), rt[:, 2:].contiguous())
    assert tuple(kv.shape) == (B, S, G, D) and tuple(sc.shape) == (B, S, G, D // 128) and rp.dtype == torch.bfloat16
    np.testing.assert_array_equal(kv.cpu().numpy(), want_codes)
    np.testing.assert_array_equal(sc.cpu().numpy(), want_scale)
    np.testing.assert_array_equal(rp.float().cpu().numpy(), rt.to(torch.bfloat16).float().cpu().numpy())
    assert cache.position() == S and cache.trim(2) == 2 and cache.position() == S - 2


def test_append_argument_errors(device):
    kv = torch.zeros((1, 4, 1, 256), dtype=torch.uint8, device=device)
    sc = torch.zeros((1, 4, 1), dtype=torch.float32, device=device)
    x = torch.zeros((1, 2, 1, 256), dtype=torch.bfloat16, device=device)
    with pytest.raises(ValueError):
        ops.kv_cache_append(x, kv_cache=kv, scale_cache=sc, position=3)                # runs past the capacity
    with pytest.raises(ValueError):
        ops.kv_cache_append(x, kv_cache=kv, scale_cache=sc, position=0, scale_block=64)
    with pytest.raises(ValueError):
        ops.kv_cache_append(x.view(torch.uint8)[..., :256].contiguous(), kv_cache=kv, scale_cache=sc, position=0)   # prepared bytes without scales
    with pytest.raises(_lib.NativeCallError):                                         # no CPU path
        ops.kv_cache_append(x.cpu(), kv_cache=kv, scale_cache=sc, position=0)


@pytest.mark.parametrize("H", [128, 32])
def test_appended_cache_feeds_the_decode_kernel(device, H):
    """Producer and consumer together: rows appended through the fused producer, a causal
    window from the index producer, attention over the views the cache returns (batch stride =
    capacity) against the oracle; then the same after a trim, where list entries that point at
    trimmed rows must be skipped."""
    rng = np.random.default_rng(9)
    B, T = 2, 200
    lat_t, lat_f = bf16_pair(rng.standard_normal((B, T, 1, 512)), device)
    rope_t, rope_f = bf16_pair(rng.standard_normal((B, T, 1, 64)), device)
    cfg = SparseFP8KVCacheConfig(num_layers=1, batch_size=B, num_kv_heads=1, head_dim=512, max_seq_len=256, rope_dim=64,
                                 scale_block=128, pow2_scales=True)
    cache = SparseFP8KVCache(cfg, device)
    cache.append_latent(0, lat_t[:, :150].contiguous(), rope_t[:, :150].contiguous())
    for s in range(150, T):                                                          # then token by token
        kv, sc, rp = cache.append_latent(0, lat_t[:, s:s + 1].contiguous(), rope_t[:, s:s + 1].contiguous())
    assert not kv.is_contiguous() and kv.stride(0) == 256 * 512
    codes, scale = okv.quantize_block128(lat_f, pow2=True)
    rows = om.dequant_block_latent(codes, scale, rope_f, 128)
    q, qf = bf16_pair(rng.standard_normal((B, 1, H, 576)), device)
    idx = causal_sparse_indices(B, 1, 1, 96, query_offset=T - 1, key_length=T, device=device)
    idx_np = idx.cpu().numpy().astype(np.int64)
    sinks = rng.standard_normal(H).astype(np.float32)
    sm = torch.tensor([576 ** -0.5], dtype=torch.float32, device=device)              # read on the device
    has = torch.ones(1, dtype=torch.int32, device=device)
    out = torch.zeros((B, 1, H, 512), dtype=torch.bfloat16, device=device)
    lse = torch.zeros((B, 1, H), dtype=torch.float32, device=device)

    def attend(kv, sc, rp):
        ops.sparse_mla_forward(q, kv, idx, sm_scale=sm, d_v=512, out=out, lse=lse, sinks=to_dev(sinks, device), has_sinks=has,
                               kv_spec=ops.QuantSpec(_lib.SCALE_F32_BLOCK, sc, 128), kv_rope=rp)
        torch.cuda.synchronize()
        return out.float().cpu().numpy(), lse.cpu().numpy()

    for flag in (1, 0):
        has.fill_(flag)
        got_out, got_lse = attend(kv, sc, rp)
        want_out, want_lse = om.sparse_mla_oracle(qf, rows, idx_np, sm_scale=576 ** -0.5, d_v=512, sinks=sinks if flag else None)
        err, ref = error_report(got_out, want_out)
        assert err <= 2e-2 * ref
        assert np.abs(got_lse - want_lse).max() <= 5e-3
    # trimmed rows stay in the buffer; the shorter views make them unattendable
    assert cache.trim(30) == 30
    layer = cache.sparse_fp8_layers[0]
    n = cache.position()
    got_out, got_lse = attend(layer.kv[:, :n], layer.scale[:, :n], layer.rope[:, :n])
    want_out, want_lse = om.sparse_mla_oracle(qf, rows[:, :n], idx_np, sm_scale=576 ** -0.5, d_v=512)
    err, ref = error_report(got_out, want_out)
    assert err <= 2e-2 * ref
    assert np.abs(got_lse - want_lse).max() <= 5e-3
    with pytest.raises(ValueError, match="batch pitch"):
        ops.sparse_mla_forward(q, layer.kv[:, :n], idx, sm_scale=sm, d_v=512, out=out, lse=lse,
                               kv_spec=ops.QuantSpec(_lib.SCALE_F32_BLOCK, layer.scale[:, :n].contiguous(), 128),
                               kv_rope=layer.rope[:, :n])
