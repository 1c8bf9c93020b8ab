"""GPU parity: indexer scores -> top-k (through the C ABI) vs the oracle.

Indices are integer work: with integer-valued inputs every product and sum is exact in any
order, so the selection must equal the oracle's bit for bit, ties included.  With Gaussian inputs
the scores carry rounding; they are held to 2e-4 of the score scale against the float64
oracle, the selection must be exactly the oracle's selection on the scores the kernel wrote, and
against the float64 selection only entries within that tolerance of the k-th score may differ.
"""

import numpy as np
import pytest
import torch

from cppmega_mlx_amd import ops
from cppmega_mlx_amd.nn import lightning_indexer as li
from oracle import indexer as oi
from tests._inputs import to_dev

pytestmark = pytest.mark.gpu

SCORE_TOL = 2e-4


def _int_inputs(rng, B, Sq, H, D, Skv):
    q = rng.integers(-3, 4, (B, Sq, H, D)).astype(np.float32)
    k = rng.integers(-3, 4, (B, Skv, D)).astype(np.float32)
    w = rng.integers(-2, 3, (B, Sq, H)).astype(np.float32)
    return q, k, w


INT_CASES = [
    # B, Sq, H, D, Skv, topk, carrier
    (2, 37, 4, 32, 300, 16, torch.float32),
    (2, 37, 4, 32, 300, 16, torch.bfloat16),
    (1, 16, 64, 128, 1024, 64, torch.bfloat16),
    (3, 1, 8, 64, 2048, 128, torch.bfloat16),          # decode: one query row per sequence
    (1, 5, 3, 40, 77, 77, torch.float32),              # head_dim and key count off every vector width; topk = Skv
    (1, 9, 2, 20, 130, 9, torch.bfloat16),
    (1, 100, 8, 64, 512, 32, torch.bfloat16),          # 32 query rows per workgroup, the last one ragged
    (2, 70, 4, 128, 300, 16, torch.float32),
    (1, 130, 4, 96, 260, 8, torch.bfloat16),           # three 32-channel steps
]


@pytest.mark.parametrize("case", INT_CASES, ids=lambda c: "B%d_S%d_H%d_D%d_T%d_k%d_%s" % (c[:6] + (str(c[6]).split(".")[-1],)))
@pytest.mark.parametrize("order", ["index", "value"])
def test_integer_inputs_select_exactly_the_oracle_set(device, case, order):
    B, Sq, H, D, Skv, topk, carrier = case
    rng = np.random.default_rng(B * 1000 + Sq * 10 + D)
    q, k, w = _int_inputs(rng, B, Sq, H, D, Skv)
    starts = rng.integers(0, Skv // 4, B * Sq).astype(np.int32)
    ends = rng.integers(Skv // 2, Skv + 1, B * Sq).astype(np.int32)
    ends[0] = starts[0] + 3                                    # fewer selectable keys than topk: -1 padding
    want = oi.indexer_topk_oracle(q, k, w, sm_scale=0.125, index_topk=topk, starts=starts, ends=ends, order=order)
    qt, kt, wt = (to_dev(a, device).to(carrier) for a in (q, k, w))
    out = torch.full((B, Sq, topk), -9, dtype=torch.int32, device=device)
    scores = torch.zeros((B, Sq, Skv), dtype=torch.float32, device=device)
    got = ops.indexer_topk(qt, kt, wt, sm_scale=0.125, topk=topk, out=out, starts=to_dev(starts, device),
                           ends=to_dev(ends, device), order=order, scores_out=scores)
    torch.cuda.synchronize()
    assert got is out
    np.testing.assert_array_equal(scores.cpu().numpy(), oi.indexer_scores_oracle(q, k, w, sm_scale=0.125).astype(np.float32))
    np.testing.assert_array_equal(out.cpu().numpy(), want)
    # the same through the chunked path (no score matrix kept), in passes of a few rows
    for chunk_rows in (0, 16 if Sq > 16 else 2):
        out2 = torch.full((B, Sq, topk), -9, dtype=torch.int32, device=device)
        ops.indexer_topk(qt, kt, wt, sm_scale=0.125, topk=topk, out=out2, starts=to_dev(starts, device),
                         ends=to_dev(ends, device), order=order, chunk_rows=chunk_rows)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out2.cpu().numpy(), want)


BOUND_CASES = [
    # B, Sq, H, D, Skv, topk: bf16 rows, so that the wavefront-per-row head sum runs
    (1, 300, 64, 128, 2048, 64),       # sixteen heads-of-four in flight, no tail
    (1, 200, 100, 128, 1536, 48),      # one full round of heads and a tail of 36
    (2, 150, 8, 64, 1300, 40),         # eight heads per load: the tail loop only
    (1, 90, 6, 256, 1024, 32),         # two heads per load
]


@pytest.mark.parametrize("case", BOUND_CASES, ids=lambda c: "B%d_S%d_H%d_D%d_T%d_k%d" % c)
def test_tight_bounds_leave_unscored_keys_unread(device, case):
    """Sliding causal windows: a query tile scores only the keys between the smallest start and the
    largest end of its rows.  The workspace is poisoned first (NaN patterns and huge values), so a
    selection that looked at a key nobody scored would show."""
    B, Sq, H, D, Skv, topk = case
    rng = np.random.default_rng(Sq + H + D)
    q, k, w = _int_inputs(rng, B, Sq, H, D, Skv)
    pos = (np.arange(Sq) * (Skv - 1) // max(Sq - 1, 1)).astype(np.int64)
    ends = np.tile(pos + 1, B).astype(np.int32)
    starts = np.maximum(ends - 400, 0).astype(np.int32)
    want = oi.indexer_topk_oracle(q, k, w, sm_scale=0.125, index_topk=topk, starts=starts, ends=ends, order="index")
    qt, kt, wt = (to_dev(a, device).to(torch.bfloat16) for a in (q, k, w))
    need = ops.indexer_topk_workspace_bytes(qt, kt, wt, topk=topk)
    for poison in (0x7fc00000, 0x7f000000):
        ws = torch.full(((need + 3) // 4,), poison, dtype=torch.int32, device=device).view(torch.uint8)
        out = torch.full((B, Sq, topk), -9, dtype=torch.int32, device=device)
        ops.indexer_topk(qt, kt, wt, sm_scale=0.125, topk=topk, out=out, starts=to_dev(starts, device),
                         ends=to_dev(ends, device), order="index", workspace=ws)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out.cpu().numpy(), want)


def test_additive_mask_and_masked_positions(device):
    rng = np.random.default_rng(5)
    B, Sq, H, D, Skv, topk = 2, 24, 4, 32, 64, 20
    q, k, w = _int_inputs(rng, B, Sq, H, D, Skv)
    mask = np.zeros((B, Sq, Skv), dtype=np.float32)
    for s in range(Sq):
        mask[:, s, s + 8:] = -np.inf                          # causal: row s sees s + 8 keys, some rows fewer than topk
    mask[:, :, 3] = 5.0                                        # and a finite additive term
    want = oi.indexer_topk_oracle(q, k, w, sm_scale=0.25, index_topk=topk, mask=mask)
    out = torch.zeros((B, Sq, topk), dtype=torch.int32, device=device)
    for mask_t in (to_dev(mask, device), to_dev(mask, device).to(torch.bfloat16)):
        ops.indexer_topk(to_dev(q, device), to_dev(k, device), to_dev(w, device), sm_scale=0.25, topk=topk, out=out, mask=mask_t)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out.cpu().numpy(), want)
    assert (want[:, 0, 8:] == -1).all()


@pytest.mark.parametrize("carrier", [torch.float32, torch.bfloat16])
def test_gaussian_inputs_scores_and_selection(device, carrier):
    rng = np.random.default_rng(6)
    B, Sq, H, D, Skv, topk = 2, 50, 16, 128, 4096, 256
    qt, kt, wt = (to_dev(rng.standard_normal(s).astype(np.float32), device).to(carrier)
                  for s in ((B, Sq, H, D), (B, Skv, D), (B, Sq, H)))
    q, k, w = (t.float().cpu().numpy() for t in (qt, kt, wt))
    sm = D ** -0.5
    want_scores = oi.indexer_scores_oracle(q, k, w, sm_scale=sm)
    scores = torch.zeros((B, Sq, Skv), dtype=torch.float32, device=device)
    out = torch.zeros((B, Sq, topk), dtype=torch.int32, device=device)
    ops.indexer_topk(qt, kt, wt, sm_scale=sm, topk=topk, out=out, scores_out=scores)
    torch.cuda.synchronize()
    got_scores = scores.cpu().numpy()
    tol = SCORE_TOL * np.abs(want_scores).max()
    assert np.abs(got_scores - want_scores).max() <= tol
    got = out.cpu().numpy()
    # exact on the scores the kernel wrote
    np.testing.assert_array_equal(got, oi.indexer_topk_oracle(None, None, None, sm_scale=sm, index_topk=topk, scores=got_scores))
    # against the float64 selection: only near-boundary entries may differ
    want = oi.indexer_topk_oracle(q, k, w, sm_scale=sm, index_topk=topk)
    for b in range(B):
        for s in range(Sq):
            kth = np.sort(want_scores[b, s])[-topk]
            odd = np.setxor1d(got[b, s], want[b, s])
            assert np.all(np.abs(want_scores[b, s, odd] - kth) <= 2 * tol)
    # the chunked path computes the same scores, so it selects the same indices
    out2 = torch.zeros_like(out)
    ops.indexer_topk(qt, kt, wt, sm_scale=sm, topk=topk, out=out2, chunk_rows=32)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


def test_module_forward_matches_the_oracle_chain(device):
    """LightningIndexer end to end (reference shapes of tests/v4/test_lightning_indexer.py:65-107):
    projections, rope and LayerNorm in float64 on the host, then the oracle's score and selection."""
    cfg = li.LightningIndexerConfig(hidden_size=64, n_heads=4, head_dim=32, rope_head_dim=16, q_lora_rank=48, index_topk=6)
    ix = li.LightningIndexer(cfg, device=device, seed=3)
    rng = np.random.default_rng(7)
    B, T = 2, 40
    x = rng.standard_normal((B, T, 64)).astype(np.float32)
    qr = rng.standard_normal((B, T, 48)).astype(np.float32)
    ang = np.outer(np.arange(T), 1.0 / (10000 ** (np.arange(8) / 8))).astype(np.float32)
    cos, sin = np.cos(ang), np.sin(ang)
    got = ix(to_dev(x, device), to_dev(qr, device), (to_dev(cos, device), to_dev(sin, device)))
    torch.cuda.synchronize()
    assert got.dtype == torch.int32 and tuple(got.shape) == (B, T, 6)
    wq, wk, wp = (t.double().cpu().numpy() for t in (ix.wq_b, ix.wk, ix.weights_proj))
    q = (qr.astype(np.float64) @ wq.T).reshape(B, T, 4, 32)
    q = np.concatenate([oi.apply_non_interleaved_rope(q[..., :16], cos, sin), q[..., 16:]], axis=-1)
    kk = x.astype(np.float64) @ wk.T
    kk = (kk - kk.mean(-1, keepdims=True)) / np.sqrt(kk.var(-1, keepdims=True) + 1e-6)
    kk = np.concatenate([oi.apply_non_interleaved_rope(kk[..., :16], cos, sin), kk[..., 16:]], axis=-1)
    w = (x.astype(np.float64) @ wp.T) * 4 ** -0.5
    scores = oi.indexer_scores_oracle(q, kk, w, sm_scale=32 ** -0.5)
    want = oi.indexer_topk_oracle(q, kk, w, sm_scale=32 ** -0.5, index_topk=6)
    g = got.cpu().numpy()
    tol = 1e-4 * np.abs(scores).max()
    for b in range(B):
        for t in range(T):
            odd = np.setxor1d(g[b, t], want[b, t])
            assert np.all(np.abs(scores[b, t, odd] - np.sort(scores[b, t])[-6]) <= tol)
    # index_topk above the key count is clipped (tests/v4/test_lightning_indexer.py:80-92)
    wide = li.LightningIndexer(li.LightningIndexerConfig(hidden_size=64, n_heads=4, head_dim=32, rope_head_dim=16,
                                                         q_lora_rank=48, index_topk=100), device=device)
    assert tuple(wide(to_dev(x, device), to_dev(qr, device), (to_dev(cos, device), to_dev(sin, device))).shape) == (B, T, T)


def test_fp8_module_overlaps_the_float_module(device):
    """The reference's own acceptance test for the FP8 indexer (tests/v4/test_lightning_indexer_fp8.py:58-89):
    mean top-k overlap with the float indexer of at least 0.4 after weight quantisation."""
    base = li.LightningIndexerConfig(hidden_size=128, n_heads=4, head_dim=32, rope_head_dim=16, q_lora_rank=64, index_topk=8)
    f32 = li.LightningIndexer(base, device=device, seed=11)
    fp8 = li.LightningIndexerFP8(li.LightningIndexerFP8Config(hidden_size=128, n_heads=4, head_dim=32, rope_head_dim=16,
                                                              q_lora_rank=64, index_topk=8), device=device)
    fp8.load_fp8_weights(**li.quantize_indexer_weights_for_fp8(f32))
    with pytest.raises(TypeError, match="uint8"):
        fp8.load_fp8_weights(torch.zeros((128, 64), device=device), torch.ones((1, 1), device=device), f32.wk, f32.weights_proj)
    rng = np.random.default_rng(11)
    B, T = 2, 24
    x = to_dev(rng.standard_normal((B, T, 128)).astype(np.float32), device)
    qr = to_dev(rng.standard_normal((B, T, 64)).astype(np.float32), device)
    ang = np.outer(np.arange(T), 1.0 / (10000 ** (np.arange(8) / 8))).astype(np.float32)
    freqs = (to_dev(np.cos(ang), device), to_dev(np.sin(ang), device))
    a = f32(x, qr, freqs).cpu().numpy()
    b = fp8(x, qr, freqs).cpu().numpy()
    assert b.dtype == np.int32 and b.shape == (B, T, 8)
    overlap = np.mean([len(set(a[i, t]) & set(b[i, t])) / 8 for i in range(B) for t in range(T)])
    assert overlap >= 0.4, overlap


def test_argument_errors(device):
    q = torch.zeros((1, 2, 2, 32), device=device); k = torch.zeros((1, 8, 32), device=device); w = torch.zeros((1, 2, 2), device=device)
    out = torch.zeros((1, 2, 4), dtype=torch.int32, device=device)
    with pytest.raises(ValueError):
        ops.indexer_topk(q, k, w, sm_scale=1.0, topk=9, out=torch.zeros((1, 2, 9), dtype=torch.int32, device=device))
    with pytest.raises(ValueError):
        ops.indexer_topk(q, k[:, :, :16].contiguous(), w, sm_scale=1.0, topk=4, out=out)
    with pytest.raises(TypeError):
        ops.indexer_topk(q.half(), k, w, sm_scale=1.0, topk=4, out=out)
    with pytest.raises(ValueError):
        ops.indexer_topk(q, k, w, sm_scale=1.0, topk=4, out=out.long())
