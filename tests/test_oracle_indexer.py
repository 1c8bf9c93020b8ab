"""The indexer oracle against an explicit loop evaluation, the head-sum-first identity,
NumPy's argpartition on distinct scores, and the reference's rope known answers
(tests/v4/test_lightning_indexer.py:36-57); plus the host-side configuration checks (:25-33)."""

import numpy as np
import pytest
import torch

from cppmega_mlx_amd.nn import lightning_indexer as li
from oracle import indexer as oi


def _inputs(rng, B=2, Sq=3, H=4, D=6, Skv=9):
    return (rng.standard_normal((B, Sq, H, D)), rng.standard_normal((B, Skv, D)), rng.standard_normal((B, Sq, H)))


def test_scores_equal_the_four_loop_evaluation():
    rng = np.random.default_rng(1)
    q, k, w = _inputs(rng)
    mask = rng.standard_normal((2, 3, 9))
    got = oi.indexer_scores_oracle(q, k, w, sm_scale=0.3, mask=mask)
    want = np.zeros((2, 3, 9))
    for b in range(2):
        for s in range(3):
            for t in range(9):
                acc = 0.0
                for h in range(4):
                    dot = 0.0
                    for d in range(6):
                        dot += q[b, s, h, d] * k[b, t, d]
                    acc += w[b, s, h] * dot
                want[b, s, t] = acc * 0.3 + mask[b, s, t]
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
    # a transposed operand or a dropped weight changes the result
    assert np.abs(got - oi.indexer_scores_oracle(q, k, np.ones_like(w), sm_scale=0.3, mask=mask)).max() > 1e-2


def test_head_sum_first_identity():
    rng = np.random.default_rng(2)
    q, k, w = _inputs(rng, B=1, Sq=5, H=7, D=8, Skv=11)
    qw = np.einsum("bqh,bqhd->bqd", w, q)
    np.testing.assert_allclose(oi.indexer_scores_oracle(q, k, w, sm_scale=0.5), 0.5 * np.einsum("bqd,bkd->bqk", qw, k),
                               rtol=1e-12, atol=1e-12)


def test_selection_is_the_argpartition_set_and_clips_topk():
    rng = np.random.default_rng(3)
    q, k, w = _inputs(rng, B=2, Sq=4, H=3, D=8, Skv=40)
    scores = oi.indexer_scores_oracle(q, k, w, sm_scale=8 ** -0.5)
    got = oi.indexer_topk_oracle(q, k, w, sm_scale=8 ** -0.5, index_topk=7)
    part = np.argpartition(-scores.astype(np.float32), 6, axis=-1)[..., :7]
    assert got.dtype == np.int32 and got.shape == (2, 4, 7)
    np.testing.assert_array_equal(got, np.sort(part, axis=-1))
    # index_topk above the key count is clipped to it (tests/v4/test_lightning_indexer.py:80-92)
    assert oi.indexer_topk_oracle(q, k, w, sm_scale=1.0, index_topk=100).shape == (2, 4, 40)
    # masked (-inf) positions are never returned; the slots they would take hold -1
    mask = np.zeros((2, 4, 40))
    mask[:, :, 5:] = -np.inf
    sel = oi.indexer_topk_oracle(q, k, w, sm_scale=1.0, index_topk=7, mask=mask)
    np.testing.assert_array_equal(sel[..., :5], np.broadcast_to(np.arange(5), (2, 4, 5)))
    assert (sel[..., 5:] == -1).all()


def test_rope_known_answers():
    np.testing.assert_allclose(oi.apply_non_interleaved_rope(np.arange(16.0).reshape(2, 8), np.ones((4,)), np.zeros((4,))),
                               np.arange(16.0).reshape(2, 8))
    out = oi.apply_non_interleaved_rope(np.array([[1.0, 2, 3, 4, 5, 6]]), np.zeros((3,)), np.ones((3,)))
    np.testing.assert_allclose(out, [[-4.0, -5.0, -6.0, 1.0, 2.0, 3.0]])
    with pytest.raises(ValueError, match="rope dim must be even"):
        oi.apply_non_interleaved_rope(np.zeros((1, 3)), np.zeros((1,)), np.zeros((1,)))
    # the torch mirror used by the module agrees, including the broadcast over a head axis
    rng = np.random.default_rng(4)
    x = rng.standard_normal((2, 5, 3, 8))
    ang = rng.standard_normal((5, 4))
    got = li._apply_non_interleaved_rope(torch.from_numpy(x), torch.from_numpy(np.cos(ang)), torch.from_numpy(np.sin(ang)))
    np.testing.assert_allclose(got.numpy(), oi.apply_non_interleaved_rope(x, np.cos(ang), np.sin(ang)), rtol=1e-12)
    with pytest.raises(ValueError, match="rope dim must be even"):
        li._apply_non_interleaved_rope(torch.zeros(1, 3), torch.zeros(1), torch.zeros(1))


def test_config_validation():
    with pytest.raises(ValueError):
        li.LightningIndexerConfig(hidden_size=16, n_heads=2, head_dim=0)
    with pytest.raises(ValueError):
        li.LightningIndexerConfig(hidden_size=16, n_heads=2, head_dim=16, rope_head_dim=24)
    with pytest.raises(ValueError):
        li.LightningIndexerConfig(hidden_size=16, n_heads=0, head_dim=16)
    with pytest.raises(ValueError):
        li.LightningIndexerConfig(hidden_size=16, n_heads=2, head_dim=16, index_topk=0)
    assert li.LightningIndexerFP8Config(hidden_size=16, n_heads=2).fp8_blocks is True
