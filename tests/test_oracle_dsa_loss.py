"""The DSA indexer-loss oracle against closed forms and an explicit loop."""

import numpy as np
import pytest

from oracle import dsa_loss as od


def test_uniform_attention_against_uniform_index_is_a_log_ratio():
    ASq, AB, AH, AD, Sk = 5, 2, 3, 4, 7
    q = np.zeros((ASq, AB, AH, AD)); k = np.zeros((Sk, AB, AH, AD))
    loss = od.dsa_indexer_loss_per_position(np.zeros((AB, ASq, Sk)), q, k, softmax_scale=0.5)
    want = np.log(Sk) - np.log(np.arange(1, ASq + 1))          # p uniform over sq + 1 keys, q uniform over all Sk
    np.testing.assert_allclose(loss, np.broadcast_to(want, (AB, ASq)), atol=1e-8)


def test_index_equal_to_log_attention_gives_zero_on_a_full_row():
    rng = np.random.default_rng(3)
    ASq, AB, AH, AD = 6, 1, 2, 5
    Sk = ASq
    q = rng.standard_normal((ASq, AB, AH, AD)); k = rng.standard_normal((Sk, AB, AH, AD))
    sq = ASq - 1                                               # the last row sees every key: both softmaxes range over the same set
    p = np.zeros(Sk)
    for h in range(AH):
        s = k[:, 0, h] @ q[sq, 0, h] * 0.3
        e = np.exp(s - s.max()); p += e / e.sum()
    p /= AH
    idx = np.zeros((AB, ASq, Sk)); idx[0, sq] = np.log(p)
    loss = od.dsa_indexer_loss_per_position(idx, q, k, softmax_scale=0.3)
    assert abs(loss[0, sq]) < 1e-8
    # a different index distribution gives a positive divergence
    idx[0, sq] = np.log(p[::-1])
    assert od.dsa_indexer_loss_per_position(idx, q, k, softmax_scale=0.3)[0, sq] > 1e-3


def test_explicit_loop_with_sparse_mask_and_wrapper_contract():
    rng = np.random.default_rng(4)
    ASq, AB, AH, AD, Sk, topk = 4, 2, 2, 3, 6, 3
    q = rng.standard_normal((ASq, AB, AH, AD)); k = rng.standard_normal((Sk, AB, AH, AD))
    idx = rng.standard_normal((AB, ASq, Sk))
    top = np.stack([np.stack([rng.choice(Sk, topk, replace=False) for _ in range(ASq)]) for _ in range(AB)])
    mask = od.sparse_index_mask(top, Sk)
    assert mask.shape == (AB, ASq, Sk) and (np.isinf(mask).sum(-1) == Sk - topk).all()
    got = od.dsa_indexer_loss_per_position(idx, q, k, softmax_scale=0.7, index_mask=mask)
    want = np.zeros((AB, ASq))
    for b in range(AB):
        for sq in range(ASq):
            n = sq + 1
            p = np.zeros(n)
            for h in range(AH):
                s = np.array([0.7 * sum(q[sq, b, h, d] * k[j, b, h, d] for d in range(AD)) + mask[b, sq, j] for j in range(n)])
                if np.isfinite(s.max()):
                    e = np.exp(s - s.max()); p += e / e.sum()
            p /= AH
            v = idx[b, sq] + mask[b, sq]
            e1 = np.exp(v - v.max()); qd = e1 / e1.sum()
            want[b, sq] = sum(p[j] * (np.log(p[j] + 1e-10) - np.log(qd[j] + 1e-10)) for j in range(n))
    np.testing.assert_allclose(got, want, atol=1e-12)
    total = od.dsa_indexer_loss(idx, top, q, k, 0.7, 0.25, True)
    assert abs(total - want.mean() * 0.25) < 1e-12
    assert od.dsa_indexer_loss(idx[:, :0], top[:, :0], q[:0], k, 0.7, 1.0, True) == 0.0
    with pytest.raises(ValueError):
        od.sparse_index_mask(top + Sk, Sk)
