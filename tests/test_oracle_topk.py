"""Pins oracle/topk.py against the reference tests' known answers and brute force."""

import json

import numpy as np
import pytest

from oracle import topk


@pytest.fixture(scope="module")
def kats(golden_dir):
    return json.loads((golden_dir / "reference_kats.json").read_text())


def test_exact_order_known_answers(kats):
    case = kats["topk_exact_order_ties"]
    got = topk.topk_selector_oracle(np.array(case["scores"], np.float32), case["k"], order="value")
    assert got.tolist() == case["expected_value_order"]


def test_masked_ties_known_answers(kats):
    case = kats["topk_masked_ties"]
    got = topk.topk_selector_oracle(np.array(case["scores"], np.float32), case["k"], starts=case["starts"],
                                    ends=case["ends"], order="value")
    assert got.tolist() == case["expected_value_order"]
    by_index = topk.topk_selector_oracle(np.array(case["scores"], np.float32), case["k"], starts=case["starts"],
                                         ends=case["ends"], order="index")
    assert by_index.tolist() == [[1, 2, 4, 6], [2, 3, 4, 5], [6, 7, -1, -1]]


def test_short_and_empty_intervals(kats):
    case = kats["topk_short_and_empty_intervals"]
    got = topk.topk_selector_oracle(np.array(case["scores"], np.float32), case["k"], starts=case["starts"], ends=case["ends"])
    assert [sorted(set(r)) for r in got.tolist()] == [sorted(s) for s in case["expected_sets"]]
    assert got[1].tolist() == [-1, -1, -1, -1]


def test_k_one_and_full_width(kats):
    case = kats["topk_k_one_argmax"]
    assert topk.topk_selector_oracle(np.array(case["scores"], np.float32), 1).tolist() == case["expected"]
    rng = np.random.default_rng(0)
    s = rng.standard_normal((2, 32)).astype(np.float32)
    assert topk.topk_selector_oracle(s, 32).tolist() == [list(range(32))] * 2


def test_bruteforce_on_tiny_rows_with_heavy_ties():
    rng = np.random.default_rng(4)
    for trial in range(50):
        T = int(rng.integers(2, 24))
        k = int(rng.integers(1, T + 1))
        s = rng.integers(-3, 4, size=(3, T)).astype(np.float32)   # few distinct values -> many ties
        s[s == 0] = rng.choice([0.0, -0.0], size=(s == 0).sum())
        got = topk.topk_selector_oracle(s, k)
        assert [set(r) for r in got.tolist()] == topk.topk_bruteforce(s, k)
        val = topk.topk_selector_oracle(s, k, order="value")
        assert [set(r) for r in val.tolist()] == [set(r) for r in got.tolist()]
        for r in range(3):
            picked = s[r, val[r]]
            assert (np.diff(picked) <= 0).all()                     # value descending
            same = np.diff(picked) == 0
            assert (np.diff(val[r])[same] > 0).all()                # lower index first among equals


def test_validation_errors():
    s = np.zeros((2, 4), np.float32)
    with pytest.raises(ValueError, match="expects a \\(B, T\\) array"):
        topk.topk_selector_oracle(np.zeros(4, np.float32), 1)
    with pytest.raises(ValueError, match="topk must be >= 1"):
        topk.topk_selector_oracle(s, 0)
    with pytest.raises(ValueError, match="exceeds sequence length"):
        topk.topk_selector_oracle(s, 5)


def test_neg_inf_and_nan_handling():
    s = np.array([[1.0, -np.inf, 2.0, np.nan, -np.inf]], np.float32)
    assert topk.topk_selector_oracle(s, 4, order="value").tolist() == [[2, 0, 1, 4]]
    assert topk.topk_selector_oracle(s, 4, order="value", neg_inf_is_masked=True).tolist() == [[2, 0, -1, -1]]
    assert topk.topk_selector_oracle(s, 5, order="index").tolist() == [[0, 1, 2, 4, -1]]
