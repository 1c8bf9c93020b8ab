"""GPU parity: the radix-select kernel (through the C ABI) vs the oracle, bit-exact."""

import json

import numpy as np
import pytest
import torch

from cppmega_mlx_amd.nn._tilelang import topk_selector as tk
from oracle import topk as otopk
from tests._inputs import to_dev, topk_scores

pytestmark = pytest.mark.gpu


def _run(scores_t, k, device, *, starts=None, ends=None, order="index", fill=-7, **kw):
    out = torch.full((scores_t.shape[0], k), fill, dtype=torch.int32, device=device)
    st = None if starts is None else to_dev(np.asarray(starts, np.int32), device)
    en = None if ends is None else to_dev(np.asarray(ends, np.int32), device)
    got = tk.topk_selector_tilelang_direct(scores_t, k, out=out, starts=st, ends=en, order=order, **kw)
    assert got is out
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_reference_known_answers(device, golden_dir):
    kats = json.loads((golden_dir / "reference_kats.json").read_text())
    c = kats["topk_exact_order_ties"]
    assert _run(to_dev(np.array(c["scores"], np.float32), device), c["k"], device, order="value").tolist() == c["expected_value_order"]
    c = kats["topk_masked_ties"]
    assert _run(to_dev(np.array(c["scores"], np.float32), device), c["k"], device, starts=c["starts"], ends=c["ends"],
                order="value").tolist() == c["expected_value_order"]
    c = kats["topk_short_and_empty_intervals"]
    got = _run(to_dev(np.array(c["scores"], np.float32), device), c["k"], device, starts=c["starts"], ends=c["ends"])
    assert [sorted(set(r)) for r in got.tolist()] == [sorted(s) for s in c["expected_sets"]]
    c = kats["topk_k_one_argmax"]
    assert _run(to_dev(np.array(c["scores"], np.float32), device), 1, device).tolist() == c["expected"]


@pytest.mark.parametrize("rows,width,k", [(4, 64, 8), (3, 512, 64), (5, 2048, 256), (6, 8192, 2048), (2, 8192, 1),
                                          (2, 8192, 8192), (3, 100, 7), (2, 1001, 500), (2, 4096, 2048), (1, 4, 4), (2, 20000, 3000), (1, 65536, 2048), (2, 9001, 100),
                                          (3, 16384, 2048), (2, 12288, 4096), (2, 32768, 2048), (2, 20004, 5000), (1, 30001, 7), (2, 16384, 16384), (2, 16380, 1), (2, 8196, 8000)])
@pytest.mark.parametrize("masked", [False, True])
@pytest.mark.parametrize("order", ["index", "value"])
def test_random_rows_bit_exact(device, rows, width, k, masked, order):
    rng = np.random.default_rng(rows * 7919 + width * 31 + k + (5 if masked else 0))
    s = topk_scores(rng, rows, width)
    starts = ends = None
    if masked:
        starts = rng.integers(0, max(1, width // 2), rows).astype(np.int32)
        ends = (starts + rng.integers(0, width, rows)).astype(np.int32)
        ends[0] = starts[0]                      # an empty interval
        starts[-1] = -5                          # clipped to 0
    got = _run(to_dev(s, device), k, device, starts=starts, ends=ends, order=order)
    want = otopk.topk_selector_oracle(s, k, starts=starts, ends=ends, order=order)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_half_precision_scores(device, dtype):
    rng = np.random.default_rng(17)
    t = to_dev(topk_scores(rng, 5, 2048), device).to(dtype)
    s = t.to(torch.float32).cpu().numpy()       # many exact ties after rounding
    for order in ("index", "value"):
        np.testing.assert_array_equal(_run(t, 300, device, order=order), otopk.topk_selector_oracle(s, 300, order=order))


def test_special_values_zero_signs_denormals_infinities_nan(device):
    s = np.array([[0.0, -0.0, 0.0, -0.0, 1e-40, -1e-40, np.inf, -np.inf, np.nan, 3.0, 3.0, -np.inf]], np.float32)
    t = to_dev(s, device)
    for k in (1, 3, 5, 7, 9, 11, 12):
        for order in ("index", "value"):
            np.testing.assert_array_equal(_run(t, k, device, order=order), otopk.topk_selector_oracle(s, k, order=order))
    np.testing.assert_array_equal(_run(t, 12, device, order="value", neg_inf_is_masked=True),
                                  otopk.topk_selector_oracle(s, 12, order="value", neg_inf_is_masked=True))


def test_constant_and_two_valued_rows(device):
    s = np.zeros((3, 8192), np.float32)
    s[1] = 5.0
    s[2, ::3] = 1.0
    np.testing.assert_array_equal(_run(to_dev(s, device), 2048, device), otopk.topk_selector_oracle(s, 2048))
    np.testing.assert_array_equal(_run(to_dev(s, device), 3000, device, order="value"),
                                  otopk.topk_selector_oracle(s, 3000, order="value"))


def test_misaligned_view_takes_the_scalar_load_path(device):
    rng = np.random.default_rng(23)
    s = topk_scores(rng, 4, 1030)
    base = to_dev(np.concatenate([np.zeros(1, np.float32), s.reshape(-1)]), device)
    t = base[1:].view(4, 1030)                   # 4-byte aligned only
    assert t.data_ptr() % 16 != 0
    np.testing.assert_array_equal(_run(t, 77, device), otopk.topk_selector_oracle(s, 77))


def test_headline_config_full_size_bit_exact(device):
    """[4, 1024, 8192] fp32 scores, 5% ties, causal bounds, k = 2048 (both the all-visible and the padded window)."""
    rng = np.random.default_rng(2048)
    B, S, T, k = 4, 1024, 8192, 2048
    s = topk_scores(rng, B * S, T)
    for off in (T - S, 0):
        ends = np.tile(off + np.arange(S, dtype=np.int32) + 1, B)
        masked = s.copy()
        masked[np.arange(T)[None, :] >= ends[:, None]] = -np.inf
        out = tk.topk_selector(to_dev(masked.reshape(B, S, T), device), k, ends=to_dev(ends, device))
        torch.cuda.synchronize()
        assert tuple(out.shape) == (B, S, k)
        got = out.reshape(B * S, k).cpu().numpy()
        want = otopk.topk_selector_oracle(masked, k, ends=ends)
        np.testing.assert_array_equal(got, want)
        valid = np.minimum(ends, k)
        assert ((got >= 0).sum(axis=1) == valid).all()


def test_public_entry_points(device):
    rng = np.random.default_rng(3)
    s = topk_scores(rng, 3, 256)
    t = to_dev(s, device)
    ref = tk.topk_selector_reference(t, 16)
    np.testing.assert_array_equal(ref.cpu().numpy(), otopk.topk_selector_oracle(s, 16, order="value"))
    for backend in ("auto", "hip", "path_c", "mlx"):
        np.testing.assert_array_equal(tk.topk_selector(t, 16, backend=backend).cpu().numpy(), otopk.topk_selector_oracle(s, 16))
    assert tk.topk_selector_path_c_status().available


@pytest.mark.parametrize("rows,width,k", [(32, 65536, 2048), (3, 40000, 4000), (2, 24576, 8192), (5, 16388, 100)])
def test_wide_rows_two_stage_and_single_workgroup_paths_agree_with_the_oracle(device, rows, width, k):
    """Rows wider than 16384 columns: k best of every 8192-column segment, then k of those.  Ties that
    straddle segments, bounds that empty whole segments, -inf and NaN entries."""
    import ctypes as C
    from cppmega_mlx_amd import _lib, ops
    rng = np.random.default_rng(rows + width + k)
    s = topk_scores(rng, rows, width, tie_fraction=0.2)
    s[0, ::5] = 1.5                                      # one value far beyond k times, in every segment
    s[1, 100:9000] = np.nan
    s[1, 9000:9500] = -np.inf
    starts = rng.integers(0, width // 3, rows).astype(np.int32)
    ends = rng.integers(width // 2, width + 1, rows).astype(np.int32)
    starts[-1], ends[-1] = 9000, 9000 + k // 2           # fewer selectable columns than k, inside one segment
    t = to_dev(s, device)
    for order in ("index", "value"):
        for bounds in (False, True):
            st = to_dev(starts, device) if bounds else None
            en = to_dev(ends, device) if bounds else None
            want = otopk.topk_selector_oracle(s, k, starts=starts if bounds else None, ends=ends if bounds else None,
                                              order=order, neg_inf_is_masked=True)
            for two_stage in (True, False):
                out = torch.full((rows, k), -7, dtype=torch.int32, device=device)
                ops.topk_select(t, k, out=out, starts=st, ends=en, order=order, neg_inf_is_masked=True, two_stage=two_stage)
                torch.cuda.synchronize()
                np.testing.assert_array_equal(out.cpu().numpy(), want)
    a = _lib.TopkArgs()
    a.struct_size = C.sizeof(a)
    a.rows, a.width, a.row_stride, a.k = rows, width, width, k
    need = C.c_size_t(0)
    assert _lib.load().cppmega_mi355_topk_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)) == _lib.OK
    assert (need.value > 0) == (width % 4 == 0 and width > 16384)
