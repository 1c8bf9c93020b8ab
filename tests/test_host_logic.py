"""Host-side mirror of the reference interface: policy, validation order, error
classes and the owner-output calling convention.  No kernel runs here; where a
launch would happen the launcher is replaced by a recording fake, the way the
reference's own boundary tests do (tests/test_tilelang_topk.py:357-463)."""

import pytest
import torch

from cppmega_mlx_amd import _lib, ops
from cppmega_mlx_amd.nn import sparse_mla as mla
from cppmega_mlx_amd.nn._tilelang import (
    _engine_dispatch as ed,
    fp8_msl_kernels,
    fp8_vecmat_path_c as vm,
    sparse_mla_blockscaled_path_c as bs,
    sparse_mla_fp8_path_c as f8,
    sparse_mla_path_c as pc,
    topk_selector as tk,
)
from cppmega_mlx_amd.runtime import kernel_policy as kp

import importlib

fg = importlib.import_module("cppmega_mlx_amd.nn._tilelang.fused_fp8_gemm")


# ---- kernel policy ----------------------------------------------------------

def test_selected_path_env_contract(monkeypatch):
    monkeypatch.delenv("CPPMEGA_KERNEL_PATH", raising=False)
    monkeypatch.delenv("CPPMEGA_KERNEL_PATH__SPARSE_MLA", raising=False)
    assert kp.selected_path("sparse_mla") is kp.KernelPath.AUTO
    for raw, want in [("ref", kp.KernelPath.REFERENCE), ("Reference", kp.KernelPath.REFERENCE), ("a", kp.KernelPath.REFERENCE),
                      ("PATH_B", kp.KernelPath.PATH_B), ("c", kp.KernelPath.PATH_C), ("bogus", kp.KernelPath.AUTO), ("", kp.KernelPath.AUTO)]:
        monkeypatch.setenv("CPPMEGA_KERNEL_PATH", raw)
        assert kp.selected_path("anything") is want
    monkeypatch.setenv("CPPMEGA_KERNEL_PATH", "ref")
    monkeypatch.setenv("CPPMEGA_KERNEL_PATH__SPARSE_MLA", "path_c")
    assert kp.selected_path("sparse_mla") is kp.KernelPath.PATH_C
    assert kp.selected_path("topk") is kp.KernelPath.REFERENCE
    with pytest.raises(TypeError):
        kp.selected_path(3)


def test_dispatch_log_is_bounded_and_validated():
    kp.clear_dispatch_log()
    for i in range(300):
        kp.record_dispatch("sparse_mla", kp.KernelPath.AUTO, f"k{i}")
    log = kp.get_dispatch_log()
    assert len(log) == 256 and log[-1] == {"op_name": "sparse_mla", "path": "auto", "kernel_used": "k299"}
    with pytest.raises(ValueError):
        kp.record_dispatch("", kp.KernelPath.AUTO, "k")
    with pytest.raises(TypeError):
        kp.record_dispatch("op", "auto", "k")
    kp.clear_dispatch_log()
    assert kp.get_dispatch_log() == []


# ---- shape contracts (raised before any device work) ---------------------------

def test_resolve_shapes_messages():
    q = torch.zeros(2, 3, 4, 16); kv = torch.zeros(2, 9, 2, 16); idx = torch.zeros(2, 3, 2, 5, dtype=torch.int32)
    s = mla._resolve_shapes(q, kv, idx, d_v=12)
    assert (s.head_kv, s.tail_dim, s.topk, s.seq_len_kv) == (2, 4, 5, 9)
    with pytest.raises(ValueError, match="q must be 4D"):
        mla._resolve_shapes(q[0], kv, idx, d_v=None)
    with pytest.raises(ValueError, match="q.batch=2 != kv.batch=1"):
        mla._resolve_shapes(q, kv[:1], idx, d_v=None)
    with pytest.raises(ValueError, match="not divisible"):
        mla._resolve_shapes(q[:, :, :3], kv, idx, d_v=None)
    with pytest.raises(ValueError, match="d_v must be in"):
        mla._resolve_shapes(q, kv, idx, d_v=0)
    with pytest.raises(ValueError, match="does not match"):
        mla._resolve_shapes(q, kv, idx[:, :2], d_v=None)


def test_policy_routing_of_sparse_mla_attention(monkeypatch):
    q = torch.zeros(1, 1, 2, 8, dtype=torch.bfloat16); kv = torch.zeros(1, 4, 1, 8, dtype=torch.bfloat16)
    idx = torch.zeros(1, 1, 1, 2, dtype=torch.int32)
    calls = []
    monkeypatch.setattr(mla, "_float_carrier_forward", lambda *a, **k: calls.append(k["kernel"]) or "out")
    monkeypatch.setattr(ops, "sparse_mla_selected_kernel", lambda *a, **k: "scalar")
    kp.clear_dispatch_log()
    monkeypatch.setenv("CPPMEGA_KERNEL_PATH", "ref")
    assert mla.sparse_mla_attention(q, kv, idx) == "out"
    monkeypatch.setenv("CPPMEGA_KERNEL_PATH", "path_c")
    mla.sparse_mla_attention(q, kv, idx)
    monkeypatch.setenv("CPPMEGA_KERNEL_PATH", "auto")
    mla.sparse_mla_attention(q, kv, idx)
    monkeypatch.setenv("CPPMEGA_KERNEL_PATH", "path_b")
    with pytest.raises(RuntimeError, match="retired"):
        mla.sparse_mla_attention(q, kv, idx)
    assert calls == ["scalar", "mfma", "scalar"]
    assert [e["kernel_used"] for e in kp.get_dispatch_log()] == [
        "hip_scalar_fp32", "hip_mfma_gfx950", "hip_scalar_fp32", "direct_msl_path_b_retired"]


def test_topk_validation_and_error_classes():
    s = torch.zeros(2, 8)
    out = torch.zeros(2, 3, dtype=torch.int32)
    with pytest.raises(ValueError, match="expects a \\(B, T\\) array"):
        tk.topk_selector_tilelang_direct(torch.zeros(8), 2, out=out)
    with pytest.raises(ValueError, match="topk must be in \\[1, 8\\]"):
        tk.topk_selector_tilelang_direct(s, 9, out=out)
    with pytest.raises(tk.TopKPathCDirectError, match="empty"):
        tk.topk_selector_tilelang_direct(torch.zeros(0, 8), 2, out=torch.zeros(0, 2, dtype=torch.int32))
    with pytest.raises(tk.TopKPathCDirectError, match="without hidden casts"):
        tk.topk_selector_tilelang_direct(s.double(), 3, out=out)
    with pytest.raises(ValueError, match="out shape must be"):
        tk.topk_selector_tilelang_direct(s, 2, out=out)
    with pytest.raises(ValueError, match="out dtype must be"):
        tk.topk_selector_tilelang_direct(s, 3, out=out.long())
    with pytest.raises(ValueError, match="unknown backend"):
        tk.topk_selector(s, 3, backend="cuda")
    with pytest.raises(RuntimeError, match="retired"):
        tk.topk_selector(s, 3, backend="metal")
    with pytest.raises(ValueError, match="topk must be >= 1"):
        tk.topk_selector_reference(s, 0)
    with pytest.raises(ValueError, match="exceeds sequence length"):
        tk.topk_selector_reference(s, 9)
    assert tk.topk_selector_metal(s, 3) is None
    assert tk.topk_selector_path_b_status().available is False
    # a CPU tensor reaches the boundary and is refused there: no CPU fallback exists
    with pytest.raises(tk.TopKPathCDirectError, match="no CPU path"):
        tk.topk_selector_tilelang_direct(s, 3, out=out)


def test_topk_owner_output_identity_and_argument_order(monkeypatch):
    seen = {}

    def fake(scores, k, *, out, starts, ends, order, neg_inf_is_masked):
        seen.update(scores=scores, k=k, out=out, starts=starts, ends=ends, order=order)
        return out

    monkeypatch.setattr(ops, "topk_select", fake)
    s = torch.zeros(2, 8); out = torch.zeros(2, 3, dtype=torch.int32)
    st = torch.zeros(2, dtype=torch.int32); en = torch.full((2,), 8, dtype=torch.int32)
    assert tk.topk_selector_tilelang_direct(s, 3, out=out, starts=st, ends=en) is out
    assert seen["scores"] is s and seen["out"] is out and seen["starts"] is st and seen["ends"] is en
    assert seen["order"] == "value" and seen["k"] == 3
    monkeypatch.setattr(ops, "topk_select", lambda *a, **k: torch.zeros(2, 3, dtype=torch.int32))
    with pytest.raises(tk.TopKPathCDirectError, match="caller-owned"):
        tk.topk_selector_tilelang_direct(s, 3, out=out)
    monkeypatch.setattr(tk, "topk_selector_path_c_status", lambda: tk.PathCStatus(False, "no device"))
    assert tk.topk_selector_tilelang(s, 3, out=out) is None


def _prepared(B=1, S=2, H=4, G=2, Skv=6, K=64, topk=3):
    return dict(
        q=torch.zeros(B, S, H, K, dtype=torch.uint8), kv=torch.zeros(B, Skv, G, K, dtype=torch.uint8),
        idx=torch.zeros(B, S, G, topk, dtype=torch.int32),
        q_e8=torch.zeros(B, S, H, K // 32, dtype=torch.uint8), kv_e8=torch.zeros(B, Skv, G, K // 32, dtype=torch.uint8),
        q_tok=torch.ones(B, S, H), kv_tok=torch.ones(B, Skv, G),
        out=torch.zeros(B, S, H, K, dtype=torch.float16), lse=torch.zeros(B, S, H),
    )


def test_blockscaled_prepared_validation(monkeypatch):
    p = _prepared()
    monkeypatch.setattr(bs, "sparse_mla_blockscaled_path_c_status", lambda: bs.SparseMLABlockScaledPathCStatus(True, "ok"))
    with pytest.raises(ValueError, match="requires both out and lse"):
        bs.sparse_mla_blockscaled_path_c_apply(p["q"], p["q_e8"], p["kv"], p["kv_e8"], p["idx"], sm_scale=1.0, out=p["out"])
    with pytest.raises(TypeError, match="uint8 E8M0 scales"):
        bs.sparse_mla_blockscaled_path_c_apply_direct(p["q"], p["q_tok"], p["kv"], p["kv_tok"], p["idx"], sm_scale=1.0, out=p["out"], lse=p["lse"])
    with pytest.raises(TypeError, match="uint8 FP8 storage"):
        bs.sparse_mla_blockscaled_path_c_apply_direct(p["q"].float(), p["q_e8"], p["kv"], p["kv_e8"], p["idx"], sm_scale=1.0, out=p["out"], lse=p["lse"])
    with pytest.raises(TypeError, match="int32 or torch.int64 indices"):
        bs.sparse_mla_blockscaled_path_c_apply_direct(p["q"], p["q_e8"], p["kv"], p["kv_e8"], p["idx"].short(), sm_scale=1.0, out=p["out"], lse=p["lse"])
    with pytest.raises(ValueError, match="q_scale must have shape"):
        bs.sparse_mla_blockscaled_path_c_apply_direct(p["q"], p["q_e8"][..., :1], p["kv"], p["kv_e8"], p["idx"], sm_scale=1.0, out=p["out"], lse=p["lse"])
    with pytest.raises(ValueError, match="d_v must be in"):
        bs.sparse_mla_blockscaled_path_c_apply_direct(p["q"], p["q_e8"], p["kv"], p["kv_e8"], p["idx"], sm_scale=1.0, out=p["out"], lse=p["lse"], d_v=65)
    with pytest.raises(ValueError, match="out must have shape"):
        bs.sparse_mla_blockscaled_path_c_apply_direct(p["q"], p["q_e8"], p["kv"], p["kv_e8"], p["idx"], sm_scale=1.0, out=p["out"][..., :8], lse=p["lse"])
    with pytest.raises(TypeError, match="lse must be torch.float32"):
        bs.sparse_mla_blockscaled_path_c_apply_direct(p["q"], p["q_e8"], p["kv"], p["kv_e8"], p["idx"], sm_scale=1.0, out=p["out"], lse=p["lse"].half())
    q2 = torch.zeros(1, 2, 4, 48, dtype=torch.uint8); kv2 = torch.zeros(1, 6, 2, 48, dtype=torch.uint8)
    with pytest.raises(ValueError, match="divisible by 32"):
        bs.sparse_mla_blockscaled_path_c_apply_direct(q2, p["q_e8"], kv2, p["kv_e8"], p["idx"], sm_scale=1.0, out=p["out"], lse=p["lse"])


def test_prepared_launch_receives_reference_argument_order_and_returns_owner_outputs(monkeypatch):
    p = _prepared()
    seen = {}

    def fake(q, kv, indices, **kw):
        seen.update(q=q, kv=kv, indices=indices, **kw)
        return kw["out"], kw["lse"]

    monkeypatch.setattr(ops, "sparse_mla_forward", fake)
    monkeypatch.setattr(bs, "sparse_mla_blockscaled_path_c_status", lambda: bs.SparseMLABlockScaledPathCStatus(True, "ok"))
    monkeypatch.setattr(f8, "sparse_mla_fp8_path_c_status", lambda: f8.SparseMLAFp8PathCStatus(True, "ok"))
    o, l = bs.sparse_mla_blockscaled_path_c_apply(p["q"], p["q_e8"], p["kv"], p["kv_e8"], p["idx"], sm_scale=0.5, out=p["out"], lse=p["lse"], return_lse=True)
    assert o is p["out"] and l is p["lse"]
    assert seen["q"] is p["q"] and seen["kv"] is p["kv"] and seen["indices"] is p["idx"]
    assert seen["q_spec"].kind == _lib.SCALE_E8M0 and seen["q_spec"].scale is p["q_e8"] and seen["kv_spec"].block == 32
    assert seen["sm_scale"] == 0.5 and seen["d_v"] == 64 and seen["sinks"] is None

    sinks = torch.zeros(4)
    o = f8.sparse_mla_fp8_path_c_apply(p["q"], p["q_tok"], p["kv"], p["kv_tok"], p["idx"], sm_scale=0.25, out=p["out"], lse=p["lse"], sinks=sinks, d_v=32) if False else None
    out32 = torch.zeros(1, 2, 4, 32, dtype=torch.bfloat16)
    o = f8.sparse_mla_fp8_path_c_apply(p["q"], p["q_tok"], p["kv"], p["kv_tok"], p["idx"], sm_scale=0.25, out=out32, lse=p["lse"], sinks=sinks, d_v=32)
    assert o is out32 and seen["sinks"] is sinks and seen["q_spec"].kind == _lib.SCALE_PER_TOKEN and seen["d_v"] == 32
    with pytest.raises(ValueError, match="sinks must have shape"):
        f8.sparse_mla_fp8_path_c_apply(p["q"], p["q_tok"], p["kv"], p["kv_tok"], p["idx"], sm_scale=0.25, out=out32, lse=p["lse"], sinks=torch.zeros(3), d_v=32)
    with pytest.raises(TypeError, match="out must be torch.float16"):
        f8.sparse_mla_fp8_path_c_apply(p["q"], p["q_tok"], p["kv"], p["kv_tok"], p["idx"], sm_scale=0.25, out=out32, lse=p["lse"], d_v=32, output_dtype=torch.float16)
    with pytest.raises(TypeError, match="must be float32; got"):
        f8.sparse_mla_fp8_path_c_apply(p["q"], p["q_e8"], p["kv"], p["kv_e8"], p["idx"], sm_scale=0.25, out=out32, lse=p["lse"], d_v=32)

    # latent layout: fp32 scale per 128 + bf16 rope tail + bf16 query
    q = torch.zeros(1, 2, 4, 320, dtype=torch.bfloat16); kv = torch.zeros(1, 6, 1, 256, dtype=torch.uint8)
    sc = torch.ones(1, 6, 1, 2); rope = torch.zeros(1, 6, 1, 64, dtype=torch.bfloat16)
    idx = torch.zeros(1, 2, 1, 3, dtype=torch.int64)
    out = torch.zeros(1, 2, 4, 256, dtype=torch.bfloat16)
    bs.sparse_mla_blockscaled_path_c_apply(q, None, kv, sc, idx, sm_scale=1.0, out=out, lse=p["lse"], kv_rope=rope)
    assert seen["kv_spec"].kind == _lib.SCALE_F32_BLOCK and seen["kv_spec"].block == 128 and seen["kv_rope"] is rope
    assert seen["q_spec"].kind == _lib.SCALE_NONE and seen["d_v"] == 256
    with pytest.raises(ValueError, match="latent width 256 \\+ rope width 0"):
        bs.sparse_mla_blockscaled_path_c_apply(q, None, kv, sc, idx, sm_scale=1.0, out=out, lse=p["lse"])

    def boom(*a, **k):
        raise _lib.NativeCallError(_lib.ERR_LAUNCH, "hipErrorLaunchFailure")

    monkeypatch.setattr(ops, "sparse_mla_forward", boom)
    with pytest.raises(bs.SparseMLABlockScaledPathCDirectError) as info:
        bs.sparse_mla_blockscaled_path_c_apply(p["q"], p["q_e8"], p["kv"], p["kv_e8"], p["idx"], sm_scale=0.5, out=p["out"], lse=p["lse"])
    assert isinstance(info.value.__cause__, _lib.NativeCallError)


def test_vecmat_validation_and_owner_output(monkeypatch):
    monkeypatch.setattr(vm, "fp8_vecmat_path_c_status", lambda: vm.FP8VecmatPathCStatus(True, "ok"))
    x = torch.zeros(64, dtype=torch.uint8); W = torch.zeros(8, 64, dtype=torch.uint8)
    sx = torch.ones(1); sw = torch.ones(8); out = torch.zeros(8)
    with pytest.raises(vm.FP8VecmatPathCLegacyError, match="no-out dispatch is retired"):
        vm.fp8_scaled_vecmat_path_c(x, W, scale_x=sx, scale_w=sw)
    with pytest.raises(TypeError, match="Python scalars"):
        vm.fp8_scaled_vecmat_path_c(x, W, scale_x=1.0, scale_w=sw, out=out)
    with pytest.raises(ValueError, match="shape mismatch"):
        vm.fp8_scaled_vecmat_path_c(x[:32], W, scale_x=sx, scale_w=sw, out=out)
    with pytest.raises(ValueError, match="scale_w size 1 or 8"):
        vm.fp8_scaled_vecmat_path_c(x, W, scale_x=sx, scale_w=torch.ones(3), out=out)
    with pytest.raises(ValueError, match="out shape must be"):
        vm.fp8_scaled_vecmat_path_c(x, W, scale_x=sx, scale_w=sw, out=torch.zeros(7))
    with pytest.raises(ValueError, match="out dtype must be"):
        vm.fp8_scaled_vecmat_path_c(x, W, scale_x=sx, scale_w=sw, out=out.double())
    seen = {}
    monkeypatch.setattr(ops, "fp8_vecmat", lambda x, w, s, **k: seen.update(x=x, w=w, s=s, **k) or k["out"])
    assert vm.fp8_scaled_vecmat_path_c(x, W, scale_x=sx, scale_w=sw, out=out) is out
    assert seen["scale_w_kind"] == _lib.WSCALE_PER_ROW and seen["scale_x"] is sx
    xb = torch.zeros(4, 256, dtype=torch.bfloat16); Wb = torch.zeros(130, 256, dtype=torch.uint8); ob = torch.zeros(4, 130, dtype=torch.bfloat16)
    vm.fp8_scaled_vecmat_path_c(xb, Wb, scale_x=None, scale_w=torch.ones(130, 2), out=ob)
    assert seen["scale_w_kind"] == _lib.WSCALE_ROW_BLOCK
    vm.fp8_scaled_vecmat_path_c(xb, Wb, scale_x=None, scale_w=torch.ones(2, 2), out=ob)
    assert seen["scale_w_kind"] == _lib.WSCALE_GRID_128
    with pytest.raises(TypeError, match="expected dtype"):
        fp8_msl_kernels.fp8_scaled_vecmat(x.float(), W, scale_x=1.0, scale_w=1.0)
    with pytest.raises(ValueError, match="multiple of 4"):
        fp8_msl_kernels.fp8_scaled_vecmat(x[:6], W[:, :6], scale_x=1.0, scale_w=1.0)
    with pytest.raises(ValueError, match="w_scale_inv shape"):
        fg.fused_fp8_gemm(Wb, torch.ones(3, 3), xb)
    with pytest.raises(TypeError, match="w_fp8 must be uint8"):
        fg.fused_fp8_gemm(Wb.float(), torch.ones(2, 2), xb)


def test_dispatch_lower_returns_owner_output_callable(monkeypatch):
    monkeypatch.delenv("CPPMEGA_MLX_TILELANG_ENGINE", raising=False)
    assert ed.tilelang_engine_mode() == "auto"
    kernel = ed.dispatch_lower(ed.topk_spec(k=3), "hip")
    assert kernel._tilelang_engine_target == "hip" and kernel.result_indices == (1,) and kernel.num_params == 4
    seen = {}
    monkeypatch.setitem(ed._LAUNCHERS, "topk_selector", lambda bufs, attrs: seen.update(bufs=bufs, attrs=attrs))
    ends, starts, scores = torch.zeros(2, dtype=torch.int32), torch.zeros(2, dtype=torch.int32), torch.zeros(2, 8)
    indices = torch.zeros(2, 3, dtype=torch.int32)
    assert kernel(ends, scores, starts, out=indices) is indices          # inputs in PrimFunc order minus outputs
    assert seen["bufs"]["indices"] is indices and seen["bufs"]["scores"] is scores and seen["bufs"]["ends"] is ends
    assert kernel(ends, indices, scores, starts) is indices               # full-ABI form
    with pytest.raises(ed.NativeKernelRuntimeError, match="caller-owned out="):
        kernel(ends, scores, starts)
    with pytest.raises(ed.NativeKernelRuntimeError, match="expected 3 inputs"):
        kernel(ends, scores, out=indices)
    with pytest.raises(ed.NativeKernelRuntimeError, match="Metal-only"):
        ed.dispatch_lower(ed.topk_spec(k=3), "hip", return_msl=True)
    with pytest.raises(ed.NativeKernelRuntimeError, match="target must be"):
        ed.dispatch_lower(ed.topk_spec(k=3), "metal")
    monkeypatch.setenv("CPPMEGA_MLX_TILELANG_ENGINE", "nonsense")
    with pytest.warns(UserWarning):
        assert ed.tilelang_engine_mode() == "auto"
    assert ed.normalize_out_idx(-1, num_params=5) == (4,)
    with pytest.raises(ed.NativeKernelRuntimeError, match="duplicate"):
        ed.normalize_out_idx([1, 1], num_params=3)
    mla_kernel = ed.dispatch_lower(ed.fp8_mla_spec(B=1, S=1, H=1, G=1, Skv=1, topk=1, K=4, d_v=4), "gfx950")
    assert mla_kernel.result_indices == (8, 9)


def test_path_c_float_carrier_owner_output_validation(monkeypatch):
    monkeypatch.setattr(pc, "sparse_mla_path_c_status", lambda: pc.SparseMLAPathCStatus(True, "ok"))
    q = torch.zeros(1, 1, 2, 8, dtype=torch.bfloat16); kv = torch.zeros(1, 4, 1, 8, dtype=torch.bfloat16)
    idx = torch.zeros(1, 1, 1, 2, dtype=torch.int32)
    out = torch.zeros(1, 1, 2, 8, dtype=torch.bfloat16); lse = torch.zeros(1, 1, 2)
    with pytest.raises(pc.SparseMLAPathCDirectError, match="together"):
        pc.sparse_mla_fwd_path_c(q, kv, idx, out=out)
    with pytest.raises(ValueError, match="sm_scale_buf"):
        pc.sparse_mla_fwd_path_c(q, kv, idx, sm_scale_buf=torch.ones(2), out=out, lse=lse)
    with pytest.raises(ValueError, match="out must have shape"):
        pc.sparse_mla_fwd_path_c(q, kv, idx, sm_scale_buf=torch.ones(1), out=out[..., :4], lse=lse)
    with pytest.raises(TypeError, match="indices must be int32 or int64"):
        pc.sparse_mla_fwd_path_c(q, kv, idx.short(), sm_scale_buf=torch.ones(1), out=out, lse=lse)


# ---- index producers and the sparse FP8 cache: argument contracts (no GPU needed) -----------

def test_causal_sparse_indices_argument_contract():
    from cppmega_mlx_amd.nn.attention import causal_sparse_indices
    for bad in (dict(batch_size=0), dict(seq_length=0), dict(kv_group=0), dict(topk=0), dict(query_offset=-1), dict(key_length=0)):
        args = dict(batch_size=1, seq_length=2, kv_group=1, topk=2, query_offset=0, key_length=2)
        args.update(bad)
        with pytest.raises(ValueError):
            causal_sparse_indices(**args, device="cpu")


def test_mask_sparse_indices_argument_contract():
    import torch
    from cppmega_mlx_amd.nn.attention import sparse_indices_from_attention_mask
    kw = dict(batch_size=1, seq_length=3, kv_group=1, topk=2, key_length=4)
    m = torch.ones((3, 4), dtype=torch.bool)
    with pytest.raises(TypeError):
        sparse_indices_from_attention_mask([[True]], **kw)
    with pytest.raises(ValueError):
        sparse_indices_from_attention_mask(m[None, None, None], **kw)
    with pytest.raises(ValueError):
        sparse_indices_from_attention_mask(m, **{**kw, "key_length": 5})
    with pytest.raises(ValueError):
        sparse_indices_from_attention_mask(m.expand(3, 3, 4), **kw)
    with pytest.raises(ValueError):
        sparse_indices_from_attention_mask(m.expand(1, 3, 3, 4), **kw)
    for bad in ("batch_size", "seq_length", "kv_group", "topk", "key_length"):
        with pytest.raises(ValueError):
            sparse_indices_from_attention_mask(m, **{**kw, bad: 0})


def test_sparse_fp8_cache_config_contract():
    from cppmega_mlx_amd.inference import SparseFP8KVCacheConfig
    ok = dict(num_layers=1, batch_size=1, num_kv_heads=1, head_dim=512, max_seq_len=16)
    SparseFP8KVCacheConfig(**ok)
    for bad in ("num_layers", "batch_size", "num_kv_heads", "head_dim", "max_seq_len"):
        with pytest.raises(ValueError):
            SparseFP8KVCacheConfig(**{**ok, bad: 0})
        with pytest.raises(TypeError):
            SparseFP8KVCacheConfig(**{**ok, bad: 1.5})
    with pytest.raises(ValueError):
        SparseFP8KVCacheConfig(**{**ok, "head_dim": 100})
    with pytest.raises(ValueError):
        SparseFP8KVCacheConfig(**{**ok, "scale_block": 64})
    with pytest.raises(ValueError):
        SparseFP8KVCacheConfig(**{**ok, "rope_dim": -1})
