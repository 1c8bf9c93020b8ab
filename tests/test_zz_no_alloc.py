"""GPU: the entry point that allocates nothing (``cppmega_mi355_sparse_mla_fwd_noalloc``) against
``cppmega_mi355_sparse_mla_fwd`` with a caller workspace, both called through the C ABI.

Same kernels and the same key-split plan, so outputs must be bit-identical.  Two calls in a row
share the per-GPU static array, the second with a smaller input; a request beyond the array is
refused before anything is launched.
"""

import ctypes as C

import numpy as np
import pytest
import torch

from cppmega_mlx_amd import _lib, ops
from oracle import sparse_mla as om
from tests._inputs import bf16_pair, error_report, latent_cache, to_dev

pytestmark = pytest.mark.gpu


def _case(rng, device, B, H, Skv, topk, pow2):
    codes, scale, rope, rows = latent_cache(rng, B, Skv, 1, 512, 64, device, pow2=pow2)
    q, qf = bf16_pair(rng.standard_normal((B, 1, H, 576)), device)
    idx = np.stack([rng.choice(Skv, size=topk, replace=False) for _ in range(B)]).reshape(B, 1, 1, topk)
    idx[:, :, :, -5:] = -1
    return q, qf, codes, scale, rope, rows, idx


def _args(q, codes, scale, rope, idx_t, out, lse, sinks):
    spec = ops.QuantSpec(_lib.SCALE_F32_BLOCK, scale, 128)
    return ops._fill_mla_args(q, ops.QuantSpec(), codes, spec, rope, idx_t, 576 ** -0.5, 512, sinks, out, lse, "auto")


def test_noalloc_entry_point_matches_the_workspace_entry_point(device):
    lib = _lib.load()
    rng = np.random.default_rng(77)
    stream = _lib.current_stream(device)
    poison = torch.full((_lib.NOALLOC_SCRATCH_BYTES // 4,), float("nan"), dtype=torch.float32, device=device)
    for B, H, Skv, topk, pow2, with_sinks in ((6, 128, 8192, 2048, False, False), (2, 64, 4096, 1024, True, True)):
        print(f"case B={B} H={H} Skv={Skv} topk={topk} pow2={pow2} sinks={with_sinks}", flush=True)
        q, qf, codes, scale, rope, rows, idx = _case(rng, device, B, H, Skv, topk, pow2)
        idx_t = to_dev(idx.astype(np.int32), device)
        sinks_np = rng.standard_normal(H).astype(np.float32) if with_sinks else None
        sinks = None if sinks_np is None else to_dev(sinks_np, device)
        outs = []
        for entry in ("cppmega_mi355_sparse_mla_fwd", "cppmega_mi355_sparse_mla_fwd_noalloc"):
            out = torch.full((B, 1, H, 512), 7.0, dtype=torch.bfloat16, device=device)
            lse = torch.full((B, 1, H), 7.0, dtype=torch.float32, device=device)
            a = _args(q, codes, scale, rope, idx_t, out, lse, sinks)
            need = C.c_size_t(0)
            assert lib.cppmega_mi355_sparse_mla_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)) == _lib.OK
            assert 0 < need.value <= _lib.NOALLOC_SCRATCH_BYTES      # the split-KV path: scratch is in use
            assert lib.cppmega_mi355_sparse_mla_select_kernel(C.byref(a), C.sizeof(a)) == _lib.MLA_KERNEL_MFMA
            if entry.endswith("noalloc"):
                a.workspace, a.workspace_bytes = None, 0            # ignored by this entry point
            else:
                ws = poison[: (need.value + 3) // 4]                 # NaN-filled: nothing may depend on its contents
                a.workspace, a.workspace_bytes = ws.data_ptr(), need.value
            before = torch.cuda.memory_allocated(device)
            rc = getattr(lib, entry)(C.byref(a), C.sizeof(a), stream)
            assert rc == _lib.OK, lib.cppmega_mi355_last_error()
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated(device) == before
            outs.append((out, lse))
        (out_ws, lse_ws), (out_na, lse_na) = outs
        assert torch.equal(out_ws, out_na) and torch.equal(lse_ws, lse_na)
        want_out, want_lse = om.sparse_mla_oracle(qf, rows, idx, sm_scale=576 ** -0.5, d_v=512, sinks=sinks_np)
        err, ref = error_report(out_na.float().cpu().numpy(), want_out)
        assert err <= 2e-2 * ref
        assert np.abs(lse_na.cpu().numpy() - want_lse).max() <= 5e-3


def test_noalloc_entry_point_refuses_what_does_not_fit(device):
    """Shapes only: the check comes before any pointer is used."""
    lib = _lib.load()
    a = _lib.SparseMlaArgs()
    a.struct_size = C.sizeof(a)
    a.kernel = _lib.MLA_KERNEL_AUTO
    a.q_dtype, a.kv_dtype, a.kv_scale_kind, a.kv_scale_block = _lib.BF16, _lib.E4M3, _lib.SCALE_F32_BLOCK, 128
    a.rope_dtype, a.rope_dim, a.index_dtype, a.out_dtype = _lib.BF16, 64, _lib.I32, _lib.BF16
    a.batch, a.seq_q, a.heads, a.kv_groups, a.seq_kv, a.topk, a.d_qk, a.d_v = 96, 1, 128, 1, 65536, 2048, 576, 512
    a.sm_scale = 576 ** -0.5
    a.q = a.kv = a.kv_scale = a.kv_rope = a.indices = a.out = 0x1000     # 16-byte aligned, never dereferenced
    need = C.c_size_t(0)
    assert lib.cppmega_mi355_sparse_mla_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)) == _lib.OK
    assert need.value > _lib.NOALLOC_SCRATCH_BYTES
    assert lib.cppmega_mi355_sparse_mla_fwd_noalloc(C.byref(a), C.sizeof(a), None) == _lib.ERR_WORKSPACE
    assert b"static array holds" in lib.cppmega_mi355_last_error()
    torch.cuda.synchronize()
