"""Host-side launch helpers: torch tensors in, one C-ABI call out.

These functions fill the argument structs of ``include/cppmega_mi355.h`` from
dense device tensors and enqueue the kernel on torch's current HIP stream.
They validate what the C side cannot see (tensor ranks, devices, contiguity)
and leave value/shape contracts to the library, whose status codes come back as
``ValueError`` / ``TypeError`` / ``NativeCallError``.  Outputs are caller-owned;
the only tensor this module ever creates is the split-KV / split-K workspace,
kept per device and reused, unless the caller passes ``workspace=``.
"""

from __future__ import annotations

import ctypes as C
import threading
from dataclasses import dataclass

import torch

from . import _lib

_ws_lock = threading.Lock()
_workspaces: dict[tuple[int, int], torch.Tensor] = {}


def _workspace(device: torch.device, nbytes: int, stream: int) -> torch.Tensor | None:
    """Per-(device, stream) scratch, grown geometrically, never shrunk."""
    if nbytes <= 0:
        return None
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    with _ws_lock:
        buf = _workspaces.get(key)
        if buf is None or buf.numel() < nbytes:
            size = max(nbytes, 1 << 20)
            if buf is not None:
                size = max(size, 2 * buf.numel())
            buf = torch.zeros(size, dtype=torch.uint8, device=device)
            _workspaces[key] = buf
        return buf


def _dtype_or_raise(t: torch.Tensor, name: str, allowed: tuple[int, ...]) -> int:
    code = _lib.dtype_code(t)
    if code is None or code not in allowed:
        raise TypeError(f"{name}: unsupported dtype {t.dtype}")
    return code


# ---------------------------------------------------------------------------
# top-k
# ---------------------------------------------------------------------------

def topk_select(
    scores: torch.Tensor,
    k: int,
    *,
    out: torch.Tensor,
    starts: torch.Tensor | None = None,
    ends: torch.Tensor | None = None,
    order: str = "index",
    neg_inf_is_masked: bool = False,
    workspace: torch.Tensor | None = None,
    two_stage: bool = True,
) -> torch.Tensor:
    """Write the per-row top-k indices of ``scores`` (rows, width) into ``out`` (rows, k).  Rows wider
    than 16384 columns go through a workspace in two stages unless ``two_stage`` is off."""
    _lib.require_device_tensor(scores, "scores")
    _lib.require_device_tensor(out, "out", scores)
    if scores.ndim != 2:
        raise ValueError(f"topk_selector expects a (B, T) array; got shape {tuple(scores.shape)}")
    rows, width = scores.shape
    if out.dtype != torch.int32:
        raise ValueError(f"topk_selector: out dtype must be torch.int32; got {out.dtype}")
    if tuple(out.shape) != (rows, int(k)):
        raise ValueError(f"topk_selector: out shape must be ({rows}, {int(k)}); got {tuple(out.shape)}")
    if order not in ("index", "value"):
        raise ValueError(f"unknown order {order!r}")
    for name, bound in (("starts", starts), ("ends", ends)):
        if bound is None:
            continue
        _lib.require_device_tensor(bound, name, scores)
        if tuple(bound.shape) != (rows,) or bound.dtype != torch.int32:
            raise ValueError(f"starts/ends must be int32 with shape ({rows},); got {name}={tuple(bound.shape)} {bound.dtype}")
    args = _lib.TopkArgs()
    args.struct_size = C.sizeof(args)
    args.score_dtype = _dtype_or_raise(scores, "scores", (_lib.F32, _lib.F16, _lib.BF16))
    args.scores = scores.data_ptr()
    args.row_stride = width
    args.rows, args.width, args.k = rows, width, int(k)
    args.order = _lib.TOPK_ORDER_VALUE if order == "value" else _lib.TOPK_ORDER_INDEX
    args.starts = _lib.ptr(starts)
    args.ends = _lib.ptr(ends)
    args.indices = out.data_ptr()
    args.neg_inf_is_masked = 1 if neg_inf_is_masked else 0
    lib = _lib.load()
    stream = _lib.current_stream(scores.device)
    need = C.c_size_t(0)
    _lib.check(lib.cppmega_mi355_topk_workspace_bytes(C.byref(args), C.sizeof(args), C.byref(need)), "topk_select")
    if need.value and two_stage:
        if workspace is None:
            workspace = _workspace(scores.device, need.value, stream)
        else:
            _lib.require_device_tensor(workspace, "workspace", scores)
        args.workspace = workspace.data_ptr()
        args.workspace_bytes = workspace.numel() * workspace.element_size()
    with torch.cuda.device(scores.device):
        rc = lib.cppmega_mi355_topk_select(C.byref(args), C.sizeof(args), stream)
    _lib.check(rc, "topk_select")
    return out


# ---------------------------------------------------------------------------
# indexer scores -> top-k
# ---------------------------------------------------------------------------
def _fill_indexer_args(q, k, weights, sm_scale, topk, out, mask, starts, ends, order, scores_out, chunk_rows):
    if q.ndim != 4 or k.ndim != 3 or weights.ndim != 3:
        raise ValueError("indexer expects q [B,Sq,H,D], k [B,Skv,D], weights [B,Sq,H]")
    B, Sq, H, D = q.shape
    Skv = k.shape[1]
    if tuple(weights.shape) != (B, Sq, H) or k.shape[0] != B or k.shape[2] != D:
        raise ValueError(f"indexer shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}, weights {tuple(weights.shape)}")
    if order not in ("index", "value"):
        raise ValueError(f"unknown order {order!r}")
    a = _lib.IndexerArgs()
    a.struct_size = C.sizeof(a)
    a.q_dtype = _dtype_or_raise(q, "q", (_lib.F32, _lib.BF16))
    a.w_dtype = _dtype_or_raise(weights, "weights", (_lib.F32, _lib.BF16))
    a.k_dtype = _dtype_or_raise(k, "k", (_lib.F32, _lib.BF16))
    a.q, a.weights, a.k = q.data_ptr(), weights.data_ptr(), k.data_ptr()
    if mask is not None:
        if tuple(mask.shape) != (B, Sq, Skv):
            raise ValueError(f"mask must have shape {(B, Sq, Skv)}; got {tuple(mask.shape)}")
        a.mask, a.mask_dtype = mask.data_ptr(), _dtype_or_raise(mask, "mask", (_lib.F32, _lib.F16, _lib.BF16))
    for name, bound in (("starts", starts), ("ends", ends)):
        if bound is not None and (bound.numel() != B * Sq or bound.dtype != torch.int32):
            raise ValueError(f"{name} must be int32 with {B * Sq} entries; got {bound.dtype} {tuple(bound.shape)}")
    a.starts, a.ends = _lib.ptr(starts), _lib.ptr(ends)
    a.order = _lib.TOPK_ORDER_VALUE if order == "value" else _lib.TOPK_ORDER_INDEX
    a.batch, a.seq_q, a.heads, a.head_dim, a.seq_kv, a.topk = B, Sq, H, D, Skv, int(topk)
    a.sm_scale = float(sm_scale)
    a.chunk_rows = int(chunk_rows)
    if out is not None:
        if out.dtype != torch.int32 or tuple(out.shape) != (B, Sq, int(topk)):
            raise ValueError(f"out must be int32 with shape {(B, Sq, int(topk))}; got {out.dtype} {tuple(out.shape)}")
        a.indices = out.data_ptr()
    if scores_out is not None:
        if scores_out.dtype != torch.float32 or tuple(scores_out.shape) != (B, Sq, Skv):
            raise ValueError(f"scores_out must be float32 with shape {(B, Sq, Skv)}")
        a.scores_out = scores_out.data_ptr()
    return a


def indexer_topk_workspace_bytes(q, k, weights, *, topk: int, chunk_rows: int = 0) -> int:
    a = _fill_indexer_args(q, k, weights, 1.0, topk, None, None, None, None, "index", None, chunk_rows)
    need = C.c_size_t(0)
    _lib.check(_lib.load().cppmega_mi355_indexer_topk_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)), "indexer_topk")
    return int(need.value)


def indexer_topk(
    q: torch.Tensor,
    k: torch.Tensor,
    weights: torch.Tensor,
    *,
    sm_scale: float,
    topk: int,
    out: torch.Tensor,
    mask: torch.Tensor | None = None,
    starts: torch.Tensor | None = None,
    ends: torch.Tensor | None = None,
    order: str = "index",
    scores_out: torch.Tensor | None = None,
    workspace: torch.Tensor | None = None,
    chunk_rows: int = 0,
) -> torch.Tensor:
    """indices[b,s,:] = top-k over t of sm_scale * sum_h weights[b,s,h] * (q[b,s,h,:] . k[b,t,:]) (+ mask),
    into caller-owned int32 ``out`` [B,Sq,topk].  ``scores_out`` (float32 [B,Sq,Skv]) keeps every score."""
    for name, t in (("q", q), ("k", k), ("weights", weights), ("out", out), ("mask", mask), ("starts", starts),
                    ("ends", ends), ("scores_out", scores_out)):
        if t is not None:
            _lib.require_device_tensor(t, name, q if name != "q" else None)
    a = _fill_indexer_args(q, k, weights, sm_scale, topk, out, mask, starts, ends, order, scores_out, chunk_rows)
    lib = _lib.load()
    stream = _lib.current_stream(q.device)
    need = C.c_size_t(0)
    _lib.check(lib.cppmega_mi355_indexer_topk_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)), "indexer_topk")
    if need.value:
        if workspace is None:
            workspace = _workspace(q.device, need.value, stream)
        else:
            _lib.require_device_tensor(workspace, "workspace", q)
        a.workspace = workspace.data_ptr()
        a.workspace_bytes = workspace.numel() * workspace.element_size()
    with torch.cuda.device(q.device):
        rc = lib.cppmega_mi355_indexer_topk(C.byref(a), C.sizeof(a), stream)
    _lib.check(rc, "indexer_topk")
    return out


# ---------------------------------------------------------------------------
# per-head projections (absorbed MLA decode) and block-128 FP8 weight dequantisation
# ---------------------------------------------------------------------------
def head_gemm(x: torch.Tensor, w: torch.Tensor, *, out: torch.Tensor) -> torch.Tensor:
    """out[m, g, n] = sum_k x[m, g, k] * w[g, n, k] into caller-owned ``out``.

    ``x`` [M, G, K] and ``out`` [M, G, N] may be views with their own row and group strides (the
    last axis contiguous); ``w`` [G, N, K] is dense.  float32 / bfloat16 operands, fp32 accumulation."""
    for name, t in (("x", x), ("w", w), ("out", out)):
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"{name} must be a torch.Tensor")
        if not t.is_cuda:
            raise _lib.NativeCallError(_lib.ERR_UNSUPPORTED, f"{name} lives on {t.device}; there is no CPU path")
    if x.ndim != 3 or w.ndim != 3 or out.ndim != 3:
        raise ValueError("head_gemm expects x [M,G,K], w [G,N,K], out [M,G,N]")
    M, G, K = x.shape
    N = w.shape[1]
    if tuple(w.shape) != (G, N, K) or tuple(out.shape) != (M, G, N):
        raise ValueError(f"head_gemm shape mismatch: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    if not w.is_contiguous():
        raise ValueError("head_gemm: w must be dense [G, N, K] (the contraction index contiguous)")
    for name, t in (("x", x), ("out", out)):
        if t.shape[-1] > 1 and t.stride(-1) != 1:
            raise ValueError(f"head_gemm: the last axis of {name} must be contiguous; got strides {t.stride()}")
    a = _lib.HeadGemmArgs()
    a.struct_size = C.sizeof(a)
    a.x_dtype = _dtype_or_raise(x, "x", (_lib.F32, _lib.BF16))
    a.w_dtype = _dtype_or_raise(w, "w", (_lib.F32, _lib.BF16))
    a.y_dtype = _dtype_or_raise(out, "out", (_lib.F32, _lib.F16, _lib.BF16))
    a.x, a.w, a.y = x.data_ptr(), w.data_ptr(), out.data_ptr()
    a.m, a.groups, a.n, a.k = M, G, N, K
    a.x_row_pitch, a.x_group_pitch = x.stride(0), x.stride(1)
    a.y_row_pitch, a.y_group_pitch = out.stride(0), out.stride(1)
    with torch.cuda.device(x.device):
        rc = _lib.load().cppmega_mi355_head_gemm(C.byref(a), C.sizeof(a), _lib.current_stream(x.device))
    _lib.check(rc, "head_gemm")
    return out


def dequant_block_fp8(weight: torch.Tensor, scale_inv: torch.Tensor, *, out: torch.Tensor) -> torch.Tensor:
    """out[r, c] = dec(weight[r, c]) * scale_inv[r // 128, c // 128] (e4m3 bytes, float32 scales)."""
    for name, t in (("weight", weight), ("scale_inv", scale_inv), ("out", out)):
        _lib.require_device_tensor(t, name, weight if name != "weight" else None)
    if weight.ndim != 2 or weight.dtype != torch.uint8:
        raise TypeError(f"weight must be 2D uint8 (fp8 storage); got {weight.dtype} {tuple(weight.shape)}")
    m, n = weight.shape
    want = ((m + 127) // 128, (n + 127) // 128)
    if tuple(scale_inv.shape) != want or scale_inv.dtype != torch.float32:
        raise ValueError(f"scale_inv must be float32 with shape {want}; got {scale_inv.dtype} {tuple(scale_inv.shape)}")
    if tuple(out.shape) != (m, n):
        raise ValueError(f"out must have shape {(m, n)}; got {tuple(out.shape)}")
    a = _lib.DequantBlockArgs()
    a.struct_size = C.sizeof(a)
    a.out_dtype = _dtype_or_raise(out, "out", (_lib.F32, _lib.F16, _lib.BF16))
    a.weight, a.scale_inv, a.out = weight.data_ptr(), scale_inv.data_ptr(), out.data_ptr()
    a.rows, a.cols = m, n
    with torch.cuda.device(weight.device):
        rc = _lib.load().cppmega_mi355_dequant_block_fp8(C.byref(a), C.sizeof(a), _lib.current_stream(weight.device))
    _lib.check(rc, "dequant_block_fp8")
    return out


# ---------------------------------------------------------------------------
# DSA indexer KL loss (training side)
# ---------------------------------------------------------------------------
def dsa_indexer_loss(query: torch.Tensor, key: torch.Tensor, index_scores: torch.Tensor, *, softmax_scale: float,
                     out: torch.Tensor, index_mask: torch.Tensor | None = None,
                     topk_indices: torch.Tensor | None = None) -> torch.Tensor:
    """Per-position KL(attention || index) into caller-owned float32 ``out`` [AB, ASq];
    ``query`` [ASq, AB, AH, AD], ``key`` [Sk, AB, AH, AD], ``index_scores`` / ``index_mask`` float32 [AB, ASq, Sk];
    ``topk_indices`` int32 / int64 [AB, ASq, topk] restricts both distributions to the listed keys."""
    for name, t in (("query", query), ("key", key), ("index_scores", index_scores), ("out", out), ("index_mask", index_mask),
                    ("topk_indices", topk_indices)):
        if t is not None:
            _lib.require_device_tensor(t, name, query if name != "query" else None)
    if query.ndim != 4 or key.ndim != 4 or tuple(query.shape[1:]) != tuple(key.shape[1:]):
        raise ValueError(f"query/key shape mismatch: query {tuple(query.shape)}, key {tuple(key.shape)}")
    ASq, AB, AH, AD = query.shape
    Sk = key.shape[0]
    if key.dtype != query.dtype:
        raise TypeError("query/key dtypes must match")
    for name, t in (("index_scores", index_scores), ("index_mask", index_mask)):
        if t is not None and (tuple(t.shape) != (AB, ASq, Sk) or t.dtype != torch.float32):
            raise ValueError(f"{name} must be float32 with shape {(AB, ASq, Sk)}; got {t.dtype} {tuple(t.shape)}")
    if tuple(out.shape) != (AB, ASq) or out.dtype != torch.float32:
        raise ValueError(f"out must be float32 with shape {(AB, ASq)}; got {out.dtype} {tuple(out.shape)}")
    a = _lib.DsaLossArgs()
    a.struct_size = C.sizeof(a)
    a.in_dtype = _dtype_or_raise(query, "query", (_lib.F32, _lib.F16, _lib.BF16))
    a.query, a.key, a.index_scores, a.index_mask, a.loss = (query.data_ptr(), key.data_ptr(), index_scores.data_ptr(),
                                                            _lib.ptr(index_mask), out.data_ptr())
    a.seq_q, a.batch, a.heads, a.head_dim, a.seq_k = ASq, AB, AH, AD, Sk
    a.softmax_scale = float(softmax_scale)
    if topk_indices is not None:
        if topk_indices.ndim != 3 or tuple(topk_indices.shape[:2]) != (AB, ASq):
            raise ValueError(f"topk_indices must have shape (AB={AB}, ASq={ASq}, TOPK); got {tuple(topk_indices.shape)}")
        a.topk_indices, a.topk = topk_indices.data_ptr(), int(topk_indices.shape[2])
        a.index_dtype = _dtype_or_raise(topk_indices, "topk_indices", (_lib.I32, _lib.I64))
    with torch.cuda.device(query.device):
        rc = _lib.load().cppmega_mi355_dsa_indexer_loss(C.byref(a), C.sizeof(a), _lib.current_stream(query.device))
    _lib.check(rc, "dsa_indexer_loss")
    return out


# ---------------------------------------------------------------------------
# sparse MLA
# ---------------------------------------------------------------------------

@dataclass
class QuantSpec:
    """How one operand of the attention is stored."""

    kind: int = _lib.SCALE_NONE
    scale: torch.Tensor | None = None
    block: int = 0


_KERNELS = {"auto": _lib.MLA_KERNEL_AUTO, "scalar": _lib.MLA_KERNEL_SCALAR, "mfma": _lib.MLA_KERNEL_MFMA}


def _cache_pitch(kv, kv_scale, kv_rope) -> int:
    """Key rows between two batches of the cache buffers: one value for kv, its scales and its rope."""
    pitches = {name: _lib.batch_pitch(t) for name, t in (("kv", kv), ("kv_scale", kv_scale), ("kv_rope", kv_rope))
               if t is not None and t.ndim >= 2 and t.shape[:2] == kv.shape[:2]}
    if len(set(pitches.values())) > 1 or None in pitches.values():
        raise ValueError(f"kv, kv_scale and kv_rope must share one batch pitch; got {pitches}")
    return int(pitches["kv"])


def _fill_mla_args(q, q_spec, kv, kv_spec, kv_rope, indices, sm_scale, d_v, sinks, out, lse, kernel, has_sinks=None):
    B, S, H, d_qk = q.shape
    _, Skv, G, d_kv = kv.shape
    rope_dim = 0 if kv_rope is None else kv_rope.shape[-1]
    a = _lib.SparseMlaArgs()
    a.struct_size = C.sizeof(a)
    a.kernel = _KERNELS[kernel]
    a.q = q.data_ptr()
    a.q_scale = _lib.ptr(q_spec.scale)
    a.q_dtype = _dtype_or_raise(q, "q", (_lib.F32, _lib.F16, _lib.BF16, _lib.E4M3))
    a.q_scale_kind, a.q_scale_block = q_spec.kind, q_spec.block
    a.kv = kv.data_ptr()
    a.kv_scale = _lib.ptr(kv_spec.scale)
    a.kv_dtype = _dtype_or_raise(kv, "kv", (_lib.F32, _lib.F16, _lib.BF16, _lib.E4M3))
    a.kv_scale_kind, a.kv_scale_block = kv_spec.kind, kv_spec.block
    a.kv_rope = _lib.ptr(kv_rope)
    a.rope_dtype = _dtype_or_raise(kv_rope, "kv_rope", (_lib.F32, _lib.F16, _lib.BF16)) if kv_rope is not None else 0
    a.rope_dim = rope_dim
    a.indices = indices.data_ptr()
    a.index_dtype = _dtype_or_raise(indices, "indices", (_lib.I32, _lib.I64))
    a.batch, a.seq_q, a.heads, a.kv_groups, a.seq_kv, a.topk = B, S, H, G, Skv, indices.shape[-1]
    a.d_qk, a.d_v = d_qk, int(d_v)
    if isinstance(sm_scale, torch.Tensor):
        _lib.require_device_tensor(sm_scale, "sm_scale", q)
        if sm_scale.dtype != torch.float32 or sm_scale.numel() != 1:
            raise ValueError(f"a device sm_scale must be one float32; got {sm_scale.dtype} {tuple(sm_scale.shape)}")
        a.sm_scale, a.sm_scale_dev = 0.0, sm_scale.data_ptr()
    else:
        a.sm_scale = float(sm_scale)
    if has_sinks is not None:
        _lib.require_device_tensor(has_sinks, "has_sinks", q)
        if has_sinks.dtype != torch.int32 or has_sinks.numel() != 1:
            raise ValueError(f"has_sinks must be one int32; got {has_sinks.dtype} {tuple(has_sinks.shape)}")
        a.has_sinks_dev = has_sinks.data_ptr()
    pitch = _cache_pitch(kv, kv_spec.scale, kv_rope)
    a.seq_kv_pitch = 0 if pitch == Skv else pitch
    a.sinks = _lib.ptr(sinks)
    a.out = _lib.ptr(out)
    a.lse = _lib.ptr(lse)
    a.out_dtype = _dtype_or_raise(out, "out", (_lib.F32, _lib.F16, _lib.BF16)) if out is not None else _lib.BF16
    return a


def sparse_mla_forward(
    q: torch.Tensor,
    kv: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float | torch.Tensor,
    d_v: int,
    out: torch.Tensor,
    lse: torch.Tensor | None = None,
    q_spec: QuantSpec | None = None,
    kv_spec: QuantSpec | None = None,
    kv_rope: torch.Tensor | None = None,
    sinks: torch.Tensor | None = None,
    has_sinks: torch.Tensor | None = None,
    kernel: str = "auto",
    workspace: torch.Tensor | None = None,
    no_alloc: bool = False,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Sparse MLA forward into caller-owned ``out`` [B,S,H,d_v] (and ``lse`` [B,S,H]).

    ``no_alloc`` takes the entry point whose split-KV partials live in the library's fixed
    per-GPU array (``_lib.NOALLOC_SCRATCH_BYTES``): no workspace tensor, nothing allocated;
    shapes that need more raise, and calls overlapping on one GPU must be ordered.

    ``sm_scale`` is a Python float or a device float32[1] the kernels read on the stream (the
    reference's ``sm_scale_buf``); ``has_sinks`` is an optional device int32[1] that switches
    ``sinks`` off when it holds 0.  ``kv`` (with its scales and rope) may be a ``cache[:, :n]``
    view of a dense buffer: only the first ``n`` rows of every batch are attendable.
    """
    q_spec = q_spec or QuantSpec()
    kv_spec = kv_spec or QuantSpec()
    if kernel not in _KERNELS:
        raise ValueError(f"unknown kernel {kernel!r}")
    named = [("q", q), ("kv", kv), ("indices", indices), ("out", out), ("lse", lse), ("kv_rope", kv_rope),
             ("sinks", sinks), ("q_scale", q_spec.scale), ("kv_scale", kv_spec.scale)]
    for name, t in named:
        if t is not None:
            _lib.require_device_tensor(t, name, q if name != "q" else None,
                                       allow_batch_pitch=name in ("kv", "kv_rope", "kv_scale"))
    if q.ndim != 4 or kv.ndim != 4 or indices.ndim != 4:
        raise ValueError("sparse_mla: q, kv and indices must be rank 4")
    B, S, H, _ = q.shape
    if tuple(out.shape) != (B, S, H, int(d_v)):
        raise ValueError(f"out must have shape {(B, S, H, int(d_v))}; got {tuple(out.shape)}")
    if lse is not None and (tuple(lse.shape) != (B, S, H) or lse.dtype != torch.float32):
        raise ValueError(f"lse must be float32 with shape {(B, S, H)}; got {lse.dtype} {tuple(lse.shape)}")
    if sinks is not None and (tuple(sinks.shape) != (H,) or sinks.dtype != torch.float32):
        raise ValueError(f"sinks must be float32 with shape ({H},), got {sinks.dtype} {tuple(sinks.shape)}")
    a = _fill_mla_args(q, q_spec, kv, kv_spec, kv_rope, indices, sm_scale, d_v, sinks, out, lse, kernel, has_sinks)
    lib = _lib.load()
    stream = _lib.current_stream(q.device)
    if no_alloc:
        with torch.cuda.device(q.device):
            rc = lib.cppmega_mi355_sparse_mla_fwd_noalloc(C.byref(a), C.sizeof(a), stream)
        _lib.check(rc, "sparse_mla_fwd_noalloc")
        return out, lse
    need = C.c_size_t(0)
    _lib.check(lib.cppmega_mi355_sparse_mla_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)), "sparse_mla")
    if need.value:
        if workspace is None:
            workspace = _workspace(q.device, need.value, stream)
        else:
            _lib.require_device_tensor(workspace, "workspace", q)
        a.workspace = workspace.data_ptr()
        a.workspace_bytes = workspace.numel() * workspace.element_size()
    with torch.cuda.device(q.device):
        rc = lib.cppmega_mi355_sparse_mla_fwd(C.byref(a), C.sizeof(a), stream)
    _lib.check(rc, "sparse_mla_fwd")
    return out, lse


def sparse_mla_backward(q: torch.Tensor, kv: torch.Tensor, d_out: torch.Tensor, indices: torch.Tensor, *,
                        sm_scale: float | torch.Tensor, d_v: int, dq: torch.Tensor, dkv: torch.Tensor,
                        clear_dkv: bool = True, q_scale: torch.Tensor | None = None,
                        kv_scale: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """Gradients of the sparse MLA forward into caller-owned ``dq`` [B,S,H,D] (any float carrier) and
    ``dkv`` [B,Skv,G,D] (float32, accumulated with atomic adds; cleared first unless ``clear_dkv``
    is off).  q / kv are float carriers, or uint8 e4m3 bytes with per-token float32 scales."""
    for name, t in (("q", q), ("kv", kv), ("d_out", d_out), ("indices", indices), ("dq", dq), ("dkv", dkv),
                    ("q_scale", q_scale), ("kv_scale", kv_scale)):
        if t is not None:
            _lib.require_device_tensor(t, name, q if name != "q" else None)
    if q.ndim != 4 or kv.ndim != 4 or indices.ndim != 4:
        raise ValueError("sparse_mla: q, kv and indices must be rank 4")
    B, S, H, D = q.shape
    Bk, Skv, G, Dk = kv.shape
    if Bk != B or Dk != D:
        raise ValueError(f"kv must have shape ({B}, Skv, G, {D}) to go with q {tuple(q.shape)}; got {tuple(kv.shape)}")
    if G < 1 or H % G:
        raise ValueError(f"heads {H} not divisible by kv_group {G}")
    if tuple(indices.shape[:3]) != (B, S, G):
        raise ValueError(f"indices shape {tuple(indices.shape)} does not match (B,S,G,topk)=({B},{S},{G},*)")
    if not 0 < int(d_v) <= D:
        raise ValueError(f"d_v must be in (0, {D}], got {int(d_v)}")
    if tuple(d_out.shape) != (B, S, H, int(d_v)):
        raise ValueError(f"d_out must have shape {(B, S, H, int(d_v))}; got {tuple(d_out.shape)}")
    if tuple(dq.shape) != (B, S, H, D):
        raise ValueError(f"dq must have shape {(B, S, H, D)}; got {tuple(dq.shape)}")
    if tuple(dkv.shape) != tuple(kv.shape) or dkv.dtype != torch.float32:
        raise ValueError(f"dkv must be float32 with shape {tuple(kv.shape)}; got {dkv.dtype} {tuple(dkv.shape)}")
    a = _lib.SparseMlaBwdArgs()
    a.struct_size = C.sizeof(a)
    a.q_dtype = _dtype_or_raise(q, "q", (_lib.F32, _lib.F16, _lib.BF16, _lib.E4M3))
    a.kv_dtype = _dtype_or_raise(kv, "kv", (_lib.F32, _lib.F16, _lib.BF16, _lib.E4M3))
    a.d_out_dtype = _dtype_or_raise(d_out, "d_out", (_lib.F32, _lib.F16, _lib.BF16))
    a.dq_dtype = _dtype_or_raise(dq, "dq", (_lib.F32, _lib.F16, _lib.BF16))
    for name, t, scale, want in (("q", q, q_scale, (B, S, H)), ("kv", kv, kv_scale, (B, Skv, G))):
        if t.dtype == torch.uint8 and (scale is None or tuple(scale.shape) != want or scale.dtype != torch.float32):
            raise ValueError(f"{name}_scale must be float32 with shape {want} for e4m3 {name}")
    a.q_scale, a.kv_scale = _lib.ptr(q_scale), _lib.ptr(kv_scale)
    a.index_dtype = _dtype_or_raise(indices, "indices", (_lib.I32, _lib.I64))
    a.q, a.kv, a.d_out, a.indices, a.dq, a.dkv = (t.data_ptr() for t in (q, kv, d_out, indices, dq, dkv))
    a.batch, a.seq_q, a.heads, a.kv_groups, a.seq_kv, a.topk, a.d_qk, a.d_v = B, S, H, G, Skv, indices.shape[-1], D, int(d_v)
    if isinstance(sm_scale, torch.Tensor):
        _lib.require_device_tensor(sm_scale, "sm_scale", q)
        if sm_scale.dtype != torch.float32 or sm_scale.numel() != 1:
            raise ValueError(f"a device sm_scale must be one float32; got {sm_scale.dtype} {tuple(sm_scale.shape)}")
        a.sm_scale_dev = sm_scale.data_ptr()
    else:
        a.sm_scale = float(sm_scale)
    a.clear_dkv = 1 if clear_dkv else 0
    with torch.cuda.device(q.device):
        rc = _lib.load().cppmega_mi355_sparse_mla_bwd(C.byref(a), C.sizeof(a), _lib.current_stream(q.device))
    _lib.check(rc, "sparse_mla_bwd")
    return dq, dkv


def sparse_mla_scores(
    q: torch.Tensor,
    kv: torch.Tensor,
    indices: torch.Tensor,
    *,
    sm_scale: float,
    scores: torch.Tensor,
    q_spec: QuantSpec | None = None,
    kv_spec: QuantSpec | None = None,
    kv_rope: torch.Tensor | None = None,
) -> torch.Tensor:
    """scores[b,s,h,j] = sm_scale * q . key(indices[b,s,g,j]) into caller-owned float32
    ``scores`` [B,S,H,topk]; skipped slots hold the most negative finite float32."""
    q_spec = q_spec or QuantSpec()
    kv_spec = kv_spec or QuantSpec()
    for name, t in (("q", q), ("kv", kv), ("indices", indices), ("scores", scores), ("kv_rope", kv_rope),
                    ("q_scale", q_spec.scale), ("kv_scale", kv_spec.scale)):
        if t is not None:
            _lib.require_device_tensor(t, name, q if name != "q" else None)
    if q.ndim != 4 or kv.ndim != 4 or indices.ndim != 4:
        raise ValueError("sparse_mla: q, kv and indices must be rank 4")
    B, S, H, _ = q.shape
    want = (B, S, H, indices.shape[-1])
    if tuple(scores.shape) != want or scores.dtype != torch.float32:
        raise ValueError(f"scores must be float32 with shape {want}; got {scores.dtype} {tuple(scores.shape)}")
    d_kv = kv.shape[-1]
    a = _fill_mla_args(q, q_spec, kv, kv_spec, kv_rope, indices, sm_scale, d_kv, None, None, None, "scalar")
    with torch.cuda.device(q.device):
        rc = _lib.load().cppmega_mi355_sparse_mla_scores(C.byref(a), C.sizeof(a), scores.data_ptr(),
                                                         _lib.current_stream(q.device))
    _lib.check(rc, "sparse_mla_scores")
    return scores


def sparse_mla_workspace_bytes(q, kv, indices, *, d_v, q_spec=None, kv_spec=None, kv_rope=None, kernel="auto") -> int:
    a = _fill_mla_args(q, q_spec or QuantSpec(), kv, kv_spec or QuantSpec(), kv_rope, indices, 1.0, d_v, None,
                       None, None, kernel)
    need = C.c_size_t(0)
    _lib.check(_lib.load().cppmega_mi355_sparse_mla_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)),
               "sparse_mla")
    return int(need.value)


def sparse_mla_selected_kernel(q, kv, indices, *, d_v, q_spec=None, kv_spec=None, kv_rope=None, kernel="auto") -> str:
    a = _fill_mla_args(q, q_spec or QuantSpec(), kv, kv_spec or QuantSpec(), kv_rope, indices, 1.0, d_v, None,
                       None, None, kernel)
    rc = _lib.load().cppmega_mi355_sparse_mla_select_kernel(C.byref(a), C.sizeof(a))
    if rc < 0:
        _lib.check(-rc, "sparse_mla_select_kernel")
    return {v: k for k, v in _KERNELS.items()}[rc]


# ---------------------------------------------------------------------------
# FP8 vecmat
# ---------------------------------------------------------------------------

def fp8_vecmat(
    x: torch.Tensor,
    w: torch.Tensor,
    scale_w: torch.Tensor,
    *,
    out: torch.Tensor,
    scale_x: torch.Tensor | None = None,
    scale_w_kind: int,
    workspace: torch.Tensor | None = None,
) -> torch.Tensor:
    """out[m, n] = sum_k dec(w[n,k]) * scale_w(n,k) * x[m,k];  x is [M,K] or [K]."""
    for name, t in (("x", x), ("w", w), ("scale_w", scale_w), ("out", out), ("scale_x", scale_x)):
        if t is not None:
            _lib.require_device_tensor(t, name, w if name != "w" else None)
    if w.ndim != 2:
        raise ValueError(f"W must be 2D [N, K]; got {tuple(w.shape)}")
    n, k = w.shape
    m = 1 if x.ndim == 1 else x.shape[0]
    a = _lib.VecmatArgs()
    a.struct_size = C.sizeof(a)
    a.x_dtype = _dtype_or_raise(x, "x", (_lib.F32, _lib.F16, _lib.BF16, _lib.E4M3))
    a.x = x.data_ptr()
    a.scale_x = _lib.ptr(scale_x)
    a.w = w.data_ptr()
    a.scale_w = scale_w.data_ptr()
    a.scale_w_kind = scale_w_kind
    a.m, a.n, a.k = m, n, k
    a.out_dtype = _dtype_or_raise(out, "out", (_lib.F32, _lib.F16, _lib.BF16))
    a.out = out.data_ptr()
    lib = _lib.load()
    need = C.c_size_t(0)
    _lib.check(lib.cppmega_mi355_fp8_vecmat_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)), "fp8_vecmat")
    stream = _lib.current_stream(w.device)
    if need.value:
        if workspace is None:
            workspace = _workspace(w.device, need.value, stream)
        a.workspace = workspace.data_ptr()
        a.workspace_bytes = workspace.numel() * workspace.element_size()
    with torch.cuda.device(w.device):
        rc = lib.cppmega_mi355_fp8_vecmat(C.byref(a), C.sizeof(a), stream)
    _lib.check(rc, "fp8_vecmat")
    return out


# ---------------------------------------------------------------------------
# FP8 producers
# ---------------------------------------------------------------------------

_QUANT_MODES = {"per_token": _lib.QUANT_PER_TOKEN, "per_tensor": _lib.QUANT_PER_TENSOR, "mxfp8": _lib.QUANT_MXFP8}
_scratch_words: dict[int, torch.Tensor] = {}


def _scratch_word(device: torch.device) -> torch.Tensor:
    key = device.index if device.index is not None else torch.cuda.current_device()
    buf = _scratch_words.get(key)
    if buf is None:
        buf = torch.zeros(1, dtype=torch.int32, device=device)
        _scratch_words[key] = buf
    return buf


def fp8_quantize(x: torch.Tensor, mode: str, *, codes: torch.Tensor | None = None, scale: torch.Tensor | None = None,
                 recovered: torch.Tensor | None = None):
    """Quantise ``x[..., K]`` to e4m3 into caller-owned buffers (any subset of them):
    ``codes`` uint8 like x; ``scale`` float32 ``x.shape[:-1]`` (per_token / per_tensor) or uint8
    ``[..., K/32]`` (mxfp8); ``recovered`` = dec(codes) * scale in x's dtype."""
    if mode not in _QUANT_MODES:
        raise ValueError(f"unknown quantiser mode {mode!r}")
    _lib.require_device_tensor(x, "x", None)
    if not x.is_contiguous():
        raise ValueError("fp8_quantize: x must be contiguous")
    k = int(x.shape[-1])
    rows = x.numel() // k if k else 0
    for name, t, dt, shape in (
        ("codes", codes, torch.uint8, tuple(x.shape)),
        ("scale", scale, torch.uint8 if mode == "mxfp8" else torch.float32,
         tuple(x.shape[:-1]) + (k // 32,) if mode == "mxfp8" else tuple(x.shape[:-1])),
        ("recovered", recovered, x.dtype, tuple(x.shape)),
    ):
        if t is None:
            continue
        _lib.require_device_tensor(t, name, x)
        if t.dtype != dt or tuple(t.shape) != shape or not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous {dt} with shape {shape}; got {t.dtype} {tuple(t.shape)}")
    a = _lib.QuantizeArgs()
    a.struct_size = C.sizeof(a)
    a.x_dtype = _dtype_or_raise(x, "x", (_lib.F32, _lib.F16, _lib.BF16))
    a.x = x.data_ptr()
    a.rows, a.k, a.mode = rows, k, _QUANT_MODES[mode]
    a.codes, a.scale, a.recovered = _lib.ptr(codes), _lib.ptr(scale), _lib.ptr(recovered)
    if mode == "per_tensor":
        a.scratch = _scratch_word(x.device).data_ptr()
    with torch.cuda.device(x.device):
        rc = _lib.load().cppmega_mi355_fp8_quantize(C.byref(a), C.sizeof(a), _lib.current_stream(x.device))
    _lib.check(rc, "fp8_quantize")
    return codes, scale, recovered


def fp8_dequantize(codes: torch.Tensor, scale: torch.Tensor, *, out: torch.Tensor) -> torch.Tensor:
    """out = dec(codes) * scale; ``scale`` float32 ``codes.shape[:-1]`` or E8M0 uint8 ``[..., K/32]``."""
    for name, t in (("codes", codes), ("scale", scale), ("out", out)):
        _lib.require_device_tensor(t, name, codes if name != "codes" else None)
    k = int(codes.shape[-1])
    if codes.dtype != torch.uint8 or tuple(out.shape) != tuple(codes.shape) or not (codes.is_contiguous() and out.is_contiguous()):
        raise ValueError("fp8_dequantize: codes must be contiguous uint8 and out a contiguous tensor of the same shape")
    if scale.dtype == torch.uint8:
        mode, want = _lib.DEQUANT_MXFP8, tuple(codes.shape[:-1]) + (k // 32,)
    elif scale.dtype == torch.float32:
        mode, want = _lib.DEQUANT_PER_TOKEN, tuple(codes.shape[:-1])
    else:
        raise TypeError(f"scale must be float32 (per row) or uint8 (E8M0 per 32); got {scale.dtype}")
    if tuple(scale.shape) != want or not scale.is_contiguous():
        raise ValueError(f"scale must be contiguous with shape {want}; got {tuple(scale.shape)}")
    a = _lib.QuantizeArgs()
    a.struct_size = C.sizeof(a)
    a.x_dtype = _dtype_or_raise(out, "out", (_lib.F32, _lib.F16, _lib.BF16))
    a.rows, a.k, a.mode = (codes.numel() // k if k else 0), k, mode
    a.codes, a.scale, a.recovered = codes.data_ptr(), scale.data_ptr(), out.data_ptr()
    with torch.cuda.device(codes.device):
        rc = _lib.load().cppmega_mi355_fp8_quantize(C.byref(a), C.sizeof(a), _lib.current_stream(codes.device))
    _lib.check(rc, "fp8_dequantize")
    return out


def e4m3_convert(src: torch.Tensor, *, out: torch.Tensor) -> torch.Tensor:
    """The bare e4m3 conversions into a caller-owned buffer of the same shape: float16 / bfloat16 /
    float32 ``src`` -> uint8 codes (round to nearest even, saturating at +-448), or uint8 codes ->
    their float values in ``out``'s dtype."""
    _lib.require_device_tensor(src, "src", None)
    _lib.require_device_tensor(out, "out", src)
    if tuple(src.shape) != tuple(out.shape) or not (src.is_contiguous() and out.is_contiguous()):
        raise ValueError("e4m3_convert: src and out must be contiguous tensors of one shape")
    a = _lib.QuantizeArgs()
    a.struct_size = C.sizeof(a)
    if src.dtype == torch.uint8:
        a.mode, a.x_dtype = _lib.DEQUANT_UNIT, _dtype_or_raise(out, "out", (_lib.F32, _lib.F16, _lib.BF16))
        a.codes, a.recovered = src.data_ptr(), out.data_ptr()
    else:
        if out.dtype != torch.uint8:
            raise TypeError(f"e4m3_convert: codes must be uint8, got {out.dtype}")
        a.mode, a.x_dtype = _lib.QUANT_UNIT, _dtype_or_raise(src, "src", (_lib.F32, _lib.F16, _lib.BF16))
        a.x, a.codes = src.data_ptr(), out.data_ptr()
    a.rows, a.k = src.numel(), 1
    if src.numel():
        with torch.cuda.device(src.device):
            rc = _lib.load().cppmega_mi355_fp8_quantize(C.byref(a), C.sizeof(a), _lib.current_stream(src.device))
        _lib.check(rc, "e4m3_convert")
    return out


def kv_cache_append(src: torch.Tensor, *, kv_cache: torch.Tensor, scale_cache: torch.Tensor, position,
                    src_scale: torch.Tensor | None = None, rope: torch.Tensor | None = None,
                    rope_cache: torch.Tensor | None = None, scale_block: int = 0, pow2_scales: bool = False) -> None:
    """Write ``src[B, S_new, G, D]`` into the preallocated cache at ``position`` (an int, or an
    int32 device tensor ``[B]``).  uint8 ``src`` + float32 ``src_scale`` are copied as prepared
    bytes; a float ``src`` is quantised to e4m3 on the way (one scale per row, or per 128
    channels with ``scale_block=128``).  ``rope[B, S_new, G, R]`` lands in ``rope_cache`` as bf16."""
    _lib.require_device_tensor(src, "src", None)
    for name, t in (("kv_cache", kv_cache), ("scale_cache", scale_cache), ("src_scale", src_scale), ("rope", rope), ("rope_cache", rope_cache)):
        if t is not None:
            _lib.require_device_tensor(t, name, src)
            if not t.is_contiguous():
                raise ValueError(f"{name} must be contiguous")
    if src.ndim != 4 or not src.is_contiguous():
        raise ValueError("src must be contiguous with shape (batch, sequence, kv_heads, head_dim)")
    B, S, G, D = (int(d) for d in src.shape)
    if kv_cache.dtype != torch.uint8 or kv_cache.ndim != 4 or kv_cache.shape[0] != B or kv_cache.shape[2] != G or kv_cache.shape[3] != D:
        raise ValueError(f"kv_cache must be uint8 [B, capacity, G, D] matching src; got {kv_cache.dtype} {tuple(kv_cache.shape)}")
    cap = int(kv_cache.shape[1])
    nsc = D // scale_block if scale_block else 1
    want_scale = (B, cap, G) if not scale_block else (B, cap, G, nsc)
    if scale_cache.dtype != torch.float32 or tuple(scale_cache.shape) != want_scale:
        raise ValueError(f"scale_cache must be float32 {want_scale}; got {scale_cache.dtype} {tuple(scale_cache.shape)}")
    prepared = src.dtype == torch.uint8
    if prepared:
        want = (B, S, G) if not scale_block else (B, S, G, nsc)
        if src_scale is None or src_scale.dtype != torch.float32 or tuple(src_scale.shape) != want:
            raise ValueError(f"prepared bytes need float32 src_scale {want}")
    a = _lib.CacheAppendArgs()
    a.struct_size = C.sizeof(a)
    a.src_dtype = _lib.E4M3 if prepared else _dtype_or_raise(src, "src", (_lib.F32, _lib.F16, _lib.BF16))
    a.src, a.src_scale = src.data_ptr(), _lib.ptr(src_scale)
    a.kv_cache, a.scale_cache = kv_cache.data_ptr(), scale_cache.data_ptr()
    a.scale_block, a.pow2_scales = int(scale_block), int(bool(pow2_scales))
    if rope is not None or rope_cache is not None:
        if rope is None or rope_cache is None:
            raise ValueError("rope and rope_cache go together")
        R = int(rope.shape[-1])
        if tuple(rope.shape) != (B, S, G, R) or rope_cache.dtype != torch.bfloat16 or tuple(rope_cache.shape) != (B, cap, G, R):
            raise ValueError("rope must be [B, S_new, G, R] and rope_cache bfloat16 [B, capacity, G, R]")
        a.rope, a.rope_cache, a.rope_dim = rope.data_ptr(), rope_cache.data_ptr(), R
        a.rope_dtype = _dtype_or_raise(rope, "rope", (_lib.F32, _lib.F16, _lib.BF16))
    if isinstance(position, torch.Tensor):
        _lib.require_device_tensor(position, "position", src)
        if position.dtype != torch.int32 or tuple(position.shape) != (B,) or not position.is_contiguous():
            raise ValueError("position tensor must be contiguous int32 [B]")
        a.positions = position.data_ptr()
    else:
        a.position = int(position)
    a.batch, a.new_tokens, a.groups, a.dim, a.capacity = B, S, G, D, cap
    with torch.cuda.device(src.device):
        rc = _lib.load().cppmega_mi355_kv_cache_append(C.byref(a), C.sizeof(a), _lib.current_stream(src.device))
    _lib.check(rc, "kv_cache_append")


def causal_sparse_indices(out: torch.Tensor, *, query_offset: int = 0, key_length: int) -> torch.Tensor:
    """Fill ``out[B, S, G, topk]`` (int32 / int64) with the causal window ``q_pos - j`` (or -1)."""
    _lib.require_device_tensor(out, "indices", None)
    if out.ndim != 4 or not out.is_contiguous() or out.dtype not in (torch.int32, torch.int64):
        raise ValueError("indices must be a contiguous int32/int64 tensor [B, S, G, topk]")
    a = _lib.CausalIndicesArgs()
    a.struct_size = C.sizeof(a)
    a.index_dtype = _lib.I32 if out.dtype == torch.int32 else _lib.I64
    a.indices = out.data_ptr()
    a.batch, a.seq, a.groups, a.topk = (int(d) for d in out.shape)
    a.query_offset, a.key_length = int(query_offset), int(key_length)
    with torch.cuda.device(out.device):
        rc = _lib.load().cppmega_mi355_causal_sparse_indices(C.byref(a), C.sizeof(a), _lib.current_stream(out.device))
    _lib.check(rc, "causal_sparse_indices")
    return out


_MASK_DTYPES = {torch.bool: _lib.MASK_BOOL, torch.uint8: _lib.MASK_BOOL, torch.float32: _lib.MASK_F32,
                torch.float16: _lib.MASK_F16, torch.bfloat16: _lib.MASK_BF16}


def mask_sparse_indices(mask: torch.Tensor, out: torch.Tensor, *, topk: int) -> torch.Tensor:
    """``mask`` is a 4-D view ``[B or 1, G or 1, S, K]`` with a unit stride along K (broadcast
    dimensions may have stride 0); ``out`` int32 ``[B, S, G, min(topk, K)]``."""
    _lib.require_device_tensor(mask, "mask", None)
    _lib.require_device_tensor(out, "indices", mask)
    if mask.dtype not in _MASK_DTYPES:
        raise TypeError(f"mask dtype {mask.dtype} is not bool/uint8/float32/float16/bfloat16")
    if mask.ndim != 4 or (mask.shape[-1] > 1 and mask.stride(-1) != 1):
        raise ValueError("mask must be 4-D with a unit stride along the key axis")
    B, S, G, n = (int(d) for d in out.shape)
    K = int(mask.shape[-1])
    if out.dtype != torch.int32 or not out.is_contiguous() or n != min(int(topk), K):
        raise ValueError("indices must be contiguous int32 [B, S, G, min(topk, key_length)]")
    a = _lib.MaskIndicesArgs()
    a.struct_size = C.sizeof(a)
    a.mask_dtype = _MASK_DTYPES[mask.dtype]
    a.mask = mask.data_ptr()
    a.stride_b = int(mask.stride(0)) if mask.shape[0] > 1 else 0
    a.stride_g = int(mask.stride(1)) if mask.shape[1] > 1 else 0
    a.stride_s = int(mask.stride(2))
    a.batch, a.seq, a.groups, a.topk, a.key_length = B, S, G, int(topk), K
    a.indices = out.data_ptr()
    with torch.cuda.device(out.device):
        rc = _lib.load().cppmega_mi355_mask_sparse_indices(C.byref(a), C.sizeof(a), _lib.current_stream(out.device))
    _lib.check(rc, "mask_sparse_indices")
    return out
