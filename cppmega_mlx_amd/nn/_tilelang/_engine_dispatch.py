"""Kernel boundary: ``dispatch_lower`` hands out launchable HIP kernels.

In the reference (``cppmega_mlx/nn/_tilelang/_engine_dispatch.py:242-304``)
``dispatch_lower(prim_func, target, ...)`` turns a TileLang PrimFunc into a
compiled artifact stamped with ``_tilelang_engine_target``, and
``compile_native_tilelang_kernel`` (:127-185) wraps it in
``NativeTileLangKernel`` whose call takes device buffers in PrimFunc parameter
order plus caller-owned ``out=`` buffers and must return those same objects
(``_mlx_runtime.py:147-215``).

Here nothing is compiled at run time: the kernels are prebuilt for gfx950, so
the "PrimFunc" is a :class:`KernelSpec` naming one of them and the artifact is
a :class:`NativeHipKernel` that keeps the same calling convention (parameter
order and ``out_idx`` of the reference kernel it replaces).
"""

from __future__ import annotations

import os
import warnings
from dataclasses import dataclass, field
from typing import Any, Callable, Sequence

import torch

from ... import _lib, ops

__all__ = [
    "KernelSpec",
    "NativeHipKernel",
    "NativeKernelRuntimeError",
    "compile_native_tilelang_kernel",
    "dispatch_lower",
    "normalize_out_idx",
    "tilelang_engine_mode",
]

_VALID_MODES = ("auto", "engine", "shim", "engine_with_msl_extraction")
_FLAG_ENV = "CPPMEGA_MLX_TILELANG_ENGINE"
_VALID_TARGETS = ("hip", "rocm", "gfx950", "hip-gfx950")


class NativeKernelRuntimeError(RuntimeError):
    """Raised when the native kernel boundary is misused."""


def tilelang_engine_mode() -> str:
    """Dispatcher mode from ``$CPPMEGA_MLX_TILELANG_ENGINE`` (unknown -> "auto" with a warning)."""
    raw = os.environ.get(_FLAG_ENV, "auto").strip().lower()
    if raw in _VALID_MODES:
        return raw
    warnings.warn(f"{_FLAG_ENV}={raw!r} is not one of {_VALID_MODES!r}; defaulting to 'auto'.", UserWarning, stacklevel=2)
    return "auto"


def normalize_out_idx(out_idx, *, num_params: int | None = None) -> tuple[int, ...]:
    """Positive, duplicate-free result positions (negative values count from the end)."""
    if out_idx is None:
        return ()
    raw = (out_idx,) if isinstance(out_idx, int) else tuple(int(i) for i in out_idx)
    result = []
    for idx in raw:
        if idx < 0 and num_params is not None:
            idx += num_params
        if num_params is not None and not 0 <= idx < num_params:
            raise NativeKernelRuntimeError(f"out_idx {idx} is outside the kernel parameter range [0, {num_params})")
        result.append(idx)
    if len(set(result)) != len(result):
        raise NativeKernelRuntimeError(f"out_idx contains duplicate result positions: {tuple(result)}")
    return tuple(result)


@dataclass(frozen=True)
class KernelSpec:
    """Names a prebuilt kernel and the parameter order of the reference kernel it replaces.

    ``params`` lists the buffer names in PrimFunc order; ``out_idx`` marks the
    outputs among them; ``attrs`` carries the compile-time constants the
    reference bakes into its PrimFunc (k, sm_scale is a buffer, d_v, ...).
    """

    op: str
    params: tuple[str, ...]
    out_idx: tuple[int, ...]
    attrs: dict = field(default_factory=dict)


def _launch_topk(bufs: dict, attrs: dict):
    ops.topk_select(bufs["scores"], int(attrs["k"]), out=bufs["indices"], starts=bufs.get("starts"),
                    ends=bufs.get("ends"), order=attrs.get("order", "value"))


def _launch_vecmat(bufs: dict, attrs: dict):
    w, sw = bufs["B"], bufs["B_scale"]
    kind = _lib.WSCALE_PER_ROW if sw.numel() == w.shape[0] and sw.numel() != 1 else _lib.WSCALE_SCALAR
    x = bufs["A"].reshape(-1)
    ops.fp8_vecmat(x, w, sw, out=bufs["C"].reshape(-1), scale_x=bufs["A_scale"], scale_w_kind=kind)


def _launch_mla(q_kind: int, kv_kind: int, block: int):
    def run(bufs: dict, attrs: dict):
        B, S, H, G, Skv, topk, K, dv = (int(attrs[n]) for n in ("B", "S", "H", "G", "Skv", "topk", "K", "d_v"))
        q = bufs["q_fp8"].view(B, S, H, K)
        kv = bufs["kv_fp8"].view(B, Skv, G, K)
        idx = bufs["indices"].view(B, S, G, topk)
        nblk = K // block if block else 1
        qs = bufs["q_scale"].view(B, S, H, nblk) if block else bufs["q_scale"].view(B, S, H)
        ks = bufs["kv_scale"].view(B, Skv, G, nblk) if block else bufs["kv_scale"].view(B, Skv, G)
        # sm_scale_buf and has_sinks stay device buffers the kernel reads on the stream, as in the
        # reference: no host read-back, so the launch can be captured into a HIP graph
        ops.sparse_mla_forward(
            q, kv, idx, sm_scale=bufs["sm_scale_buf"], d_v=dv,
            out=bufs["out"].view(B, S, H, dv), lse=bufs["lse"].view(B, S, H),
            q_spec=ops.QuantSpec(q_kind, qs, block), kv_spec=ops.QuantSpec(kv_kind, ks, block),
            sinks=bufs.get("sinks"), has_sinks=bufs.get("has_sinks"))
    return run


def _launch_float_mla(bufs: dict, attrs: dict):
    B, S, H, G, Skv, topk, K, dv = (int(attrs[n]) for n in ("B", "S", "H", "G", "Skv", "topk", "K", "d_v"))
    ops.sparse_mla_forward(
        bufs["q"].view(B, S, H, K), bufs["kv"].view(B, Skv, G, K), bufs["indices"].view(B, S, G, topk),
        sm_scale=bufs["sm_scale_buf"], d_v=dv, out=bufs["out"].view(B, S, H, dv), lse=bufs["lse"].view(B, S, H))


def _launch_float_mla_bwd(bufs: dict, attrs: dict):
    B, S, H, G, Skv, topk, K, dv = (int(attrs[n]) for n in ("B", "S", "H", "G", "Skv", "topk", "K", "d_v"))
    ops.sparse_mla_backward(
        bufs["q"].view(B, S, H, K), bufs["kv"].view(B, Skv, G, K), bufs["d_out"].view(B, S, H, dv),
        bufs["indices"].view(B, S, G, topk), sm_scale=bufs["sm_scale_buf"], d_v=dv,
        dq=bufs["dq"].view(B, S, H, K), dkv=bufs["dkv"].view(B, Skv, G, K), clear_dkv=bool(attrs.get("clear_dkv", True)))


def _launch_latent_mla(bufs: dict, attrs: dict):
    B, S, H, G, Skv, topk, K, R, dv, block = (int(attrs[n]) for n in ("B", "S", "H", "G", "Skv", "topk", "K", "R", "d_v", "scale_block"))
    ops.sparse_mla_forward(
        bufs["q"].view(B, S, H, K + R), bufs["kv_fp8"].view(B, Skv, G, K), bufs["indices"].view(B, S, G, topk),
        sm_scale=bufs["sm_scale_buf"], d_v=dv, out=bufs["out"].view(B, S, H, dv), lse=bufs["lse"].view(B, S, H),
        kv_spec=ops.QuantSpec(_lib.SCALE_F32_BLOCK, bufs["kv_scale"].view(B, Skv, G, K // block), block),
        kv_rope=bufs["kv_rope"].view(B, Skv, G, R), sinks=bufs.get("sinks"), has_sinks=bufs.get("has_sinks"))


_LAUNCHERS: dict[str, Callable[[dict, dict], None]] = {
    "sparse_mla_float": _launch_float_mla,
    "sparse_mla_float_bwd": _launch_float_mla_bwd,
    "sparse_mla_latent": _launch_latent_mla,
    "topk_selector": _launch_topk,
    "fp8_vecmat": _launch_vecmat,
    "sparse_mla_blockscaled": _launch_mla(_lib.SCALE_E8M0, _lib.SCALE_E8M0, 32),
    "sparse_mla_fp8": _launch_mla(_lib.SCALE_PER_TOKEN, _lib.SCALE_PER_TOKEN, 0),
}


def topk_spec(k: int, order: str = "value") -> KernelSpec:
    """kernel(ends, indices, scores, starts), out_idx=1 (topk_selector.py:523-528, 672)."""
    return KernelSpec("topk_selector", ("ends", "indices", "scores", "starts"), (1,), {"k": k, "order": order})


def vecmat_spec() -> KernelSpec:
    """kernel(A[1,K], A_scale[1], B[N,K], B_scale[N or 1], C[1,N]), out_idx=-1 (fp8_vecmat_path_c.py:790-813)."""
    return KernelSpec("fp8_vecmat", ("A", "A_scale", "B", "B_scale", "C"), (4,))


def blockscaled_mla_spec(**shape) -> KernelSpec:
    """kernel(q_fp8,q_scale,kv_fp8,kv_scale,indices,sm_scale_buf,out,lse), out_idx=[6,7]
    (sparse_mla_blockscaled_path_c.py:1054-1064)."""
    return KernelSpec("sparse_mla_blockscaled",
                      ("q_fp8", "q_scale", "kv_fp8", "kv_scale", "indices", "sm_scale_buf", "out", "lse"), (6, 7), shape)


def fp8_mla_spec(**shape) -> KernelSpec:
    """kernel(q_fp8,q_scale,kv_fp8,kv_scale,indices,sm_scale_buf,sinks,has_sinks,out,lse), out_idx=[8,9]
    (sparse_mla_fp8_path_c.py:1821-1835, 2842-2852)."""
    return KernelSpec("sparse_mla_fp8",
                      ("q_fp8", "q_scale", "kv_fp8", "kv_scale", "indices", "sm_scale_buf", "sinks", "has_sinks",
                       "out", "lse"), (8, 9), shape)


def float_mla_spec(**shape) -> KernelSpec:
    """kernel(indices, kv, lse, out, q, sm_scale_buf), out_idx=[2, 3]: the float-carrier forward
    (sparse_mla_fwd_direct, sparse_mla_path_c.py:2291-2299, compiled with out_idx=[2, 3] at :3068 and called
    as kernel(indices, kv, q, sm_scale_buf, out=(lse, out)) at :3282-3288).  Carriers: float16 (the
    reference's), bfloat16 or float32."""
    return KernelSpec("sparse_mla_float", ("indices", "kv", "lse", "out", "q", "sm_scale_buf"), (2, 3), shape)


def float_mla_bwd_spec(**shape) -> KernelSpec:
    """kernel(d_out, dkv, dq, indices, kv, q, sm_scale_buf), out_idx=[1, 2]: the float-carrier backward
    (sparse_mla_bwd_direct, sparse_mla_path_c.py:2670-2678, out_idx=[1, 2] at :3159); dkv is float32 and is
    cleared first unless ``clear_dkv=False`` (the reference clears it with a kernel of its own, :3163-3230)."""
    return KernelSpec("sparse_mla_float_bwd", ("d_out", "dkv", "dq", "indices", "kv", "q", "sm_scale_buf"), (1, 2), shape)


def latent_mla_spec(**shape) -> KernelSpec:
    """kernel(q, kv_fp8, kv_scale, kv_rope, indices, sm_scale_buf, sinks, has_sinks, out, lse), out_idx=[8, 9]: the
    block-scaled forward over a latent cache - bfloat16 q [.., K + R], e4m3 latent [.., K] with one float32 scale
    per ``scale_block`` channels, bfloat16 rope tail [.., R].  The reference has no PrimFunc for this layout; the
    order is that of its per-token FP8 kernel (sparse_mla_fp8_path_c.py:1821-1835) with the rope tail after the
    key scales and no query scale."""
    return KernelSpec("sparse_mla_latent",
                      ("q", "kv_fp8", "kv_scale", "kv_rope", "indices", "sm_scale_buf", "sinks", "has_sinks", "out", "lse"),
                      (8, 9), shape)


class NativeHipKernel:
    """Launchable kernel with the reference's owner-output calling convention.

    ``kernel(*inputs, out=owner_outputs)`` or ``kernel(*all_params)``; outputs
    are written in place and the same objects are returned.
    """

    def __init__(self, spec: KernelSpec, target: str):
        if spec.op not in _LAUNCHERS:
            raise NativeKernelRuntimeError(f"no HIP kernel is registered for op {spec.op!r}")
        self.spec = spec
        self.result_indices = normalize_out_idx(spec.out_idx, num_params=len(spec.params))
        self.num_params = len(spec.params)
        self.target = target
        self._tilelang_engine_target = target
        self._tilelang_execution_backend = "hip_c_abi"

    def __call__(self, *inputs: Any, out: Any | None = None) -> Any:
        n_out = len(self.result_indices)
        n_in = self.num_params - n_out
        if out is None:
            if len(inputs) != self.num_params:
                raise NativeKernelRuntimeError(
                    "native kernels require caller-owned out= buffers: expected "
                    f"{n_in} inputs with out=, or {self.num_params} full-ABI arguments, got {len(inputs)}"
                )
            full = list(inputs)
            owners = tuple(full[i] for i in self.result_indices)
        else:
            if len(inputs) != n_in:
                raise NativeKernelRuntimeError(f"native kernel expected {n_in} inputs with out=, got {len(inputs)}")
            owners = tuple(out) if isinstance(out, (list, tuple)) else (out,)
            if len(owners) != n_out:
                raise NativeKernelRuntimeError(f"kernel expects {n_out} owner outputs, got {len(owners)}")
            full, it_in, it_out = [], iter(inputs), iter(owners)
            for pos in range(self.num_params):
                full.append(next(it_out) if pos in self.result_indices else next(it_in))
        bufs = dict(zip(self.spec.params, full))
        for name, buf in bufs.items():
            if buf is not None and not isinstance(buf, torch.Tensor):
                raise NativeKernelRuntimeError(f"parameter {name!r} must be a torch.Tensor")
        try:
            _LAUNCHERS[self.spec.op](bufs, self.spec.attrs)
        except (ValueError, TypeError):
            raise
        except Exception as exc:  # noqa: BLE001 - keep the original cause
            raise NativeKernelRuntimeError(f"native kernel dispatch failed: {type(exc).__name__}: {exc}") from exc
        if out is None:
            return owners if n_out != 1 else owners[0]
        return out


def compile_native_tilelang_kernel(prim_func: KernelSpec, target: Any, *, out_idx=None, pass_configs=None,
                                   allow_graph_outputs: bool = False) -> NativeHipKernel:
    """Bind ``prim_func`` (a :class:`KernelSpec`) to its prebuilt HIP kernel."""
    del pass_configs, allow_graph_outputs
    if not isinstance(prim_func, KernelSpec):
        raise TypeError("the MI355X boundary takes a KernelSpec in place of a TileLang PrimFunc")
    if out_idx is not None:
        want = normalize_out_idx(out_idx, num_params=len(prim_func.params))
        if want != normalize_out_idx(prim_func.out_idx, num_params=len(prim_func.params)):
            raise NativeKernelRuntimeError(f"out_idx {want} does not match the kernel's outputs {prim_func.out_idx}")
    _lib.load()
    return NativeHipKernel(prim_func, str(target))


def dispatch_lower(prim_func: KernelSpec, target: str, *, return_msl: bool = False, pass_configs=None) -> NativeHipKernel:
    """Return the launchable kernel for ``prim_func`` on ``target`` ("hip"/"gfx950").

    The engine mode variable is honoured as far as it applies: ``shim`` and
    MSL extraction are Metal-text paths with no HIP counterpart and raise.
    """
    mode = tilelang_engine_mode()
    if return_msl or mode in ("shim", "engine_with_msl_extraction"):
        raise NativeKernelRuntimeError("MSL text lowering is a Metal-only path; the MI355X boundary has prebuilt HIP kernels only")
    if str(target) not in _VALID_TARGETS:
        raise NativeKernelRuntimeError(f"target must be one of {_VALID_TARGETS}; got {target!r}")
    return compile_native_tilelang_kernel(prim_func, target, out_idx=None, pass_configs=pass_configs)
