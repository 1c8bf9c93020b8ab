"""ctypes binding of ``libcppmega_mi355.so`` (the C ABI in ``include/cppmega_mi355.h``).

The library is the only compute path of this package.  If it is missing or a
call fails, the error is raised to the caller; nothing here falls back to
another implementation.
"""

from __future__ import annotations

import ctypes as C
import threading
from pathlib import Path
from typing import Any

import torch

ABI_VERSION = 1
NOALLOC_SCRATCH_BYTES = 20 << 20      # CPPMEGA_MI355_NOALLOC_SCRATCH_BYTES
LIB_NAME = "libcppmega_mi355.so"
LIB_PATH = Path(__file__).resolve().parent / LIB_NAME

# status codes (include/cppmega_mi355.h)
OK, ERR_NULL, ERR_STRUCT_SIZE, ERR_SHAPE, ERR_DTYPE, ERR_UNSUPPORTED, ERR_WORKSPACE, ERR_LAUNCH, ERR_ALIGNMENT = range(9)

# element types
F32, F16, BF16, E4M3, I32, I64 = range(6)
# scale kinds
SCALE_NONE, SCALE_PER_TOKEN, SCALE_E8M0, SCALE_F32_BLOCK = range(4)
# weight-scale layouts
WSCALE_SCALAR, WSCALE_PER_ROW, WSCALE_ROW_BLOCK, WSCALE_GRID_128 = range(4)
# top-k output orders
TOPK_ORDER_INDEX, TOPK_ORDER_VALUE = 0, 1
# sparse-MLA kernels
MLA_KERNEL_AUTO, MLA_KERNEL_SCALAR, MLA_KERNEL_MFMA = 0, 1, 2

EXPORTED_SYMBOLS = (
    "cppmega_mi355_status",
    "cppmega_mi355_error_string",
    "cppmega_mi355_last_error",
    "cppmega_mi355_topk_select",
    "cppmega_mi355_topk_workspace_bytes",
    "cppmega_mi355_indexer_topk_workspace_bytes",
    "cppmega_mi355_indexer_topk",
    "cppmega_mi355_sparse_mla_workspace_bytes",
    "cppmega_mi355_sparse_mla_fwd",
    "cppmega_mi355_sparse_mla_fwd_noalloc",
    "cppmega_mi355_sparse_mla_select_kernel",
    "cppmega_mi355_sparse_mla_scores",
    "cppmega_mi355_fp8_vecmat_workspace_bytes",
    "cppmega_mi355_fp8_vecmat",
    "cppmega_mi355_fp8_quantize",
    "cppmega_mi355_head_gemm",
    "cppmega_mi355_dsa_indexer_loss",
    "cppmega_mi355_sparse_mla_bwd",
    "cppmega_mi355_dequant_block_fp8",
    "cppmega_mi355_kv_cache_append",
    "cppmega_mi355_causal_sparse_indices",
    "cppmega_mi355_mask_sparse_indices",
)


class NativeLibraryError(RuntimeError):
    """The HIP library is missing, stale or unusable."""


class NativeCallError(RuntimeError):
    """A C-ABI call returned a status that is not a shape/dtype contract error."""

    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code


class StatusStruct(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("abi_version", C.c_int32),
        ("device_count", C.c_int32),
        ("gfx950_devices", C.c_int32),
        ("built_for", C.c_char * 32),
        ("message", C.c_char * 160),
    ]


class TopkArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("score_dtype", C.c_int32),
        ("scores", C.c_void_p),
        ("row_stride", C.c_int64),
        ("rows", C.c_int32),
        ("width", C.c_int32),
        ("k", C.c_int32),
        ("order", C.c_int32),
        ("starts", C.c_void_p),
        ("ends", C.c_void_p),
        ("indices", C.c_void_p),
        ("neg_inf_is_masked", C.c_int32),
        ("reserved", C.c_int32),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
    ]


TOPK_ARGS_V1_SIZE = TopkArgs.workspace.offset


class IndexerArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("q_dtype", C.c_int32),
        ("q", C.c_void_p),
        ("weights", C.c_void_p),
        ("k", C.c_void_p),
        ("mask", C.c_void_p),
        ("w_dtype", C.c_int32),
        ("k_dtype", C.c_int32),
        ("mask_dtype", C.c_int32),
        ("order", C.c_int32),
        ("starts", C.c_void_p),
        ("ends", C.c_void_p),
        ("batch", C.c_int32),
        ("seq_q", C.c_int32),
        ("heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("seq_kv", C.c_int32),
        ("topk", C.c_int32),
        ("sm_scale", C.c_float),
        ("chunk_rows", C.c_int32),
        ("indices", C.c_void_p),
        ("scores_out", C.c_void_p),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
    ]


class SparseMlaBwdArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("q_dtype", C.c_int32),
        ("q", C.c_void_p),
        ("kv", C.c_void_p),
        ("d_out", C.c_void_p),
        ("indices", C.c_void_p),
        ("kv_dtype", C.c_int32),
        ("d_out_dtype", C.c_int32),
        ("dq_dtype", C.c_int32),
        ("index_dtype", C.c_int32),
        ("batch", C.c_int32),
        ("seq_q", C.c_int32),
        ("heads", C.c_int32),
        ("kv_groups", C.c_int32),
        ("seq_kv", C.c_int32),
        ("topk", C.c_int32),
        ("d_qk", C.c_int32),
        ("d_v", C.c_int32),
        ("sm_scale", C.c_float),
        ("clear_dkv", C.c_int32),
        ("sm_scale_dev", C.c_void_p),
        ("dq", C.c_void_p),
        ("dkv", C.c_void_p),
        ("q_scale", C.c_void_p),
        ("kv_scale", C.c_void_p),
    ]


class DsaLossArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("in_dtype", C.c_int32),
        ("query", C.c_void_p),
        ("key", C.c_void_p),
        ("index_scores", C.c_void_p),
        ("index_mask", C.c_void_p),
        ("loss", C.c_void_p),
        ("seq_q", C.c_int32),
        ("batch", C.c_int32),
        ("heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("seq_k", C.c_int32),
        ("softmax_scale", C.c_float),
        ("topk_indices", C.c_void_p),
        ("topk", C.c_int32),
        ("index_dtype", C.c_int32),
    ]


class HeadGemmArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("x_dtype", C.c_int32),
        ("x", C.c_void_p),
        ("w", C.c_void_p),
        ("y", C.c_void_p),
        ("w_dtype", C.c_int32),
        ("y_dtype", C.c_int32),
        ("m", C.c_int32),
        ("groups", C.c_int32),
        ("n", C.c_int32),
        ("k", C.c_int32),
        ("x_row_pitch", C.c_int64),
        ("x_group_pitch", C.c_int64),
        ("y_row_pitch", C.c_int64),
        ("y_group_pitch", C.c_int64),
    ]


class DequantBlockArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("out_dtype", C.c_int32),
        ("weight", C.c_void_p),
        ("scale_inv", C.c_void_p),
        ("out", C.c_void_p),
        ("rows", C.c_int32),
        ("cols", C.c_int32),
    ]


class SparseMlaArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("kernel", C.c_int32),
        ("q", C.c_void_p),
        ("q_scale", C.c_void_p),
        ("q_dtype", C.c_int32),
        ("q_scale_kind", C.c_int32),
        ("q_scale_block", C.c_int32),
        ("kv_dtype", C.c_int32),
        ("kv", C.c_void_p),
        ("kv_scale", C.c_void_p),
        ("kv_scale_kind", C.c_int32),
        ("kv_scale_block", C.c_int32),
        ("kv_rope", C.c_void_p),
        ("rope_dtype", C.c_int32),
        ("rope_dim", C.c_int32),
        ("indices", C.c_void_p),
        ("index_dtype", C.c_int32),
        ("batch", C.c_int32),
        ("seq_q", C.c_int32),
        ("heads", C.c_int32),
        ("kv_groups", C.c_int32),
        ("seq_kv", C.c_int32),
        ("topk", C.c_int32),
        ("d_qk", C.c_int32),
        ("d_v", C.c_int32),
        ("sm_scale", C.c_float),
        ("sinks", C.c_void_p),
        ("out", C.c_void_p),
        ("lse", C.c_void_p),
        ("out_dtype", C.c_int32),
        ("reserved", C.c_int32),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
        ("sm_scale_dev", C.c_void_p),
        ("has_sinks_dev", C.c_void_p),
        ("seq_kv_pitch", C.c_int32),
        ("reserved2", C.c_int32),
    ]


# struct_size of the first ABI of SparseMlaArgs (through workspace_bytes): still accepted by the library
SPARSE_MLA_ARGS_V1_SIZE = SparseMlaArgs.sm_scale_dev.offset


class VecmatArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("x_dtype", C.c_int32),
        ("x", C.c_void_p),
        ("scale_x", C.c_void_p),
        ("w", C.c_void_p),
        ("scale_w", C.c_void_p),
        ("scale_w_kind", C.c_int32),
        ("m", C.c_int32),
        ("n", C.c_int32),
        ("k", C.c_int32),
        ("out_dtype", C.c_int32),
        ("reserved", C.c_int32),
        ("out", C.c_void_p),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
    ]


class QuantizeArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("x_dtype", C.c_int32),
        ("x", C.c_void_p),
        ("rows", C.c_int64),
        ("k", C.c_int32),
        ("mode", C.c_int32),
        ("codes", C.c_void_p),
        ("scale", C.c_void_p),
        ("recovered", C.c_void_p),
        ("scratch", C.c_void_p),
    ]


QUANT_PER_TOKEN, QUANT_PER_TENSOR, QUANT_MXFP8, DEQUANT_PER_TOKEN, DEQUANT_MXFP8, QUANT_UNIT, DEQUANT_UNIT = range(7)


class CacheAppendArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("src_dtype", C.c_int32),
        ("src", C.c_void_p),
        ("src_scale", C.c_void_p),
        ("rope", C.c_void_p),
        ("rope_dtype", C.c_int32),
        ("scale_block", C.c_int32),
        ("kv_cache", C.c_void_p),
        ("scale_cache", C.c_void_p),
        ("rope_cache", C.c_void_p),
        ("positions", C.c_void_p),
        ("position", C.c_int32),
        ("batch", C.c_int32),
        ("new_tokens", C.c_int32),
        ("groups", C.c_int32),
        ("dim", C.c_int32),
        ("rope_dim", C.c_int32),
        ("capacity", C.c_int32),
        ("pow2_scales", C.c_int32),
        ("reserved", C.c_int32),
    ]


class CausalIndicesArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("index_dtype", C.c_int32),
        ("indices", C.c_void_p),
        ("batch", C.c_int32),
        ("seq", C.c_int32),
        ("groups", C.c_int32),
        ("topk", C.c_int32),
        ("query_offset", C.c_int64),
        ("key_length", C.c_int64),
    ]


MASK_BOOL, MASK_F32, MASK_F16, MASK_BF16 = range(4)


class MaskIndicesArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("mask_dtype", C.c_int32),
        ("mask", C.c_void_p),
        ("stride_b", C.c_int64),
        ("stride_g", C.c_int64),
        ("stride_s", C.c_int64),
        ("batch", C.c_int32),
        ("seq", C.c_int32),
        ("groups", C.c_int32),
        ("topk", C.c_int32),
        ("key_length", C.c_int32),
        ("reserved", C.c_int32),
        ("indices", C.c_void_p),
    ]

_lock = threading.RLock()
_lib: C.CDLL | None = None


def library_path() -> Path:
    return LIB_PATH


def load() -> C.CDLL:
    """Load the shared library once (thread-safe) and declare its prototypes."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise NativeLibraryError(
                f"{LIB_PATH} is missing: build it with `python -m cppmega_mlx_amd.build` "
                "(hipcc --offload-arch=gfx950). There is no fallback path."
            )
        try:
            lib = C.CDLL(str(LIB_PATH))
        except OSError as exc:
            raise NativeLibraryError(f"cannot load {LIB_PATH}: {exc}") from exc
        missing = [name for name in EXPORTED_SYMBOLS if not hasattr(lib, name)]
        if missing:
            raise NativeLibraryError(f"{LIB_PATH} does not export {missing}; rebuild it")
        lib.cppmega_mi355_status.argtypes = [C.POINTER(StatusStruct), C.c_size_t]
        lib.cppmega_mi355_status.restype = C.c_int
        lib.cppmega_mi355_error_string.argtypes = [C.c_int]
        lib.cppmega_mi355_error_string.restype = C.c_char_p
        lib.cppmega_mi355_last_error.argtypes = []
        lib.cppmega_mi355_last_error.restype = C.c_char_p
        lib.cppmega_mi355_topk_select.argtypes = [C.POINTER(TopkArgs), C.c_size_t, C.c_void_p]
        lib.cppmega_mi355_topk_select.restype = C.c_int
        lib.cppmega_mi355_topk_workspace_bytes.argtypes = [C.POINTER(TopkArgs), C.c_size_t, C.POINTER(C.c_size_t)]
        lib.cppmega_mi355_topk_workspace_bytes.restype = C.c_int
        lib.cppmega_mi355_indexer_topk.argtypes = [C.POINTER(IndexerArgs), C.c_size_t, C.c_void_p]
        lib.cppmega_mi355_indexer_topk.restype = C.c_int
        lib.cppmega_mi355_indexer_topk_workspace_bytes.argtypes = [C.POINTER(IndexerArgs), C.c_size_t, C.POINTER(C.c_size_t)]
        lib.cppmega_mi355_indexer_topk_workspace_bytes.restype = C.c_int
        for name in ("cppmega_mi355_sparse_mla_fwd", "cppmega_mi355_sparse_mla_fwd_noalloc"):
            getattr(lib, name).argtypes = [C.POINTER(SparseMlaArgs), C.c_size_t, C.c_void_p]
            getattr(lib, name).restype = C.c_int
        lib.cppmega_mi355_sparse_mla_workspace_bytes.argtypes = [
            C.POINTER(SparseMlaArgs), C.c_size_t, C.POINTER(C.c_size_t)]
        lib.cppmega_mi355_sparse_mla_workspace_bytes.restype = C.c_int
        lib.cppmega_mi355_sparse_mla_select_kernel.argtypes = [C.POINTER(SparseMlaArgs), C.c_size_t]
        lib.cppmega_mi355_sparse_mla_select_kernel.restype = C.c_int
        lib.cppmega_mi355_sparse_mla_scores.argtypes = [C.POINTER(SparseMlaArgs), C.c_size_t, C.c_void_p, C.c_void_p]
        lib.cppmega_mi355_sparse_mla_scores.restype = C.c_int
        lib.cppmega_mi355_fp8_vecmat.argtypes = [C.POINTER(VecmatArgs), C.c_size_t, C.c_void_p]
        lib.cppmega_mi355_fp8_vecmat.restype = C.c_int
        lib.cppmega_mi355_fp8_quantize.argtypes = [C.POINTER(QuantizeArgs), C.c_size_t, C.c_void_p]
        lib.cppmega_mi355_fp8_quantize.restype = C.c_int
        lib.cppmega_mi355_sparse_mla_bwd.argtypes = [C.POINTER(SparseMlaBwdArgs), C.c_size_t, C.c_void_p]
        lib.cppmega_mi355_sparse_mla_bwd.restype = C.c_int
        lib.cppmega_mi355_dsa_indexer_loss.argtypes = [C.POINTER(DsaLossArgs), C.c_size_t, C.c_void_p]
        lib.cppmega_mi355_dsa_indexer_loss.restype = C.c_int
        lib.cppmega_mi355_head_gemm.argtypes = [C.POINTER(HeadGemmArgs), C.c_size_t, C.c_void_p]
        lib.cppmega_mi355_head_gemm.restype = C.c_int
        lib.cppmega_mi355_dequant_block_fp8.argtypes = [C.POINTER(DequantBlockArgs), C.c_size_t, C.c_void_p]
        lib.cppmega_mi355_dequant_block_fp8.restype = C.c_int
        for fn, struct in ((lib.cppmega_mi355_kv_cache_append, CacheAppendArgs),
                           (lib.cppmega_mi355_causal_sparse_indices, CausalIndicesArgs),
                           (lib.cppmega_mi355_mask_sparse_indices, MaskIndicesArgs)):
            fn.argtypes = [C.POINTER(struct), C.c_size_t, C.c_void_p]
            fn.restype = C.c_int
        lib.cppmega_mi355_fp8_vecmat_workspace_bytes.argtypes = [
            C.POINTER(VecmatArgs), C.c_size_t, C.POINTER(C.c_size_t)]
        lib.cppmega_mi355_fp8_vecmat_workspace_bytes.restype = C.c_int
        _lib = lib
        return lib


_status_cache: dict[str, Any] | None = None


def status(refresh: bool = False) -> dict[str, Any]:
    """Probe the library (and the HIP runtime under it); the answer is cached."""
    global _status_cache
    if _status_cache is not None and not refresh:
        return dict(_status_cache)
    lib = load()
    st = StatusStruct()
    rc = lib.cppmega_mi355_status(C.byref(st), C.sizeof(st))
    if rc != OK:
        raise NativeLibraryError(f"cppmega_mi355_status returned {rc}")
    if st.abi_version != ABI_VERSION:
        raise NativeLibraryError(f"ABI version {st.abi_version} != expected {ABI_VERSION}; rebuild the library")
    _status_cache = {
        "abi_version": st.abi_version,
        "device_count": st.device_count,
        "gfx950_devices": st.gfx950_devices,
        "built_for": st.built_for.decode(),
        "message": st.message.decode(),
    }
    return dict(_status_cache)


def check(rc: int, op: str) -> None:
    """Map a status code to the reference's error classes: shape -> ValueError,
    dtype -> TypeError, everything else -> NativeCallError (a RuntimeError)."""
    if rc == OK:
        return
    lib = load()
    detail = lib.cppmega_mi355_last_error().decode(errors="replace")
    text = f"{op}: {detail or lib.cppmega_mi355_error_string(rc).decode()}"
    if rc == ERR_SHAPE:
        raise ValueError(text)
    if rc == ERR_DTYPE:
        raise TypeError(text)
    raise NativeCallError(rc, f"{text} (status {rc})")


_TORCH_DTYPE_CODES = {
    torch.float32: F32,
    torch.float16: F16,
    torch.bfloat16: BF16,
    torch.uint8: E4M3,
    torch.float8_e4m3fn: E4M3,
    torch.int32: I32,
    torch.int64: I64,
}


def dtype_code(t: torch.Tensor) -> int | None:
    return _TORCH_DTYPE_CODES.get(t.dtype)


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def batch_pitch(t: torch.Tensor) -> int | None:
    """Rows of dim 1 between two batches of ``t`` when everything but the batch stride is dense
    (a ``cache[:, :n]`` view of a dense buffer), else None."""
    if t.ndim < 2:
        return None
    inner = 1
    for size, stride in zip(reversed(t.shape[1:]), reversed(t.stride()[1:])):
        if size != 1 and stride != inner:
            return None
        inner *= size
    row = inner // max(t.shape[1], 1) if t.shape[1] else 0
    if t.shape[0] <= 1 or t.shape[1] == 0:
        return t.shape[1]
    if row == 0 or t.stride(0) % row != 0 or t.stride(0) < inner:
        return None
    return t.stride(0) // row


def require_device_tensor(t: torch.Tensor, name: str, ref: torch.Tensor | None = None, *,
                          allow_batch_pitch: bool = False) -> None:
    """Inputs must be dense device tensors; the boundary never copies or casts.  With
    ``allow_batch_pitch`` the batch stride alone may exceed the dense one."""
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor; got {type(t).__name__}")
    if not t.is_cuda:
        raise NativeCallError(
            ERR_UNSUPPORTED,
            f"{name} lives on {t.device}; the MI355X kernels take device tensors only and there is no CPU path",
        )
    if allow_batch_pitch and batch_pitch(t) is not None:
        pass
    elif not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous (the boundary does not copy); got strides {t.stride()}")
    if ref is not None and t.device != ref.device:
        raise ValueError(f"{name} is on {t.device} but other operands are on {ref.device}")


def current_stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream
