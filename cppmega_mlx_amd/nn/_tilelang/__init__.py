"""Kernel-facing operator modules (names follow ``cppmega_mlx.nn._tilelang``).

Exports the hot-path names of the reference's
``cppmega_mlx/nn/_tilelang/__init__.py:117-155``.
"""

from ._engine_dispatch import dispatch_lower, tilelang_engine_mode
from .dsa_splitk_indexer_loss import dsa_splitk_indexer_loss_tilelang, dsa_splitk_path_c_status
from .fp8_msl_kernels import fp8_scaled_vecmat
from .fp8_vecmat_path_c import (
    FP8VecmatPathCDirectError,
    FP8VecmatPathCLegacyError,
    fp8_scaled_vecmat_path_c,
    fp8_scaled_vecmat_path_c_direct,
    fp8_vecmat_path_c_status,
)
from .fused_fp8_gemm import fused_fp8_gemm
from .sparse_mla import sparse_mla_apply
from .sparse_mla_blockscaled import sparse_mla_blockscaled_apply, sparse_mla_blockscaled_reference
from .sparse_mla_fp8 import sparse_mla_fp8_apply, sparse_mla_fp8_reference
from .sparse_mla_blockscaled_path_c import (
    sparse_mla_blockscaled_path_c_apply,
    sparse_mla_blockscaled_path_c_apply_direct,
)
from .sparse_mla_fp8_path_c import sparse_mla_fp8_path_c_apply, sparse_mla_fp8_path_c_apply_direct
from .sparse_mla_path_c import sparse_mla_fwd_path_c, sparse_mla_path_c_apply
from .topk_selector import (
    topk_selector as topk_selector_fn,
    topk_selector_reference,
    topk_selector_tilelang,
    topk_selector_tilelang_direct,
)

__all__ = [
    "FP8VecmatPathCDirectError",
    "FP8VecmatPathCLegacyError",
    "dispatch_lower",
    "dsa_splitk_indexer_loss_tilelang",
    "dsa_splitk_path_c_status",
    "fp8_scaled_vecmat",
    "fp8_scaled_vecmat_path_c",
    "fp8_scaled_vecmat_path_c_direct",
    "fp8_vecmat_path_c_status",
    "fused_fp8_gemm",
    "sparse_mla_apply",
    "sparse_mla_blockscaled_apply",
    "sparse_mla_blockscaled_reference",
    "sparse_mla_fp8_apply",
    "sparse_mla_fp8_reference",
    "sparse_mla_blockscaled_path_c_apply",
    "sparse_mla_blockscaled_path_c_apply_direct",
    "sparse_mla_fp8_path_c_apply",
    "sparse_mla_fp8_path_c_apply_direct",
    "sparse_mla_fwd_path_c",
    "sparse_mla_path_c_apply",
    "tilelang_engine_mode",
    "topk_selector_fn",
    "topk_selector_reference",
    "topk_selector_tilelang",
    "topk_selector_tilelang_direct",
]
