"""MI355X-native sparse-attention inference hot path (top-k selector, sparse MLA
forward over an FP8 block-scaled latent KV cache, FP8 block-scaled vecmat).

The sub-packages mirror the module paths of the reference package so that its
callers can switch by changing the top-level package name:

    cppmega_mlx_amd.nn.sparse_mla
    cppmega_mlx_amd.nn._tilelang.{topk_selector, sparse_mla, sparse_mla_path_c,
        sparse_mla_blockscaled, sparse_mla_blockscaled_path_c, sparse_mla_fp8,
        sparse_mla_fp8_path_c, fp8_msl_kernels, fp8_vecmat_path_c,
        fused_fp8_gemm, _engine_dispatch}
    cppmega_mlx_amd.runtime.kernel_policy

All compute runs in hand-written HIP kernels for gfx950 behind the C ABI in
``include/cppmega_mi355.h``; ``torch`` supplies device memory and streams.
"""

from . import _lib

__all__ = ["_lib", "native_status"]


def native_status() -> dict:
    """Probe the HIP library; raises if it is missing or stale."""
    return _lib.status()
