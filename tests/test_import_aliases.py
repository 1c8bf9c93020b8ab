"""The reference's import paths resolve to the MI355X modules (no GPU needed: nothing is launched)."""


def test_reference_import_paths_resolve_to_the_same_modules():
    import cppmega_mlx_amd.nn._tilelang as impl
    from cppmega_mlx.nn._tilelang import dispatch_lower, topk_selector_fn, fp8_scaled_vecmat_path_c, sparse_mla_blockscaled_path_c_apply
    assert dispatch_lower is impl.dispatch_lower and topk_selector_fn is impl.topk_selector_fn
    assert fp8_scaled_vecmat_path_c is impl.fp8_scaled_vecmat_path_c
    assert sparse_mla_blockscaled_path_c_apply is impl.sparse_mla_blockscaled_path_c_apply
    import cppmega_mlx.nn.sparse_mla as a
    import cppmega_mlx_amd.nn.sparse_mla as b
    assert a is b
    from cppmega_mlx.nn._tilelang.fp8_msl_kernels import fp8_to_half, half_to_fp8  # noqa: F401
    from cppmega_mlx.runtime.kernel_policy import KernelPath
    from cppmega_mlx_amd.runtime.kernel_policy import KernelPath as K2
    assert KernelPath is K2
    from cppmega_mlx.inference.engine import SparseFP8KVCache  # noqa: F401


def test_v4_import_paths():
    from cppmega_v4.nn.lightning_indexer import LightningIndexer
    from cppmega_v4.nn.lightning_indexer_fp8 import LightningIndexerFP8
    from cppmega_v4.nn.mla_absorb import absorbed_mla_decode
    from cppmega_v4._tilelang.fused_fp8_gemm import fused_fp8_gemm
    import cppmega_mlx_amd.nn.lightning_indexer as li
    import cppmega_mlx_amd.nn.mla_absorb as ma
    assert LightningIndexer is li.LightningIndexer and LightningIndexerFP8 is li.LightningIndexerFP8
    assert absorbed_mla_decode is ma.absorbed_mla_decode and callable(fused_fp8_gemm)
