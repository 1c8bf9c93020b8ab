"""Import alias for the reference's ``cppmega_v4`` modules that lie on the hot path:
``cppmega_v4.nn.lightning_indexer`` (and ``lightning_indexer_fp8``), ``cppmega_v4.nn.mla_absorb``
and ``cppmega_v4._tilelang.fused_fp8_gemm`` resolve to the modules of ``cppmega_mlx_amd`` that
implement them (same module objects)."""

import importlib as _importlib
import sys as _sys
import types as _types

_MAP = {
    "nn.lightning_indexer": "cppmega_mlx_amd.nn.lightning_indexer",
    "nn.lightning_indexer_fp8": "cppmega_mlx_amd.nn.lightning_indexer",
    "nn.mla_absorb": "cppmega_mlx_amd.nn.mla_absorb",
    "_tilelang.fused_fp8_gemm": "cppmega_mlx_amd.nn._tilelang.fused_fp8_gemm",
}
for _pkg in ("nn", "_tilelang"):
    _mod = _types.ModuleType(__name__ + "." + _pkg)
    _mod.__path__ = []
    _sys.modules[_mod.__name__] = _mod
    globals()[_pkg] = _mod
for _alias, _real in _MAP.items():
    _module = _importlib.import_module(_real)
    _sys.modules[__name__ + "." + _alias] = _module
    _parent, _leaf = _alias.split(".")
    setattr(_sys.modules[__name__ + "." + _parent], _leaf, _module)
