"""Import alias: the reference's module paths on the MI355X implementation.

A caller of the reference imports its hot path as ``cppmega_mlx.nn._tilelang``,
``cppmega_mlx.nn.sparse_mla``, ``cppmega_mlx.runtime.kernel_policy`` ...
(cppmega_mlx/nn/_tilelang/__init__.py:117-155).  With this directory ahead of
the reference on ``sys.path`` those imports resolve to the modules of
``cppmega_mlx_amd`` of the same relative name - the same module objects, not
copies, so exception classes and caches are shared with code that imports
``cppmega_mlx_amd`` directly.  Tensors are ``torch`` tensors on the GPU where
the reference takes ``mx.array``.
"""

import importlib as _importlib
import pkgutil as _pkgutil
import sys as _sys

import cppmega_mlx_amd as _impl

for _info in _pkgutil.walk_packages(_impl.__path__, _impl.__name__ + "."):
    _leaf = _info.name.rsplit(".", 1)[1]
    if _leaf == "build" or _leaf.startswith("lib"):      # the build recipe and the shared library are not modules to alias
        continue
    _sys.modules[__name__ + _info.name[len(_impl.__name__):]] = _importlib.import_module(_info.name)
for _name in dir(_impl):
    if not _name.startswith("__"):
        globals()[_name] = getattr(_impl, _name)
