"""Kernel-path policy: which implementation serves an op, and a log of what ran.

Same environment contract as the reference's
``cppmega_mlx/runtime/kernel_policy.py:47-136``: ``CPPMEGA_KERNEL_PATH`` picks
the policy for every op and ``CPPMEGA_KERNEL_PATH__<OP>`` overrides it for one
op; values are case-insensitive (``auto``; ``ref``/``reference``/``path_a``/``a``;
``path_b``/``b``; ``path_c``/``c``) and anything else means AUTO.

On MI355X the paths map to HIP kernels only:

* REFERENCE -- the shape-agnostic fp32 kernel that restates the reference
  arithmetic one wavefront per output row (no matrix cores);
* PATH_C    -- the tuned kernel (MFMA sparse MLA, radix-select top-k, streaming
  GEMV), required to be available;
* PATH_B    -- the reference's retired direct-MSL surface: requests raise;
* AUTO      -- PATH_C where a tuned kernel covers the shape, else REFERENCE.
"""

from __future__ import annotations

import os
import threading
from collections import deque
from enum import Enum

__all__ = ["KernelPath", "clear_dispatch_log", "get_dispatch_log", "record_dispatch", "selected_path"]

_LOG_CAPACITY = 256
_ENV_GLOBAL = "CPPMEGA_KERNEL_PATH"


class KernelPath(Enum):
    AUTO = "auto"
    REFERENCE = "ref"
    PATH_B = "path_b"
    PATH_C = "path_c"


_SPELLINGS = {
    KernelPath.AUTO: ("auto", ""),
    KernelPath.REFERENCE: ("ref", "reference", "path_a", "a"),
    KernelPath.PATH_B: ("path_b", "b"),
    KernelPath.PATH_C: ("path_c", "c"),
}
_BY_SPELLING = {word: path for path, words in _SPELLINGS.items() for word in words}


def _parse(raw: str | None) -> KernelPath:
    if raw is None:
        return KernelPath.AUTO
    return _BY_SPELLING.get(raw.strip().lower(), KernelPath.AUTO)


def selected_path(op_name: str) -> KernelPath:
    """Policy for ``op_name``: the per-op variable wins over the global one."""
    if not isinstance(op_name, str):
        raise TypeError(f"op_name must be str, got {type(op_name).__name__}")
    key = op_name.strip()
    if key:
        override = os.environ.get(f"{_ENV_GLOBAL}__{key.upper()}")
        if override is not None:
            return _parse(override)
    return _parse(os.environ.get(_ENV_GLOBAL))


_log: deque[dict[str, str]] = deque(maxlen=_LOG_CAPACITY)
_log_lock = threading.Lock()


def record_dispatch(op_name: str, path: KernelPath, kernel_used: str) -> None:
    """Remember that ``kernel_used`` served ``op_name`` under ``path`` (bounded, thread-safe)."""
    if not isinstance(op_name, str) or not op_name:
        raise ValueError("op_name must be a non-empty string")
    if not isinstance(path, KernelPath):
        raise TypeError(f"path must be KernelPath, got {type(path).__name__}")
    if not isinstance(kernel_used, str) or not kernel_used:
        raise ValueError("kernel_used must be a non-empty string")
    entry = {"op_name": op_name, "path": path.value, "kernel_used": kernel_used}
    with _log_lock:
        _log.append(entry)


def get_dispatch_log() -> list[dict[str, str]]:
    with _log_lock:
        return [dict(e) for e in _log]


def clear_dispatch_log() -> None:
    with _log_lock:
        _log.clear()
