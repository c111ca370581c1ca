"""Kernel cache with the reference's surface: ``cached``, ``clear_cache``, enable / disable.

Reference: tilelang/cache/kernel_cache.py -- process-wide singleton guarded by a lock
(:42-69), key = sha256 over a JSON document of {version, source hash, out_idx,
workspace_idx, args, target, backend, pass_configs} (:71-117), memory cache first (:176-191),
``clear_cache`` empties memory and the on-disk directory (:394-407), ``disable_cache`` bypasses
both (tilelang/cache/__init__.py, tilelang/env.py:191-215).

Here kernels are pre-built into one shared library, so a cache entry is only the Python-side
kernel object; the "source hash" is the fingerprint of the library's sources and flags.  The
on-disk directory (``TLQ_CACHE_DIR``, default ``~/.tilelang_ascend_amd/cache``) holds one small
JSON record per key for inspection; clearing it never touches the in-tree library, which is
what makes the reference examples' import-time ``clear_cache()`` harmless.
"""
from __future__ import annotations

import hashlib
import json
import os
import shutil
import threading
from typing import Callable, Dict

from . import build as _build

_VERSION = "1"
_lock = threading.Lock()
_memory: Dict[str, object] = {}
_enabled = True
_fingerprint = None


def cache_dir() -> str:
    return os.environ.get("TLQ_CACHE_DIR", os.path.join(os.path.expanduser("~"), ".tilelang_ascend_amd", "cache"))


def enable_cache() -> None:
    global _enabled
    _enabled = True


def disable_cache() -> None:
    global _enabled
    _enabled = False


def is_cache_enabled() -> bool:
    return _enabled


def _lib_fingerprint() -> str:
    global _fingerprint
    if _fingerprint is None:
        _fingerprint = _build.source_fingerprint()
    return _fingerprint


def make_key(spec, out_idx, workspace_idx, target, execution_backend, pass_configs) -> str:
    doc = {
        "version": _VERSION,
        "func": hashlib.sha256((_lib_fingerprint() + spec.name).encode()).hexdigest(),
        "params": [[p.name, [str(s) for s in p.shape], p.dtype] for p in spec.params],
        "attrs": {k: str(v) for k, v in sorted(spec.attrs.items())},
        "out_idx": out_idx,
        "workspace_idx": workspace_idx,
        "target": str(target),
        "arch": _build.ARCH,
        "execution_backend": execution_backend,
        "pass_configs": {str(getattr(k, "value", k)): str(v) for k, v in sorted((pass_configs or {}).items(), key=str)},
    }
    return hashlib.sha256(json.dumps(doc, sort_keys=True).encode()).hexdigest()


def cached(key: str, builder: Callable[[], object]):
    """Memory lookup under the lock, build outside it, publish under it (double checked)."""
    if not _enabled:
        return builder()
    with _lock:
        hit = _memory.get(key)
    if hit is not None:
        return hit
    kernel = builder()
    with _lock:
        kernel = _memory.setdefault(key, kernel)
    try:
        d = os.path.join(cache_dir(), key)
        os.makedirs(d, exist_ok=True)
        with open(os.path.join(d, "params.json"), "w") as f:
            json.dump({"name": kernel.spec.name, "library": _build.LIB_PATH, "fingerprint": _lib_fingerprint()}, f)
    except OSError:
        pass  # a read-only home directory must not break kernel creation
    return kernel


def clear_cache() -> None:
    """Empty the in-memory cache and the on-disk record directory (kernel_cache.py:394-407)."""
    with _lock:
        _memory.clear()
    d = cache_dir()
    try:
        shutil.rmtree(d, ignore_errors=True)
        os.makedirs(d, exist_ok=True)
    except OSError:
        pass
