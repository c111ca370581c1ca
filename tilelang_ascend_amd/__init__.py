"""MI355X (gfx950) implementation of tilelang-ascend's quantized-matmul operators.

Import surface kept from the reference (tilelang/__init__.py:63,88-90):
``jit``, ``compile``, ``PassConfigKey``, ``cache.clear_cache()``, ``enable_cache`` /
``disable_cache``, ``autotune`` / ``AutoTuner``, and the ``quantize`` sub-package; the operators themselves live in
``tilelang_ascend_amd.ops`` under the names the reference's example scripts use.
"""
from . import cache  # noqa: F401
from .cache import disable_cache, enable_cache, is_cache_enabled  # noqa: F401
from .jit import JITKernel, KernelSpec, Param, PassConfigKey, compile, jit  # noqa: F401

__version__ = "0.1.0"

_LAZY = {"autotune": "autotuner", "AutoTuner": "autotuner", "AutotuneResult": "autotuner",
         "set_autotune_inputs": "autotuner", "TensorSupplyType": "profiler"}


def __getattr__(name):
    # sub-packages that import torch-heavy code are loaded on first use
    import importlib

    if name in ("quantize", "ops", "profiler", "autotuner"):
        return importlib.import_module(f".{name}", __name__)
    if name in _LAZY:
        return getattr(importlib.import_module(f".{_LAZY[name]}", __name__), name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
