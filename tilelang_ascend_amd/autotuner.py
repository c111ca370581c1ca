"""Autotuner over the pre-built kernel variants, with the reference's surface.

Reference: tilelang/autotuner/tuner.py -- ``AutoTuner.from_kernel(kernel, configs)
.set_compile_args(...).set_profile_args(...).run()`` (:102-595), the ``@autotune(configs=...)``
decorator stacked on ``@jit`` (:675-760; tuning is skipped when the caller passes every tunable
parameter, :441-480), ``AutotuneResult`` with ``latency / config / ref_latency / kernel``
(tilelang/autotuner/param.py:128-145), a memory cache per call signature (:656-673) and a disk
cache under ``<cache dir>/autotuner`` keyed by a hash of function, arguments and configs
(:240-281).  Example: examples/autotune/example_gemm_autotune.py.

The reference compiles one kernel per configuration; here every configuration selects one of the
kernels already built into the library (the factories' ``tile`` / ``algo`` / ``*_tuning``
arguments), so "compiling" a configuration is just creating the kernel object.  A configuration
the library rejects for the given shape (its host-side checks raise) or whose output fails the
check against ``ref_prog`` is skipped and recorded with its error.
"""
from __future__ import annotations

import hashlib
import inspect
import json
import logging
import os
import threading
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple, Union

import torch

from . import cache as _cache
from .profiler import Profiler, TensorSupplyType, do_bench

logger = logging.getLogger(__name__)


@dataclass
class AutotuneResult:
    """tilelang/autotuner/param.py:128-145."""

    latency: Optional[float] = None        # ms of the best configuration
    config: Optional[dict] = None
    ref_latency: Optional[float] = None    # ms of ref_prog on the same inputs, when one was given
    kernel: Any = None
    trials: List[Tuple[dict, Optional[float], Optional[str]]] = field(default_factory=list)  # (config, ms, error)

    def to_json(self) -> dict:
        return {"latency": self.latency, "config": self.config, "ref_latency": self.ref_latency,
                "trials": [[c, t, e] for c, t, e in self.trials]}


@dataclass
class _CompileArgs:
    out_idx: Any = None
    target: str = "auto"
    execution_backend: str = "ctypes"
    target_host: Any = None
    verbose: bool = False
    pass_configs: Optional[dict] = None


@dataclass
class _ProfileArgs:
    warmup: int = 25
    rep: int = 100
    timeout: int = 30
    supply_type: TensorSupplyType = TensorSupplyType.Auto
    ref_prog: Optional[Callable] = None
    supply_prog: Optional[Callable] = None
    rtol: float = 1e-2
    atol: float = 1e-2
    max_mismatched_ratio: float = 0.01
    skip_check: bool = False
    manual_check_prog: Optional[Callable] = None
    cache_input_tensors: bool = False


_autotune_inputs = threading.local()


class set_autotune_inputs:
    """``with set_autotune_inputs(a, b): kernel = factory(...)`` -- tune on the caller's tensors
    instead of generated ones (tilelang/autotuner/capture.py)."""

    def __init__(self, *tensors):
        self.tensors = list(tensors[0]) if len(tensors) == 1 and isinstance(tensors[0], (list, tuple)) else list(tensors)

    def __enter__(self):
        self._prev = getattr(_autotune_inputs, "value", None)
        _autotune_inputs.value = self.tensors
        return self

    def __exit__(self, *exc):
        _autotune_inputs.value = self._prev
        return False


def get_autotune_inputs():
    return getattr(_autotune_inputs, "value", None)


def _normalize(value):
    if isinstance(value, (list, tuple)):
        return [_normalize(v) for v in value]
    if isinstance(value, dict):
        return {str(k): _normalize(v) for k, v in sorted(value.items(), key=lambda kv: str(kv[0]))}
    if isinstance(value, (int, float, str, bool)) or value is None:
        return value
    return str(value)


class AutoTuner:
    """Times ``fn(**config)`` for every configuration and keeps the fastest valid kernel."""

    _memory_cache: Dict[str, AutotuneResult] = {}
    _lock = threading.Lock()

    def __init__(self, fn: Callable, configs: Union[Sequence[dict], Callable]):
        self.fn = fn
        self.configs = configs
        self.compile_args = _CompileArgs()
        self.profile_args = _ProfileArgs()
        self.jit_compile: Optional[Callable] = None
        self._kernel_parameters = None
        self._function_parameters = None

    @classmethod
    def from_kernel(cls, kernel: Callable, configs):
        return cls(kernel, configs)

    @staticmethod
    def cache_dir() -> str:
        return os.path.join(_cache.cache_dir(), "autotuner")

    def set_compile_args(self, out_idx=None, target="auto", execution_backend="ctypes", target_host=None,
                         verbose: bool = False, pass_configs: Optional[dict] = None):
        self.compile_args = _CompileArgs(out_idx, target, execution_backend, target_host, verbose, pass_configs)
        return self

    def set_profile_args(self, warmup: int = 25, rep: int = 100, timeout: int = 30,
                         supply_type: TensorSupplyType = TensorSupplyType.Auto, ref_prog: Optional[Callable] = None,
                         supply_prog: Optional[Callable] = None, rtol: float = 1e-2, atol: float = 1e-2,
                         max_mismatched_ratio: float = 0.01, skip_check: bool = False,
                         manual_check_prog: Optional[Callable] = None, cache_input_tensors: bool = False):
        if get_autotune_inputs() is not None:
            if supply_prog is not None:
                logger.warning("`supply_prog` is ignored inside `with set_autotune_inputs(...)`")
            captured = get_autotune_inputs()
            supply_prog = lambda _params: captured  # noqa: E731
        self.profile_args = _ProfileArgs(warmup, rep, timeout, supply_type, ref_prog, supply_prog, rtol, atol,
                                         max_mismatched_ratio, skip_check, manual_check_prog, cache_input_tensors)
        return self

    def set_kernel_parameters(self, k_parameters, f_parameters):
        self._kernel_parameters = k_parameters
        self._function_parameters = f_parameters

    def generate_cache_key(self, configs: Sequence[dict]) -> str:
        fn = getattr(self.fn, "__wrapped_factory__", self.fn)
        doc = {
            "library": _cache._lib_fingerprint(),
            "func": f"{getattr(fn, '__module__', '')}.{getattr(fn, '__qualname__', repr(fn))}",
            "args": _normalize(self._kernel_parameters),
            "configs": _normalize(list(configs)),
            "device": torch.cuda.get_device_name() if torch.cuda.is_available() else "none",
            "profile": [self.profile_args.rtol, self.profile_args.atol, self.profile_args.skip_check],
        }
        return hashlib.sha256(json.dumps(doc, sort_keys=True).encode()).hexdigest()

    # -- disk cache ---------------------------------------------------------------------------
    def _save_result_to_disk(self, key: str, result: AutotuneResult) -> None:
        try:
            os.makedirs(self.cache_dir(), exist_ok=True)
            tmp = os.path.join(self.cache_dir(), f"{key}.json.tmp{os.getpid()}")
            with open(tmp, "w") as f:
                json.dump(result.to_json(), f)
            os.replace(tmp, os.path.join(self.cache_dir(), f"{key}.json"))
        except OSError:
            pass

    def _load_result_from_disk(self, key: str) -> Optional[AutotuneResult]:
        try:
            with open(os.path.join(self.cache_dir(), f"{key}.json")) as f:
                doc = json.load(f)
        except (OSError, ValueError):
            return None
        if not isinstance(doc.get("config"), dict):
            return None
        return AutotuneResult(latency=doc.get("latency"), config=doc["config"], ref_latency=doc.get("ref_latency"),
                              trials=[tuple(t) for t in doc.get("trials", [])])

    # -- the search ---------------------------------------------------------------------------
    def _compile(self, config: dict):
        return self.jit_compile(**config) if self.jit_compile is not None else self.fn(**config)

    def _inputs(self, kernel) -> List[torch.Tensor]:
        pa = self.profile_args
        if pa.supply_prog is not None:
            return list(pa.supply_prog(Profiler(kernel)._get_params()))
        return Profiler(kernel, pa.supply_type)._get_inputs()

    def run(self, warmup: int = 25, rep: int = 100, timeout: int = 30) -> AutotuneResult:
        configs = self.configs() if callable(self.configs) else self.configs
        configs = [dict(c) for c in configs]
        if not configs:
            raise ValueError("autotune needs at least one configuration")
        key = self.generate_cache_key(configs)
        if _cache.is_cache_enabled():
            with self._lock:
                hit = self._memory_cache.get(key)
            if hit is None:
                hit = self._load_result_from_disk(key)
            if hit is not None:
                if hit.kernel is None:
                    hit.kernel = self._compile(hit.config)
                with self._lock:
                    self._memory_cache[key] = hit
                return hit

        pa = self.profile_args
        result = AutotuneResult()
        inputs = None
        for config in configs:
            try:
                kernel = self._compile(config)
                if inputs is None:  # every configuration is timed on the same tensors
                    inputs = self._inputs(kernel)
                profiler = Profiler(kernel, pa.supply_type)
                if not pa.skip_check:
                    if pa.manual_check_prog is not None:
                        pa.manual_check_prog(kernel(*inputs), *inputs)
                    elif pa.ref_prog is not None:
                        profiler.assert_allclose(pa.ref_prog, input_tensors=inputs, atol=pa.atol, rtol=pa.rtol,
                                                 max_mismatched_ratio=pa.max_mismatched_ratio)
                    else:
                        kernel(*inputs)  # a launch error still disqualifies the configuration
                        torch.cuda.synchronize()
                ms = do_bench(lambda: kernel(*inputs), warmup=warmup, rep=rep)  # noqa: B023
            except Exception as e:  # noqa: BLE001 -- one bad configuration must not end the search
                result.trials.append((config, None, f"{type(e).__name__}: {e}"))
                logger.debug("autotune: config %s skipped: %s", config, e)
                continue
            result.trials.append((config, ms, None))
            if result.latency is None or ms < result.latency:
                result.latency, result.config, result.kernel = ms, config, kernel
        if result.config is None:
            errors = "; ".join(f"{c}: {e}" for c, _, e in result.trials)
            raise RuntimeError(f"autotune: no configuration produced a valid kernel ({errors})")
        if pa.ref_prog is not None:
            try:
                result.ref_latency = do_bench(lambda: pa.ref_prog(*inputs), warmup=warmup, rep=rep)
            except Exception:  # noqa: BLE001 -- a CPU-only reference program cannot be timed on device tensors
                result.ref_latency = None
        with self._lock:
            self._memory_cache[key] = result
        if _cache.is_cache_enabled():
            self._save_result_to_disk(key, result)
        return result

    def __call__(self) -> AutotuneResult:
        return self.run()


class AutoTuneImpl:
    """What ``@autotune(...)`` returns: a factory with the decorated one's signature whose tunable
    parameters may be left out (tuner.py:611-673)."""

    def __init__(self, factory: Callable, **opts):
        self.factory = factory
        self.opts = opts
        self._tuner_cache: Dict[tuple, Any] = {}
        self.__wrapped_factory__ = getattr(factory, "__wrapped_factory__", factory)
        self.__name__ = getattr(self.__wrapped_factory__, "__name__", "autotuned")
        self.__doc__ = getattr(self.__wrapped_factory__, "__doc__", None)

    def _configs(self, args, kwargs) -> List[dict]:
        configs = self.opts["configs"]
        if callable(configs):
            configs = configs(*args, **kwargs)
        return [dict(c) for c in configs]

    def get_tunner(self, configs) -> AutoTuner:
        o = self.opts
        tuner = AutoTuner(self.factory, configs).set_profile_args(
            supply_type=o["supply_type"], ref_prog=o["ref_prog"], supply_prog=o["supply_prog"], rtol=o["rtol"],
            atol=o["atol"], max_mismatched_ratio=o["max_mismatched_ratio"], skip_check=o["skip_check"],
            manual_check_prog=o["manual_check_prog"], cache_input_tensors=o["cache_input_tensors"])
        return tuner

    def __call__(self, *args, **kwargs):
        configs = self._configs(args, kwargs)
        tunable = set().union(*(c.keys() for c in configs)) if configs else set()
        bound = inspect.signature(self.__wrapped_factory__).bind_partial(*args, **kwargs).arguments
        if tunable and tunable <= set(bound):
            return self.factory(*args, **kwargs)  # every tunable parameter was given: no search
        key = (tuple(args), tuple(sorted(kwargs.items())))
        if key not in self._tuner_cache:
            free = [{k: v for k, v in c.items() if k not in bound} for c in configs]
            tuner = self.get_tunner(free)
            tuner.jit_compile = lambda **config: self.factory(*args, **kwargs, **config)
            tuner.set_kernel_parameters(_normalize([list(args), kwargs]), None)
            result = tuner.run(self.opts["warmup"], self.opts["rep"], self.opts["timeout"])
            result.kernel._tuner_result = result
            self._tuner_cache[key] = result.kernel
        return self._tuner_cache[key]


def autotune(func: Callable = None, *, configs: Union[Sequence[dict], Callable], warmup: int = 25, rep: int = 100,
             timeout: int = 100, supply_type: TensorSupplyType = TensorSupplyType.Auto,
             ref_prog: Optional[Callable] = None, supply_prog: Optional[Callable] = None, rtol: float = 1e-2,
             atol: float = 1e-2, max_mismatched_ratio: float = 0.01, skip_check: bool = False,
             manual_check_prog: Optional[Callable] = None, cache_input_tensors: bool = False):
    """``@autotune(configs=[...]) @jit(...) def factory(..., tile=..., algo=...)`` -- calling the
    result without the tunable parameters searches ``configs`` on first use and returns the fastest
    kernel (``kernel.get_tuner_result()`` tells which); passing them all skips the search."""
    if callable(func):
        raise ValueError("Use tilelang.autotune to decorate func without arguments is not supported yet.")
    opts = dict(configs=configs, warmup=warmup, rep=rep, timeout=timeout, supply_type=supply_type, ref_prog=ref_prog,
                supply_prog=supply_prog, rtol=rtol, atol=atol, max_mismatched_ratio=max_mismatched_ratio,
                skip_check=skip_check, manual_check_prog=manual_check_prog, cache_input_tensors=cache_input_tensors)

    def decorator(factory: Callable):
        if not callable(factory):
            raise TypeError("autotune decorates the factory returned by @jit")
        return AutoTuneImpl(factory, **opts)

    return decorator
