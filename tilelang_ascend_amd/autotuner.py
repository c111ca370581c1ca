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


# ---- tuned kernel choice for the C entry points ------------------------------------------------------------------
# The reference's tuner result selects a compiled kernel; here it selects which pre-built W4A16 family
# ``tlq_gemm_w4a16_ws`` runs for a call signature when asked for TLQ_ALGO_AUTO.  The result lives in the library's own
# table (tlq_w4a16_choice_set), so callers of the C ABI get it too, and in one text file per device size under
# ``<cache dir>/autotuner`` (the reference's tuner cache lives there as well, tilelang/cache/tuner_cache.py), which
# ``cache.clear_cache()`` removes and which ``ops.w4a16_gemm`` installs once per process.

W4A16_FAMILIES = {"gemv": 1, "mfma": 2, "skinny": 3, "two_pass": 4, "stream": 5, "decode": 6, "panel": 7, "panel256": 8,
                  "panelm": 9}
_choices_lock = threading.Lock()
_choices_loaded = False


def w4a16_choice_path(cus: Optional[int] = None) -> str:
    """The file that holds the tuned choices for devices with ``cus`` compute units (default: the current device)."""
    from . import _abi
    if cus is None:
        cus = _abi.load().tlq_device_cu_count()
    return os.path.join(AutoTuner.cache_dir(), f"w4a16_choices_{int(cus)}cu.txt")


def load_w4a16_choices(path: Optional[str] = None) -> int:
    """Install the entries of ``path`` (default: the current device's file) into the library's table; returns how many
    entries the table holds afterwards.  A missing file installs nothing."""
    from . import _abi
    lib = _abi.load()
    path = path or w4a16_choice_path()
    if os.path.exists(path):
        _abi.check(lib.tlq_w4a16_choice_load(path.encode()))
    return int(lib.tlq_w4a16_choice_count())


def save_w4a16_choices(path: Optional[str] = None) -> str:
    """Write the library's table to ``path`` (default: the current device's file)."""
    from . import _abi
    path = path or w4a16_choice_path()
    os.makedirs(os.path.dirname(path), exist_ok=True)
    tmp = f"{path}.tmp{os.getpid()}"
    _abi.check(_abi.load().tlq_w4a16_choice_save(tmp.encode()))
    os.replace(tmp, path)
    return path


def clear_w4a16_choices() -> None:
    """Empty the library's table (the file stays; ``cache.clear_cache()`` removes it)."""
    from . import _abi
    _abi.load().tlq_w4a16_choice_clear()


def ensure_w4a16_choices_loaded() -> None:
    """Once per process: install the current device's persisted choices, if there are any.  ``TLQ_TUNED_CHOICES=0``
    turns this off.  Touches the GPU only when a choice file exists."""
    global _choices_loaded
    if _choices_loaded:
        return
    with _choices_lock:
        if _choices_loaded:
            return
        _choices_loaded = True
        if os.environ.get("TLQ_TUNED_CHOICES", "1") == "0":
            return
        try:
            d = AutoTuner.cache_dir()
            if not any(n.startswith("w4a16_choices_") and n.endswith("cu.txt") for n in os.listdir(d)):
                return
            load_w4a16_choices()
        except (OSError, RuntimeError) as e:
            logger.warning("tuned W4A16 kernel choices not installed: %s", e)


def tune_w4a16_choice(M: int, N: int, K: int, group_size: int = 128, dtype: str = "float16", zeros: Optional[str] = "tensor",
                      candidates: Optional[Sequence[str]] = None, rep: int = 20, rounds: int = 5, min_gain: float = 0.03,
                      persist: bool = True, seed: int = 0) -> Dict[str, Any]:
    """Measure the W4A16 kernel families on one call signature and make the fastest the library's choice for it.

    Every family in ``candidates`` (default: all) is run through ``tlq_gemm_w4a16_ws`` by name with the workspace it asks
    for (``tlq_w4a16_workspace_bytes_for``); families that refuse the shape are recorded under ``"skipped"`` with the
    library's message, a family whose output is not close to the rule-based choice's is recorded under ``"rejected"``.
    Timings are medians over ``rounds`` rounds of ``rep`` back-to-back launches (more for short kernels: half a
    millisecond per timed region at least), the families taking turns inside a round in a rotating order.  What is
    measured is therefore the rate of a queue of identical launches, in which the head of one launch overlaps the tail of the
    one before; for kernels of a few microseconds that can differ from a single launch's duration by a microsecond (kernels of
    many small work-groups overlap more than one work-group per CU does), so a gain below a microsecond on such a problem
    says little about a program that runs other kernels in between.
    The winner is installed (``tlq_w4a16_choice_set``) when it beats the rule-based choice by ``min_gain`` or more;
    otherwise any earlier entry for the signature is removed.  ``persist`` rewrites the device's choice file.

    Returns ``{"choice": name | "auto", "latency_us": {name: us}, "skipped": {...}, "rejected": {...}, "path": file | None}``.
    """
    import statistics
    from . import _abi
    lib = _abi.load()
    tdt = {"float16": torch.float16, "bfloat16": torch.bfloat16}[dtype]
    code = {"float16": _abi.F16, "bfloat16": _abi.BF16}[dtype]
    if zeros not in ("tensor", "scalar", None):
        raise ValueError("zeros must be 'tensor', 'scalar' or None")
    if K % group_size != 0:
        raise ValueError("group_size must divide K")
    dev = torch.device("cuda")
    g = torch.Generator(device="cpu").manual_seed(seed)
    Wp = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=g).to(dev)  # two random 4-bit codes per byte
    A = torch.randn(M, K, generator=g).to(tdt).to(dev)
    S = (torch.rand(N, K // group_size, generator=g) * 0.02 + 0.005).to(tdt).to(dev)
    Z = torch.randint(0, 16, (N, K // group_size), generator=g).to(tdt).to(dev) if zeros == "tensor" else None
    zs = 8.0 if zeros == "scalar" else 0.0
    stream = torch.cuda.current_stream().cuda_stream
    names = ["auto"] + [n for n in (candidates or W4A16_FAMILIES) if n != "auto"]
    for n in names[1:]:
        if n not in W4A16_FAMILIES:
            raise ValueError(f"unknown family {n!r}; known: {sorted(W4A16_FAMILIES)}")
    # the rule-based choice is the baseline: no entry for this signature while measuring
    _abi.check(lib.tlq_w4a16_choice_set(M, N, K, group_size, code, 0))
    need = max([lib.tlq_w4a16_workspace_bytes(M, N, K)] + [lib.tlq_w4a16_workspace_bytes_for(M, N, K, W4A16_FAMILIES[n]) for n in names[1:]])
    ws = torch.empty(max(int(need), 16), dtype=torch.uint8, device=dev)
    C = torch.empty(M, N, dtype=tdt, device=dev)

    def call(name: str) -> int:
        algo = 0 if name == "auto" else W4A16_FAMILIES[name]
        return lib.tlq_gemm_w4a16_ws(_abi.ptr(A), _abi.ptr(Wp), _abi.ptr(S), _abi.ptr(Z), _abi.ptr(C), M, N, K, group_size, zs, code,
                                     code, algo, _abi.ptr(ws), ws.numel(), stream)

    _abi.check(call("auto"))
    torch.cuda.synchronize()
    want = C.float().clone()
    scale = float(want.abs().max().clamp_min(1e-6))
    alive, skipped, rejected = ["auto"], {}, {}
    for n in names[1:]:
        C.zero_()
        if call(n) != 0:
            skipped[n] = _abi.last_error()
            continue
        torch.cuda.synchronize()
        err = float((C.float() - want).abs().max()) / scale
        if not err <= 2e-2:
            rejected[n] = f"max |difference| / max |C| = {err:.3g} against the rule-based choice"
            continue
        alive.append(n)
    times: Dict[str, List[float]] = {n: [] for n in alive}
    # short kernels: enough launches per timed region (half a millisecond or more) for the differences to be real
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    call("auto")
    e0.record()
    for _ in range(4):
        call("auto")
    e1.record()
    torch.cuda.synchronize()
    per_call_us = max(e0.elapsed_time(e1) * 1000.0 / 4, 1.0)
    rep = max(rep, min(200, int(500.0 / per_call_us) + 1))
    for r in range(max(1, rounds)):
        # (the families take turns in a rotating order: whoever runs first after a pause is measured a little slow)
        for n in alive[r % len(alive):] + alive[:r % len(alive)]:
            for _ in range(3):
                call(n)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(rep):
                call(n)
            e1.record()
            torch.cuda.synchronize()
            times[n].append(e0.elapsed_time(e1) * 1000.0 / rep)
    lat = {n: statistics.median(v) for n, v in times.items()}
    named = [n for n in lat if n != "auto"]
    best = min(named, key=lat.get) if named else "auto"
    choice = best if best != "auto" and lat[best] <= lat["auto"] * (1.0 - min_gain) else "auto"
    _abi.check(lib.tlq_w4a16_choice_set(M, N, K, group_size, code, 0 if choice == "auto" else W4A16_FAMILIES[choice]))
    path = None
    if persist:
        try:
            path = save_w4a16_choices()
        except (OSError, RuntimeError) as e:
            logger.warning("tuned W4A16 kernel choices not saved: %s", e)
    return {"choice": choice, "latency_us": lat, "skipped": skipped, "rejected": rejected, "path": path}
