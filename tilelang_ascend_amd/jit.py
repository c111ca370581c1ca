"""JIT front door and kernel objects with the reference's calling contract.

Reference behaviour mirrored here (paths relative to the reference checkout):

* ``@tilelang.jit(out_idx=..., workspace_idx=..., pass_configs=...)`` decorates a *factory*;
  calling the factory returns a kernel, memoised per ``(args, sorted kwargs)``
  (tilelang/jit/__init__.py:197-247).
* ``kernel(*inputs, stream=-1)`` consumes the parameters that are neither outputs nor
  workspaces positionally, allocates outputs with ``torch.empty(shape, dtype,
  device=inputs[0].device)``, validates contiguity / device / dtype, launches on the current
  stream without synchronising and returns the output tensor (or a list when there are
  several) -- tilelang/jit/adapter/cython/cython_wrapper.pyx:75-203.
* negative ``out_idx`` / ``workspace_idx`` are legalised, out-of-range ones raise ValueError
  (tilelang/jit/adapter/base.py:22-46).

Differences, all on the safe side: static shapes ARE checked (the reference has that check
commented out, cython_wrapper.pyx:183-187); workspace parameters are accepted but never
allocated because the fused kernels do not need them; the factories return a ``KernelSpec``
describing a pre-built HIP kernel instead of a TIR ``prim_func`` to compile.
"""
from __future__ import annotations

import enum
import functools
import threading
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple, Union

import torch

from . import _abi
from . import cache as _cache

TORCH_DTYPES = {
    "float16": torch.float16,
    "bfloat16": torch.bfloat16,
    "float32": torch.float32,
    "float": torch.float32,
    "int8": torch.int8,
    "uint8": torch.uint8,
    "int32": torch.int32,
}
ABI_DTYPE = {
    torch.float16: _abi.F16,
    torch.bfloat16: _abi.BF16,
    torch.float32: _abi.F32,
    torch.int8: _abi.I8,
    torch.int32: _abi.I32,
}


class PassConfigKey(str, enum.Enum):
    """Names of tilelang/transform/pass_config.py:8-79 that the quantized-matmul examples pass.
    They steer the reference's compiler passes; here they are accepted, recorded in the cache
    key and otherwise ignored (there is no compiler)."""

    TL_ASCEND_AUTO_SYNC = "tl.ascend_auto_sync"
    TL_ASCEND_AUTO_CV_SYNC = "tl.ascend_auto_cross_core_sync"
    TL_ASCEND_AUTO_CV_COMBINE = "tl.ascend_auto_cv_combine"
    TL_ASCEND_MEMORY_PLANNING = "tl.ascend_memory_planning"
    TIR_MERGE_STATIC_SMEM = "tir.merge_static_smem"
    TL_DISABLE_TMA_LOWER = "tl.disable_tma_lower"
    TL_DISABLE_WARP_SPECIALIZED = "tl.disable_warp_specialized"


@dataclass
class Param:
    """One kernel parameter: name, shape (ints or symbolic names) and dtype string."""

    name: str
    shape: Tuple[Union[int, str], ...]
    dtype: str


@dataclass
class KernelSpec:
    """What a factory hands to ``jit``: the parameter list in the reference's order and the
    launch function ``launch(tensors, symbols, stream)`` that calls the C ABI."""

    name: str
    params: List[Param]
    launch: Callable[[List[Optional[torch.Tensor]], Dict[str, int], int], None]
    attrs: Dict[str, Any] = field(default_factory=dict)


def _legalize_idx(idx, n_params: int, name: str) -> List[int]:
    """tilelang/jit/adapter/base.py:22-46."""
    if idx is None:
        return []
    if isinstance(idx, int):
        idx = [idx]
    elif not isinstance(idx, (list, tuple)):
        raise ValueError(f"{name} should be a list of integers")
    out = []
    for i in idx:
        if i >= n_params or i < -n_params:
            raise ValueError(f"{name} should be an integer between {-n_params} and {n_params - 1}")
        out.append(i + n_params if i < 0 else i)
    return out


class JITKernel:
    """Callable kernel: ``kernel(*inputs, stream=-1) -> tensor | list[tensor]``."""

    def __init__(self, spec: KernelSpec, out_idx=None, workspace_idx=None, pass_configs=None, target="hip",
                 execution_backend="ctypes"):
        self.spec = spec
        self.params = spec.params
        n = len(self.params)
        self.result_idx = _legalize_idx(out_idx, n, "result_idx")
        self.workspace_idx = _legalize_idx(workspace_idx, n, "workspace_idx")
        self.pass_configs = dict(pass_configs or {})
        self.target = target
        self.execution_backend = execution_backend
        self.input_idx = [i for i in range(n) if i not in self.result_idx and i not in self.workspace_idx]
        self._tuner_result = None

    # -- introspection kept for drop-in use ----------------------------------------------
    @property
    def out_idx(self):
        return self.result_idx

    def get_kernel_source(self) -> str:
        return f"// pre-built HIP kernel '{self.spec.name}' in {_abi.library_path()}"

    def get_tuner_result(self):
        """The AutotuneResult of the search that produced this kernel, or None (tilelang/jit/kernel.py)."""
        return self._tuner_result

    def get_profiler(self):
        from .profiler import Profiler

        return Profiler(self)

    # -- the launch contract -----------------------------------------------------------------
    def _resolve(self, inputs: Sequence[torch.Tensor]) -> Dict[str, int]:
        symbols: Dict[str, int] = {}
        for pos, pi in enumerate(self.input_idx):
            if pos >= len(inputs):
                break
            t = inputs[pos]
            if not isinstance(t, torch.Tensor):
                continue
            for d, s in enumerate(self.params[pi].shape):
                if isinstance(s, str) and d < t.dim() and s not in symbols:
                    symbols[s] = int(t.shape[d])
        return symbols

    def forward(self, inputs: Sequence[torch.Tensor], stream: int = -1):
        n_in = len(self.input_idx)
        if len(inputs) < n_in:
            raise ValueError(f"Expected {n_in} inputs, got {len(inputs)} with {len(self.params)} params")
        # surplus positionals are ignored, like the reference (cython_wrapper.pyx:102-141)
        inputs = list(inputs[:n_in])
        for t in inputs:
            if not isinstance(t, torch.Tensor):
                raise ValueError(f"Unsupported tensor type: {type(t)}")
        if stream == -1:
            stream = torch.cuda.current_stream().cuda_stream if torch.cuda.is_available() else 0
        symbols = self._resolve(inputs)
        device = inputs[0].device if inputs else torch.device("cuda", torch.cuda.current_device())

        tensors: List[Optional[torch.Tensor]] = []
        it = iter(inputs)
        for i, prm in enumerate(self.params):
            if i in self.workspace_idx:
                tensors.append(None)  # fused kernels need no global scratch
            elif i in self.result_idx:
                shape = []
                for s in prm.shape:
                    if isinstance(s, str):
                        if s not in symbols:
                            raise KeyError(f"Unfounded symbolic var: {s}")
                        shape.append(symbols[s])
                    else:
                        shape.append(int(s))
                tensors.append(torch.empty(*shape, dtype=TORCH_DTYPES[prm.dtype], device=device))
            else:
                tensors.append(next(it))

        for i, (prm, t) in enumerate(zip(self.params, tensors)):
            if t is None:
                continue
            if not t.is_contiguous():
                raise ValueError(f"Input tensor at index {i} must be contiguous")
            if t.device.type != device.type or (
                t.device.index is not None and device.index is not None and t.device.index != device.index
            ):
                raise ValueError(f"Buffer device mismatch for parameter {prm.name}: expected {device}, got {t.device}")
            want = TORCH_DTYPES[prm.dtype]
            if t.dtype != want:
                raise ValueError(f"Buffer dtype mismatch for parameter {prm.name}: expected {want}, got {t.dtype}")
            if t.dim() != len(prm.shape):
                raise ValueError(
                    f"Static shape mismatch for parameter {prm.name}: expected {len(prm.shape)} dims, got {tuple(t.shape)}"
                )
            for d, s in enumerate(prm.shape):
                exp = symbols.get(s) if isinstance(s, str) else int(s)
                if exp is not None and int(t.shape[d]) != exp:
                    raise ValueError(
                        f"Static shape mismatch for parameter {prm.name}: expected {exp} at index {d}, got {tuple(t.shape)}"
                    )
        if device.type != "cuda":
            raise ValueError(
                f"Buffer device mismatch for parameter {self.params[0].name}: expected a ROCm device ('cuda'), got {device}"
            )
        with torch.cuda.device(device):
            self.spec.launch(tensors, symbols, stream)
        if len(self.result_idx) == 1:
            return tensors[self.result_idx[0]]
        return [tensors[i] for i in self.result_idx]

    def __call__(self, *args, stream: int = -1):
        return self.forward(list(args), stream=stream)


def compile(func: KernelSpec = None, out_idx=None, workspace_idx=None, execution_backend="ctypes", target="auto",  # noqa: A001
            target_host=None, verbose=False, pass_configs=None, platform="auto") -> JITKernel:
    """Non-decorator form (tilelang/jit/__init__.py:36-91): turn a KernelSpec into a JITKernel,
    through the kernel cache."""
    if not isinstance(func, KernelSpec):
        raise TypeError("tilelang_ascend_amd.compile expects the KernelSpec returned by an operator factory")
    key = _cache.make_key(func, out_idx, workspace_idx, target, execution_backend, pass_configs)
    return _cache.cached(key, lambda: JITKernel(func, out_idx, workspace_idx, pass_configs, "hip", execution_backend))


class _JitImplementation:
    """tilelang/jit/__init__.py:94-247 -- memoises per call signature, thread safe."""

    def __init__(self, out_idx=None, workspace_idx=None, target="auto", target_host=None, platform="auto",
                 execution_backend="ctypes", verbose=False, pass_configs=None, debug_root_path=None):
        self.out_idx = out_idx
        self.workspace_idx = workspace_idx
        self.target = target
        self.execution_backend = execution_backend
        self.pass_configs = pass_configs
        self._kernel_cache: Dict[tuple, JITKernel] = {}
        self._lock = threading.Lock()

    def __call__(self, func: Callable) -> Callable:
        @functools.wraps(func)
        def wrapper(*args, **kwargs):
            key = (tuple(args), tuple(sorted(kwargs.items())))
            with self._lock:
                hit = self._kernel_cache.get(key)
            if hit is not None and _cache.is_cache_enabled():
                return hit
            spec = func(*args, **kwargs)
            out_idx = list(self.out_idx) if isinstance(self.out_idx, (list, tuple)) else self.out_idx
            ws_idx = list(self.workspace_idx) if isinstance(self.workspace_idx, (list, tuple)) else self.workspace_idx
            kernel = compile(spec, out_idx=out_idx, workspace_idx=ws_idx, target=self.target,
                             execution_backend=self.execution_backend, pass_configs=self.pass_configs)
            with self._lock:
                self._kernel_cache[key] = kernel
            return kernel

        wrapper.__wrapped_factory__ = func
        return wrapper


def jit(func: Callable = None, *, out_idx=None, workspace_idx=None, target="auto", target_host=None, platform="auto",
        execution_backend="ctypes", verbose=False, pass_configs=None, debug_root_path=None):
    """Decorator with the reference's keyword surface (tilelang/jit/__init__.py:250-327)."""
    impl = _JitImplementation(out_idx=out_idx, workspace_idx=workspace_idx, target=target, target_host=target_host,
                              platform=platform, execution_backend=execution_backend, verbose=verbose,
                              pass_configs=pass_configs, debug_root_path=debug_root_path)
    if callable(func):
        return impl(func)
    return impl
