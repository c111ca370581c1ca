"""Timing and validation helpers with the reference profiler's surface.

Reference: tilelang/profiler/bench.py:9-102 (``do_bench``: estimate, warm up for ~`warmup` ms,
time ~`rep` ms of repetitions with one event pair each, clear a cache-sized buffer before every
repetition, aggregate) and tilelang/profiler/__init__.py:21-293 (``Profiler.assert_allclose``,
``do_bench``, ``run_once``; obtained from ``kernel.get_profiler()``).

The flush buffer here is 512 MB: the MI355X last-level cache is 256 MB, so the reference's
256 MB buffer would leave part of the inputs resident.
"""
from __future__ import annotations

import enum
from functools import partial
from typing import Callable, List, Optional, Sequence, Union

import torch

FLUSH_BYTES = 512 * 1024 * 1024


class TensorSupplyType(enum.Enum):
    """tilelang/utils/tensor.py:14-21."""

    Integer = 1
    Uniform = 2
    Normal = 3
    Randn = 4
    Zero = 5
    One = 6
    Auto = 7


def _supply(shape, dtype: torch.dtype, kind: TensorSupplyType, device) -> torch.Tensor:
    if kind == TensorSupplyType.Zero:
        return torch.zeros(shape, dtype=dtype, device=device)
    if kind == TensorSupplyType.One:
        return torch.ones(shape, dtype=dtype, device=device)
    if not dtype.is_floating_point or kind == TensorSupplyType.Integer:
        if dtype == torch.uint8:
            return torch.randint(0, 256, shape, dtype=dtype, device=device)
        return torch.randint(-8, 8, shape, device=device).to(dtype)
    if kind == TensorSupplyType.Uniform:
        return (torch.rand(shape, device=device) * 2 - 1).to(dtype)
    return torch.randn(shape, device=device).to(dtype)


def do_bench(fn: Callable, warmup: float = 25, rep: float = 100, _n_warmup: int = 0, _n_repeat: int = 0,
             grad_to_none: Optional[List[torch.Tensor]] = None, quantiles: Optional[List[float]] = None,
             fast_flush: bool = True, return_mode: str = "mean", flush: bool = True) -> Union[float, List[float]]:
    """Milliseconds per call of ``fn`` on the current stream (argument meaning as in the
    reference; ``flush=False`` skips the cache-clearing write for back-to-back timings)."""
    assert return_mode in ["min", "max", "mean", "median"]
    fn()
    torch.cuda.synchronize()
    cache = torch.empty(FLUSH_BYTES // 4, dtype=torch.int32, device="cuda") if flush else None

    def clear():
        if cache is not None:
            cache.zero_()

    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        clear()
        fn()
    e1.record()
    torch.cuda.synchronize()
    estimate_ms = max(e0.elapsed_time(e1) / 5, 1e-4)
    n_warmup = _n_warmup if _n_warmup > 0 else max(1, int(warmup / estimate_ms))
    n_repeat = _n_repeat if _n_repeat > 0 else max(1, int(rep / estimate_ms))
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for _ in range(n_warmup):
        fn()
    for i in range(n_repeat):
        if grad_to_none is not None:
            for x in grad_to_none:
                x.grad = None
        clear()
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    times = torch.tensor([s.elapsed_time(e) for s, e in zip(starts, ends)], dtype=torch.float)
    if quantiles is not None:
        ret = torch.quantile(times, torch.tensor(quantiles, dtype=torch.float)).tolist()
        return ret[0] if len(ret) == 1 else ret
    return getattr(torch, return_mode)(times).item()


class Profiler:
    """``kernel.get_profiler()``: generates inputs for the kernel's parameter list, checks the
    kernel against a reference program and times it."""

    def __init__(self, kernel, tensor_supply_type: TensorSupplyType = TensorSupplyType.Auto):
        self.adapter = kernel
        self.params = kernel.params
        self.result_idx = list(kernel.result_idx)
        self.workspace_idx = list(kernel.workspace_idx)
        self.supply_type = tensor_supply_type

    def _get_params(self, with_output=False, with_workspace=False):
        return [p for i, p in enumerate(self.params)
                if (with_output or i not in self.result_idx) and (with_workspace or i not in self.workspace_idx)]

    def _get_inputs(self, with_output=False, with_workspace=False, symbols=None):
        from .jit import TORCH_DTYPES

        symbols = dict(symbols or {})
        ins = []
        for p in self._get_params(with_output, with_workspace):
            shape = [symbols.get(s, 128) if isinstance(s, str) else int(s) for s in p.shape]
            ins.append(_supply(shape, TORCH_DTYPES[p.dtype], self.supply_type, "cuda"))
        return ins

    @property
    def func(self):
        return self.adapter

    def __call__(self, *args, **kwds):
        return self.adapter(*args, **kwds)

    def run_once(self, func: Optional[Callable] = None):
        return (func or self.__call__)(*self._get_inputs())

    def assert_allclose(self, reference_program: Callable, input_tensors: Optional[Sequence[torch.Tensor]] = None,
                        atol: float = 1e-2, rtol: float = 1e-2, max_mismatched_ratio: float = 0.01):
        """Outputs of the kernel vs ``reference_program(*inputs)``; at most `max_mismatched_ratio`
        of the elements may fall outside |a - b| <= atol + rtol * |b|."""
        ins = list(self._get_inputs() if input_tensors is None else input_tensors)
        ref_outs = reference_program(*ins)
        torch.cuda.synchronize()
        lib_outs = self.func(*ins)
        torch.cuda.synchronize()
        as_list = lambda o: [o] if isinstance(o, torch.Tensor) else list(o or [])  # noqa: E731
        ref_outs, lib_outs = as_list(ref_outs), as_list(lib_outs)
        assert len(lib_outs) == len(ref_outs), "len(lib_tensors) not equals to len(ref_tensors) !"
        for got, want in zip(lib_outs, ref_outs):
            want = want.to(got.device)
            assert got.shape == want.shape, f"shape {tuple(got.shape)} vs {tuple(want.shape)}"
            bad = ~torch.isclose(got.double(), want.double(), rtol=rtol, atol=atol)
            n_bad, allowed = int(bad.sum()), int(max_mismatched_ratio * got.numel())
            if n_bad > allowed:
                raise AssertionError(f"{n_bad} of {got.numel()} elements mismatch (allowed {allowed}); "
                                     f"max abs diff {(got.double() - want.double()).abs().max().item():.4g}")

    def assert_consistent(self, repeat: int = 10, input_tensors: Optional[Sequence[torch.Tensor]] = None) -> None:
        """The reference's race check (tilelang/profiler/__init__.py:188-205): the kernel is run ``repeat`` more times
        on the same inputs and every run must reproduce the first.  The reference asks for ``torch.allclose``; the
        kernels here add their partial sums in a fixed order, so the bits must be equal."""
        ins = list(self._get_inputs() if input_tensors is None else input_tensors)
        as_list = lambda o: [o] if isinstance(o, torch.Tensor) else list(o or [])  # noqa: E731
        # (an output the kernel returns may be a buffer it reuses: keep copies)
        ref_outs = [o.clone() for o in as_list(self.func(*ins))]
        torch.cuda.synchronize()
        for i in range(repeat):
            lib_outs = as_list(self.func(*ins))
            torch.cuda.synchronize()
            assert len(lib_outs) == len(ref_outs)
            for lhs, rhs in zip(lib_outs, ref_outs):
                same = lhs.dtype == rhs.dtype and lhs.shape == rhs.shape and torch.equal(
                    lhs.view(torch.uint8) if lhs.dtype.is_floating_point else lhs,
                    rhs.view(torch.uint8) if rhs.dtype.is_floating_point else rhs)
                if not same:
                    raise AssertionError(f"result is not consistent: run {i + 2} differs from the first run in "
                                         f"{int((lhs != rhs).sum())} of {lhs.numel()} elements")

    def do_bench(self, func: Optional[Callable] = None, warmup: int = 25, rep: int = 100, n_warmup: int = 1,
                 n_repeat: int = 1, input_tensors: Optional[Sequence[torch.Tensor]] = None) -> float:
        """tilelang/profiler/__init__.py:228-285 (its defaults n_warmup = n_repeat = 1 included)."""
        func = func or self.adapter
        ins = self._get_inputs() if input_tensors is None else list(input_tensors)
        return do_bench(partial(func, *ins), warmup=warmup, rep=rep, _n_warmup=n_warmup, _n_repeat=n_repeat)
