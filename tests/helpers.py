"""Shared input generators and tolerance checks for the parity tests."""
from __future__ import annotations

import numpy as np
import torch

from oracle import ref

DT = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32}


def gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def make_w4(N, K, group, dtype, zeros_kind, seed, full_range=True):
    """Packed uint4 weights + per-group scales U[0.005, 0.02] + zeros of the requested kind:
    None | 'scalar8' | 'int' (tensor, U{6..9}) | 'frac' (tensor, non-integer values)."""
    g = gen(seed)
    hi = 256 if full_range else 255
    Wp = torch.randint(0, hi, (N, K // 2), dtype=torch.uint8, generator=g)
    G = K // group
    scales = (torch.rand(N, G, generator=g) * 0.015 + 0.005).to(dtype)
    if zeros_kind is None:
        zeros = None
    elif zeros_kind == "scalar8":
        zeros = 8
    elif zeros_kind == "int":
        zeros = torch.randint(6, 10, (N, G), generator=g).to(dtype)
    elif zeros_kind == "frac":
        zeros = (torch.rand(N, G, generator=g) * 3 + 6).to(dtype)
    else:
        raise ValueError(zeros_kind)
    return Wp, scales, zeros


def bits(t: torch.Tensor) -> np.ndarray:
    """Bit pattern view for exact comparisons of 16-bit float tensors."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float32:
        return t.view(torch.int32).numpy().view(np.uint32)
    return t.numpy()


def assert_bit_equal(a: torch.Tensor, b: torch.Tensor, what=""):
    assert a.shape == b.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(b.shape)}"
    assert a.dtype == b.dtype, f"{what}: dtype {a.dtype} vs {b.dtype}"
    A, B = bits(a), bits(b)
    if not np.array_equal(A, B):
        bad = np.argwhere(A != B)
        i = tuple(bad[0])
        raise AssertionError(f"{what}: {len(bad)} of {A.size} elements differ; first at {i}: "
                             f"{a.cpu()[i].item()} vs {b.cpu()[i].item()}")


def half_ulp(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Half a unit in the last place of `dtype` at magnitude |x| (0 for float32 outputs)."""
    if dtype == torch.float32:
        return torch.zeros_like(x)
    mant = 10 if dtype == torch.float16 else 7
    e = torch.floor(torch.log2(x.abs().clamp_min(2.0 ** -14)))
    return torch.pow(2.0, e - mant) * 0.5


def check_float_output(out: torch.Tensor, ref_f32: torch.Tensor, what=""):
    """The float-output bar: against the fp32-accumulated reference
       * relative L2 <= 1e-3 (both rounded to the output type),
       * max-abs <= 1e-2 on top of the output type's own rounding (half an ulp at that
         magnitude; zero for float32 outputs),
       * torch.testing.assert_close(rtol=1e-2, atol=1e-2), the reference examples' criterion."""
    out = out.detach().cpu()
    ref_cast = ref_f32.to(out.dtype)
    o, r = out.float(), ref_cast.float()
    assert torch.isfinite(o).all(), f"{what}: non-finite output"
    rel = (o - r).norm() / r.norm().clamp_min(1e-30)
    assert rel <= 1e-3, f"{what}: relative L2 {rel:.3e} > 1e-3"
    err = (o - ref_f32.float()).abs()
    allowed = 1e-2 + half_ulp(ref_f32.float(), out.dtype)
    worst = (err - allowed).max()
    assert worst <= 0, f"{what}: max-abs {err.max():.3e} exceeds 1e-2 (+ half ulp of {out.dtype}) by {worst:.3e}"
    torch.testing.assert_close(out, ref_cast, rtol=1e-2, atol=1e-2)


def w4a16_reference(A, Wp, scales, zeros, group, out_dtype="float32"):
    return ref.ref_program_w4a16(A, Wp, scales, zeros, group, out_dtype)
