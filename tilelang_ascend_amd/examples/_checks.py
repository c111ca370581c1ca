"""Torch-only reference programs the example scripts check the kernels against.

They are the examples' own golden computations (vectorised; the reference's versions loop per
element) and run on the CPU with torch, like the reference's.  Integer products go through float64,
which is exact below 2**53 and much faster than torch's CPU integer matmul.
"""
import torch

DTYPES = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32, "int8": torch.int8,
          "int32": torch.int32}


def unpack_nibbles(packed: torch.Tensor) -> torch.Tensor:
    """uint8 [N, K/2] -> int16 [N, K], element k = nibble k % 2 of byte k // 2 (low nibble first)."""
    p = packed.cpu().to(torch.int16)
    return torch.stack((p & 0xF, p >> 4), dim=-1).reshape(p.shape[0], -1)


def sign_extend4(u: torch.Tensor) -> torch.Tensor:
    return torch.where(u >= 8, u - 16, u)


def exact_int_matmul(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return (a.cpu().double() @ b.cpu().double()).to(torch.int64)
