"""Weight preparation on the GPU (HIP kernels behind tlq_pack_int4 / tlq_quantize_sym4).

``pack_int4`` is general_compress (tilelang/quantize/utils.py:53-69) for 4-bit values, optionally followed
by interleave_weight (:73-101); ``quantize_sym4`` is the quantiser inside gen_quant4 (:5-50) for weights
stored [N, K] with groups along K.  Results are bit-identical to the torch versions in ``quantize.utils``.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import _abi

_INTERLEAVE = {None: 0, "none": 0, "float16": 1, "int8": 2}
_DT = {torch.float16: _abi.F16, torch.bfloat16: _abi.BF16}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def pack_int4(values: torch.Tensor, interleave: Optional[str] = None, storage_dtype: torch.dtype = torch.int8) -> torch.Tensor:
    """values int8 / uint8 [N, K] on the GPU -> packed [N, K // 2] (storage_dtype int8 or uint8).
    interleave: None, "float16" or "int8" (the target_dtype of interleave_weight)."""
    if interleave not in _INTERLEAVE:
        raise ValueError('interleave must be None, "float16" or "int8"')
    if values.dtype not in (torch.int8, torch.uint8) or values.dim() != 2:
        raise ValueError("values must be a 2-D int8 or uint8 tensor")
    if not values.is_cuda or not values.is_contiguous():
        raise ValueError("values must be a contiguous tensor on the GPU")
    N, K = values.shape
    out = torch.empty(N, K // 2, dtype=storage_dtype, device=values.device)
    with torch.cuda.device(values.device):
        _abi.check(_abi.load().tlq_pack_int4(_abi.ptr(values), _abi.ptr(out), N, K, _INTERLEAVE[interleave], _stream()))
    return out


def quantize_sym4(W: torch.Tensor, group_size: int = -1) -> Tuple[torch.Tensor, torch.Tensor]:
    """W fp16 / bf16 [N, K] on the GPU -> (q - 8 as int8 [N, K], scales [N, K // group_size] in W's dtype):
    s = max|w| / 8 per group, q = clamp(round(w / s) + 8, 0, 16).  group_size -1 means one group per row."""
    if W.dtype not in _DT or W.dim() != 2:
        raise ValueError("W must be a 2-D float16 or bfloat16 tensor")
    if not W.is_cuda or not W.is_contiguous():
        raise ValueError("W must be a contiguous tensor on the GPU")
    N, K = W.shape
    g = K if group_size == -1 else int(group_size)
    q = torch.empty(N, K, dtype=torch.int8, device=W.device)
    s = torch.empty(N, K // g if g else 0, dtype=W.dtype, device=W.device)
    with torch.cuda.device(W.device):
        _abi.check(_abi.load().tlq_quantize_sym4(_abi.ptr(W), _abi.ptr(q), _abi.ptr(s), N, K, g, _DT[W.dtype], _stream()))
    return q, s


def scales_kn_to_nk(scales: torch.Tensor) -> torch.Tensor:
    """gen_quant4 (tilelang/quantize/utils.py:5-50) returns its scales as [K / groupsize, N], one row per group of
    input features; the kernels read [N, K / groupsize], a row per output feature next to that feature's packed
    weights.  Returns the transposed copy (works on any device)."""
    if scales.dim() != 2:
        raise ValueError("scales must be 2-D [K / groupsize, N]")
    return scales.t().contiguous()


def pack_gen_quant4(q_minus8: torch.Tensor, scales: torch.Tensor, interleave: Optional[str] = None,
                    saturate: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """Outputs of gen_quant4 -> operands of the W4A16 kernels with zero point 8.

    q_minus8: [K, N] integer tensor in [-8, 8] (gen_quant4's fourth result); scales: [K / groupsize, N] (its third).
    Returns (B_packed uint8 [N, K // 2], scales [N, K / groupsize]) on the GPU, so that
    dequantize_w4(B_packed, scales, 8, groupsize) is gen_quant4's dequantised weight, transposed to [N, K].
    gen_quant4 clamps q to [0, 16] (maxq = 16, utils.py:8 and :30), and 16 does not fit four bits: with saturate=True
    such elements (the positive maximum of a group) are stored as 15, i.e. 7 * s instead of 8 * s; with
    saturate=False their presence raises ValueError."""
    if q_minus8.dim() != 2 or scales.dim() != 2 or scales.shape[1] != q_minus8.shape[1]:
        raise ValueError("expected q_minus8 [K, N] and scales [K / groupsize, N]")
    u = q_minus8.to(torch.int16) + 8
    if int(u.min()) < 0 or int(u.max()) > 16:
        raise ValueError("q_minus8 must lie in [-8, 8]")
    if int(u.max()) == 16:
        if not saturate:
            raise ValueError("q_minus8 holds the value 8 (q = 16), which does not fit four bits")
        u = u.clamp(max=15)
    vals = u.to(torch.uint8).t().contiguous().cuda()
    return pack_int4(vals, interleave, torch.uint8), scales_kn_to_nk(scales).cuda()
