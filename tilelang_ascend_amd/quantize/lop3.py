"""Fast-decode intrinsic groups for interleaved low-bit weights.

Reference: ``get_lop3_intrin_group`` (tilelang/quantize/lop3.py:1090-1202) returns the name and the
CUDA source of a device function that decodes one 32-bit word of interleaved nibbles with
``lop3.b32`` + paired fp16 arithmetic.  The gfx950 counterparts (``v_and_or_b32`` +
``v_pk_{add,mul,fma}_f16``) live in ``csrc/decode_i4.h``; this module hands out that header's text
under the reference's naming grammar, and ``decode`` runs the same device functions on a tensor
through the C ABI (``tlq_decode_i4_interleaved``).

The quantized-matmul path uses 4-bit sources only; the 2-bit and 1-bit decoders (``csrc/decode_lowbit.h``,
``tlq_decode_lowbit_interleaved``, ``decode_lowbit``) are there for kernels written against the reference's names.  The
"_offset" decoders (storage_scope "warp" with scaling: the two halves of a word belong to different groups) exist for
4-bit sources, as in the reference's table; ``decode_offset`` runs them on a tensor.
"""
from __future__ import annotations

import os
from typing import Dict, Literal, Optional

_HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc", "decode_i4.h")
_HEADER_LOWBIT = os.path.join(os.path.dirname(_HEADER), "decode_lowbit.h")
ZEROS_MODES = {"original": 1, "rescale": 2, "quantized": 3}


def get_lop3_intrin_group(
    out_dtype: Literal["float16", "int8", "int4"],
    source_format: Literal["int", "uint"] = "uint",
    source_bit: int = 4,
    storage_dtype: Literal["int32", "int8"] = "int8",
    with_scaling: bool = False,
    with_zeros: bool = False,
    zeros_mode: Literal["original", "rescale", "quantized"] = "original",
    storage_scope: str = "local",
) -> Dict[str, str]:
    """Same arguments, checks, ``func_name`` grammar and return shape as the reference
    (lop3.py:1139-1202): {"func_name": "decode_i4u_to_f16_scale_zeros_original", "c_source": ...}.
    ``c_source`` is HIP (namespace ``tlq_decode``).  2-bit and 1-bit sources (lop3.py:423-996, 1048-1087) have the
    decoders the reference's table has: no "_offset" forms, quantized zeros for 2-bit only, the packed 4-bit target for
    2-bit only; any other combination raises KeyError as the reference's table lookup does."""
    assert out_dtype in ["float16", "int8", "int4"], (
        f"Invalid out_dtype: {out_dtype}. Expected 'float16' or 'int8' or 'int4' .")
    if source_format not in ["int", "uint"]:
        raise ValueError(f"Invalid source_format. Expected 'int' or 'uint', but got {source_format}.")
    if with_zeros and source_format == "int":
        raise ValueError(f"Zeros are not supported for signed integers, but got {source_format}")
    if with_zeros and zeros_mode not in ZEROS_MODES:
        raise ValueError(f"Invalid zeros_mode: {zeros_mode}")
    d4f = {"float16": "f16", "int8": "i8s", "int4": "i4s"}[out_dtype]
    func_name = "decode_i{}{}_to_{}".format(source_bit, "u" if source_format == "uint" else "s", d4f)
    if with_scaling:
        func_name += "_scale"
    if with_zeros:
        func_name += f"_zeros_{zeros_mode}"
    if storage_scope == "warp" and with_scaling:
        func_name += "_offset"
    if source_bit not in (4, 2, 1):
        raise KeyError(f"i{source_bit}_to_{d4f}: no decoder for {source_bit}-bit sources")
    if out_dtype != "float16" and (with_scaling or with_zeros):
        raise KeyError(f"i{source_bit}_to_{d4f[:2]}" + ("_scale" if with_scaling else "") + " has no decoder")
    if out_dtype == "int4" and source_bit != 2:
        raise KeyError(f"i{source_bit}_to_i4 has no decoder")
    if with_zeros and not with_scaling:
        raise KeyError(f"i{source_bit}_to_f16_zeros_{zeros_mode} has no decoder (zeros need scaling)")
    if source_bit != 4 and func_name.endswith("_offset"):
        raise KeyError(f"{func_name} has no decoder (two-group forms exist for 4-bit sources only)")
    if source_bit == 1 and with_zeros and zeros_mode == "quantized":
        raise KeyError("i1_to_f16_scale_zeros_quantized has no decoder")
    header = _HEADER if source_bit == 4 else _HEADER_LOWBIT
    with open(header) as f:
        source = f.read()
    if source_bit != 4:  # (the low-bit header builds on the 4-bit one's helpers)
        with open(_HEADER) as f:
            source = f.read() + "\n" + source.replace('#include "decode_i4.h"', "").replace("#pragma once", "")
    assert f" {func_name}(" in source, func_name
    return {"func_name": func_name, "c_source": source}


def decode(words, out_dtype: str = "float16", source_format: str = "uint", scale=None, zeros=None,
           zeros_mode: Optional[str] = None, group_size: int = -1):
    """Run the decoder named by the arguments on a device tensor of interleaved weights.

    words: int8 / uint8 / int32 tensor, last dimension a whole number of 32-bit words.  Returns a
    tensor with the last dimension expanded to one element per nibble (float16 or int8).
    scale (fp16) / zeros (fp16, or an integer tensor for zeros_mode='quantized'): one value per
    `group_size` consecutive weights (default: one value for everything)."""
    import torch

    from .. import _abi

    lib = _abi.load()
    assert out_dtype in ("float16", "int8")
    w = words.contiguous()
    n_bytes = w.numel() * w.element_size()
    assert n_bytes % 4 == 0, "the weights must be whole 32-bit words"
    n_words = n_bytes // 4
    last = w.shape[-1] * w.element_size() * 2
    out = torch.empty(*w.shape[:-1], last, dtype=torch.float16 if out_dtype == "float16" else torch.int8, device=w.device)
    mode = 0 if zeros_mode is None else ZEROS_MODES[zeros_mode]
    wpg = n_words if group_size in (-1, None) else group_size // 8
    s = None if scale is None else scale.to(device=w.device, dtype=torch.float16).contiguous()
    z = None
    if zeros is not None:
        z = zeros.to(device=w.device, dtype=torch.int16 if mode == 3 else torch.float16).contiguous()
    if s is not None:
        assert s.numel() * wpg >= n_words, "not enough scales for the weights"
    if z is not None:
        assert z.numel() * wpg >= n_words, "not enough zeros for the weights"
    stream = torch.cuda.current_stream().cuda_stream
    with torch.cuda.device(w.device):
        _abi.check(lib.tlq_decode_i4_interleaved(_abi.ptr(w), _abi.ptr(s), _abi.ptr(z), _abi.ptr(out), n_words, max(wpg, 1),
                                                 _abi.F16 if out_dtype == "float16" else _abi.I8,
                                                 1 if source_format == "int" else 0, mode, stream))
    return out


def decode_offset(words, scale, offset: int, source_format: str = "uint", zeros=None, zeros_mode: Optional[str] = None,
                  group_size: int = -1, zero_offset: int = 0, group_offset: int = 0):
    """Run the "_offset" decoder named by the arguments (lop3.py:82-131, 177-230, 272-322, 364-421) on a device tensor
    of interleaved weights: word i belongs to group g = i // (group_size // 8); its first four weights use scale[g] /
    zeros[g], the last four scale[g + offset] / zeros[g + offset].  For zeros_mode='quantized', zeros is an int32
    tensor of packed 4-bit zero points: the halves take field `group_offset` of zeros[g] and of zeros[g + zero_offset].
    Returns float16, last dimension expanded to one element per nibble."""
    import torch

    from .. import _abi

    lib = _abi.load()
    w = words.contiguous()
    n_bytes = w.numel() * w.element_size()
    assert n_bytes % 4 == 0, "the weights must be whole 32-bit words"
    n_words = n_bytes // 4
    out = torch.empty(*w.shape[:-1], w.shape[-1] * w.element_size() * 2, dtype=torch.float16, device=w.device)
    mode = 0 if zeros_mode is None else ZEROS_MODES[zeros_mode]
    wpg = max(n_words, 1) if group_size in (-1, None) else group_size // 8
    s = scale.to(device=w.device, dtype=torch.float16).contiguous()
    z = None
    if zeros is not None:
        z = zeros.to(device=w.device, dtype=torch.int32 if mode == 3 else torch.float16).contiguous()
    stream = torch.cuda.current_stream().cuda_stream
    with torch.cuda.device(w.device):
        _abi.check(lib.tlq_decode_i4_interleaved_offset(_abi.ptr(w), _abi.ptr(s), _abi.ptr(z), _abi.ptr(out), n_words, wpg,
                                                        s.numel(), 0 if z is None else z.numel(), offset, zero_offset,
                                                        group_offset, 1 if source_format == "int" else 0, mode, stream))
    return out


def decode_lowbit(src, source_bit: int, out_dtype: str = "float16", source_format: str = "uint", scale=None, zeros=None,
                  zeros_mode: Optional[str] = None, group_size: int = -1):
    """Run the 2-bit / 1-bit decoder named by the arguments (lop3.py:423-996, 1048-1087) on a device tensor of interleaved
    weights.  src: int8 / uint8 tensor whose last dimension is a whole number of source units (fp16 target: 2 bytes for
    2-bit, 1 byte for 1-bit sources, 8 weights each; int8 / int4 targets: 4 or 2 bytes, 16 weights each).  Returns float16
    or int8 with one element per weight in the last dimension, or, for ``out_dtype='int4'``, uint8 with two nibbles per
    byte.  scale / zeros: one value per `group_size` consecutive weights (default: one value for everything); zeros is
    fp16, or an integer tensor for zeros_mode='quantized' (2-bit only)."""
    import torch

    from .. import _abi

    lib = _abi.load()
    assert source_bit in (2, 1) and out_dtype in ("float16", "int8", "int4")
    w = src.contiguous()
    assert w.element_size() == 1, "the weights must be a byte tensor"
    out_bits = {"float16": 16, "int8": 8, "int4": 4}[out_dtype]
    per_unit = 8 if out_bits == 16 else 16
    unit_bytes = per_unit * source_bit // 8
    n_bytes = w.numel()
    assert w.shape[-1] % unit_bytes == 0, f"the last dimension must be a whole number of {unit_bytes}-byte units"
    n_units = n_bytes // unit_bytes
    weights_last = w.shape[-1] * 8 // source_bit
    if out_bits == 16:
        out = torch.empty(*w.shape[:-1], weights_last, dtype=torch.float16, device=w.device)
    elif out_bits == 8:
        out = torch.empty(*w.shape[:-1], weights_last, dtype=torch.int8, device=w.device)
    else:
        out = torch.empty(*w.shape[:-1], weights_last // 2, dtype=torch.uint8, device=w.device)
    mode = 0 if zeros_mode is None else ZEROS_MODES[zeros_mode]
    upg = max(n_units, 1) if group_size in (-1, None) else group_size // per_unit
    s = None if scale is None else scale.to(device=w.device, dtype=torch.float16).contiguous()
    z = None
    if zeros is not None:
        z = zeros.to(device=w.device, dtype=torch.int16 if mode == 3 else torch.float16).contiguous()
    if s is not None:
        assert upg >= 1 and s.numel() * upg >= n_units, "not enough scales for the weights"
    if z is not None:
        assert z.numel() * upg >= n_units, "not enough zeros for the weights"
    stream = torch.cuda.current_stream().cuda_stream
    with torch.cuda.device(w.device):
        _abi.check(lib.tlq_decode_lowbit_interleaved(_abi.ptr(w), _abi.ptr(s), _abi.ptr(z), _abi.ptr(out), n_units, max(upg, 1),
                                                     source_bit, out_bits, 1 if source_format == "int" else 0, mode, stream))
    return out
