"""Element converters of tilelang/quantize/quantization.py, evaluated on torch tensors.

The reference's functions build TVM expressions that its compiler inlines into a kernel; here
there is no expression compiler, so the same factories return functions that evaluate the
conversion elementwise on integer tensors (on whatever device they live).  Names, factory
arguments and the ``f_convert(nbit, val, pos, dtype)`` signature are kept.

``val`` is a tensor of the storage dtype (or a Python int), ``pos`` the field index inside
each storage word (int or tensor, broadcast against ``val``), ``dtype`` a dtype string.
"""
from __future__ import annotations

import torch

_DT = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32, "float": torch.float32,
       "int8": torch.int8, "int16": torch.int16, "int32": torch.int32, "int64": torch.int64, "uint8": torch.uint8}
_STORAGE = {"uint8": torch.uint8, "int8": torch.int8, "int32": torch.int32, "uint32": torch.int32, "int16": torch.int16,
            "uint16": torch.int16}


def _field(nbit: int, val, pos, storage_dtype: str) -> torch.Tensor:
    """Unsigned value of field `pos` of each storage word, as int64."""
    if isinstance(val, torch.Tensor):
        want = _STORAGE[storage_dtype]
        assert val.dtype == want or (storage_dtype.startswith("uint") and val.dtype == torch.uint8 and want == torch.uint8), \
            f"{val.dtype} != {storage_dtype}"
        bits = int(storage_dtype.lstrip("uint"))
        v = val.to(torch.int64) & ((1 << bits) - 1)
    else:
        v = torch.tensor(int(val), dtype=torch.int64) & 0xFFFFFFFF
    p = pos.to(torch.int64) if isinstance(pos, torch.Tensor) else int(pos)
    return (v >> (p * nbit)) & ((1 << nbit) - 1)


def _tir_packed_to_unsigned_convert(storage_type="uint", storage_nbit=8):
    """tilelang/quantize/quantization.py:198-206: ((val >> pos*nbit) & mask).astype(dtype)."""
    storage_dtype = storage_type + str(storage_nbit)

    def f_convert(nbit: int, val, pos, dtype: str):
        return _field(nbit, val, pos, storage_dtype).to(_DT[dtype])

    return f_convert


def _tir_packed_to_unsigned_convert_with_zeros(storage_type="uint", storage_nbit=8):
    """quantization.py:209-218: (((val >> pos*nbit) & mask) - zero).astype(dtype).  The subtraction
    is exact integer arithmetic for an integer `zero`, and is done in `dtype` for a float one."""
    storage_dtype = storage_type + str(storage_nbit)

    def f_convert(nbit: int, val, pos, zero, dtype: str):
        u = _field(nbit, val, pos, storage_dtype)
        z = zero if isinstance(zero, torch.Tensor) else torch.tensor(zero)
        if z.dtype.is_floating_point:
            return u.to(_DT[dtype]) - z.to(_DT[dtype])
        return (u - z.to(torch.int64)).to(_DT[dtype])

    return f_convert


def _tir_packed_to_signed_convert(storage_type="uint", storage_nbit=8):
    """quantization.py:186-195: offset binary, u.astype(dtype) - 2**(nbit-1)."""
    storage_dtype = storage_type + str(storage_nbit)

    def f_convert(nbit: int, val, pos, dtype: str):
        return (_field(nbit, val, pos, storage_dtype) - (1 << (nbit - 1))).to(_DT[dtype])

    return f_convert


def _tir_packed_int_to_int_convert(storage_type="uint", storage_nbit=8):
    """quantization.py:221-231: two's-complement sign extension of the field."""
    storage_dtype = storage_type + str(storage_nbit)

    def f_convert(nbit: int, val, pos, dtype: str):
        u = _field(nbit, val, pos, storage_dtype)
        return torch.where(u >= (1 << (nbit - 1)), u - (1 << nbit), u).to(_DT[dtype])

    return f_convert


def _tir_packed_int_to_int_to_float(storage_nbit: int):
    """quantization.py:68-78: the same sign extension for signed storage words."""
    return _tir_packed_int_to_int_convert("int", storage_nbit)


def _tir_packed_uint_to_uint_to_float(storage_nbit: int):
    """quantization.py:56-65: u.astype(dtype) - (2**(nbit-1) - 1)."""
    storage_dtype = "uint" + str(storage_nbit)

    def f_convert(nbit: int, val, pos, dtype: str):
        return (_field(nbit, val, pos, storage_dtype) - ((1 << (nbit - 1)) - 1)).to(_DT[dtype])

    return f_convert


def _tir_packed_to_fp4_to_f16(storage_type="uint", storage_nbit=8):
    """quantization.py:142-157: 4-bit sign + 3-bit exponent -> fp16.  exponent 0 -> 0, otherwise the
    fp16 exponent field is e | 8, i.e. the value is +-2**(e - 7)."""
    storage_dtype = storage_type + str(storage_nbit)

    def f_convert(nbit: int, val, pos, dtype: str):
        assert nbit == 4 and dtype == "float16"
        f4 = _field(4, val, pos, storage_dtype)
        s, e = f4 >> 3, f4 & 7
        bits = (((e | 8) | (s << 5)) << 10).to(torch.int16)
        out = bits.view(torch.float16) if bits.dim() else bits.reshape(1).view(torch.float16).reshape(())
        return torch.where(e == 0, torch.zeros_like(out), out)

    return f_convert


def _tir_u8_to_f8_e4m3_to_f16(nbit: int, val, dtype: str):
    """quantization.py:170-177: bit-level e4m3 -> fp16 (exact for normal e4m3 values; like the
    reference's expression it does not special-case e4m3 subnormals or NaN)."""
    assert nbit == 8 and dtype == "float16"
    v = val.to(torch.int64) & 0xFF
    s = (v >> 7) << 15
    e4 = v & 0x40
    e = ((v & 63) << 7) | (e4 << 8) | (e4 << 7)
    bits = ((s | (e ^ 0x2000)) & 0xFFFF)
    bits = torch.where(bits >= 0x8000, bits - 0x10000, bits).to(torch.int16)
    return bits.view(torch.float16)
