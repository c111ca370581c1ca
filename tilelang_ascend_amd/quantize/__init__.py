"""Weight (de)quantisation helpers with the import surface of tilelang/quantize/__init__.py:3-18."""
from .lop3 import get_lop3_intrin_group  # noqa: F401
from .quantization import (  # noqa: F401
    _tir_packed_int_to_int_convert,
    _tir_packed_int_to_int_to_float,
    _tir_packed_to_fp4_to_f16,
    _tir_packed_to_signed_convert,
    _tir_packed_to_unsigned_convert,
    _tir_packed_to_unsigned_convert_with_zeros,
    _tir_packed_uint_to_uint_to_float,
    _tir_u8_to_f8_e4m3_to_f16,
)
from .utils import gen_quant4, general_compress, interleave_weight  # noqa: F401
from .pack_io import load_packed, save_packed  # noqa: F401  (no counterpart in the reference: the on-disk form of repacked weights)
