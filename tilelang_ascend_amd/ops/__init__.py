"""Operator factories with the names, argument order and defaults of the reference's example
scripts (examples/dequantize_gemm, examples/quant_batch_matmul, examples/deepseek_v4/int8_gemm.py,
examples/deepseek_v4/act_quant.py, examples/gemv, examples/gemm_splitk, examples/batch_gemm)."""
from .act_quant import act_quant_kernel_int8_optimized  # noqa: F401
from .dequant_gemm import (  # noqa: F401
    dequant_gemm_fp16_wrapper,
    dequant_gemm_int8_wrapper,
    dequantize_w4,
    fp16_gemm,
    int8_gemm,
    torch_unpack_uint4_to_fp16,
    torch_unpack_uint4_to_int8,
    unpack_int4,
    w4a16_gemm,
)
from .int8_per_token import int8_gemm_kernel_corrected, quant_batch_matmul_per_token  # noqa: F401
from .plain import batch_matmul, gemm_splitk, simple_gemv  # noqa: F401
from .quant_matmul import simple_quant_batch_matmul, simple_quant_matmul  # noqa: F401
from .w4a8 import torch_convert, w4a8_gemm_cv  # noqa: F401
