"""Per-token x per-channel W8A8 GEMM.

Surface of examples/deepseek_v4/int8_gemm.py: ``int8_gemm_kernel_corrected(N, K, block_M=32,
block_N=32, block_K=32, in_dtype, out_dtype="float32", accum_dtype, scale_dtype)`` (:25-104)
-> ``kernel(A, B, scale_a, scale_b) -> C`` with ``out_idx=[-2]``, ``workspace_idx=[5]`` and a
symbolic M (:49).

    acc = A (int8 [M,K]) . B (int8 [N,K])^T                  int32, exact
    C   = rn_out( (f32(acc) * scale_a[m]) * scale_b[n] )     two fp32 multiplies in this order (:97-99)

``batched=True`` builds the same operator for A [Batch, M, K] with per-batch weights
B [Batch, K, N] and scale_a [Batch, M] (the shape of the quant_batch_matmul example with the
per-token x per-channel epilogue).
"""
from __future__ import annotations

from typing import Literal

from .. import _abi
from ..jit import ABI_DTYPE, TORCH_DTYPES, KernelSpec, Param, PassConfigKey, jit
from .quant_matmul import w8a8_launch

_PASS_CONFIGS = {
    PassConfigKey.TL_ASCEND_AUTO_SYNC: True,
    PassConfigKey.TL_ASCEND_AUTO_CV_SYNC: True,
    PassConfigKey.TIR_MERGE_STATIC_SMEM: True,
    PassConfigKey.TL_ASCEND_MEMORY_PLANNING: True,
}


@jit(out_idx=[-2], workspace_idx=[5], pass_configs=_PASS_CONFIGS)
def int8_gemm_kernel_corrected(N: int, K: int, block_M: int = 32, block_N: int = 32, block_K: int = 32,
                               in_dtype: Literal["int8"] = "int8",
                               out_dtype: Literal["float16", "bfloat16", "float32"] = "float32",
                               accum_dtype: Literal["int32"] = "int32",
                               scale_dtype: Literal["float32"] = "float32", tile: int = 0):
    """tile: rows per work-group of the int8 MFMA kernel (32, 128, 256; 0 = chosen by the library) -- the
    parameter an autotuner searches; the block sizes are recorded only."""
    if tile not in (0, 32, 128, 256):
        raise ValueError(f"tile must be one of 0, 32, 128, 256 (got {tile})")
    if in_dtype != "int8" or accum_dtype != "int32" or scale_dtype != "float32":
        raise ValueError("only int8 inputs, int32 accumulation and float32 scales are supported")
    tout = ABI_DTYPE[TORCH_DTYPES[out_dtype]]

    def launch(t, sym, stream):
        A, B, sa, sb, C, _ws = t
        with _abi.tuning(i8_tile=tile):
            w8a8_launch(A, B, sa, sb, C, 1, sym["M"], N, K, N, _abi.B_NK, tout, stream)

    return KernelSpec("int8_gemm_kernel_corrected",
                      [Param("A", ("M", K), in_dtype), Param("B", (N, K), in_dtype),
                       Param("scale_a", ("M",), scale_dtype), Param("scale_b", (N,), scale_dtype),
                       Param("C", ("M", N), out_dtype), Param("workspace_1", ("M", N), accum_dtype)], launch,
                      {"block": (block_M, block_N, block_K), "tile": tile})


@jit(out_idx=[-2], workspace_idx=[5], pass_configs=_PASS_CONFIGS)
def quant_batch_matmul_per_token(Batch: int, M: int, N: int, K: int, block_M: int = 128, block_N: int = 256,
                                 block_K: int = 64, out_dtype: Literal["float16", "bfloat16", "float32"] = "float16",
                                 tile: int = 0):
    """kernel(A [B,M,K] i8, W [B,K,N] i8, scale_token [B,M] f32, scale_channel [N] f32) -> C [B,M,N]:
    the batched layout of example_quant_batch_matmul.py:38-40 with the sequential two-scale
    epilogue of deepseek_v4/int8_gemm.py:97-99."""
    tout = ABI_DTYPE[TORCH_DTYPES[out_dtype]]

    def launch(t, sym, stream):
        A, B, sa, sb, C, _ws = t
        with _abi.tuning(i8_tile=tile):
            w8a8_launch(A, B, sa, sb, C, Batch, M, N, K, N, _abi.B_KN, tout, stream)

    return KernelSpec("quant_batch_matmul_per_token",
                      [Param("A", (Batch, M, K), "int8"), Param("B", (Batch, K, N), "int8"),
                       Param("scale_a", (Batch, M), "float32"), Param("scale_b", (N,), "float32"),
                       Param("C", (Batch, M, N), out_dtype), Param("workspace_1", (Batch, M, N), "int32")], launch,
                      {"block": (block_M, block_N, block_K), "tile": tile})
