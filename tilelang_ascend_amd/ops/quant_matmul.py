"""W8A8 matmul with fused rescale epilogue.

Surface of examples/quant_batch_matmul/example_quant_batch_matmul.py (``simple_quant_batch_matmul``,
:8-91) and example_quant_matmul.py (``simple_quant_matmul``, :8-90): ``kernel(A, B, scale) -> C``
with ``out_idx=[3]`` and an int32 ``workspace_1`` at ``workspace_idx=[4]``.

    acc = A[b] (int8 [M,K]) . B[b] (int8 [K,N])            int32, exact
    C   = rn_out( f32(acc) * scale[n or 0] )               CAST_RINT = round to nearest even

The reference writes acc to the global workspace and re-reads it on the vector cores
(:66-68); here the rescale runs on the MFMA accumulators.  Only with one batch and few
activation rows, where the output tiles are too few to fill the machine, K is cut into
slices that write int32 matrices into a workspace and a second pass sums and rescales
them (``w8a8_launch``) -- the same values bit for bit.
"""
from __future__ import annotations

from typing import Literal

import torch

from .. import _abi
from ..jit import ABI_DTYPE, TORCH_DTYPES, KernelSpec, Param, PassConfigKey, jit

_PASS_CONFIGS = {
    PassConfigKey.TL_ASCEND_AUTO_SYNC: True,
    PassConfigKey.TL_ASCEND_AUTO_CV_SYNC: True,
    PassConfigKey.TL_ASCEND_AUTO_CV_COMBINE: True,
}


def _check_types(scale_size, in_dtype, out_dtype, accum_dtype, scale_dtype):
    if scale_size not in ("1", "N"):
        raise ValueError(f'scale_size must be "1" or "N", got {scale_size!r}')
    if in_dtype != "int8" or accum_dtype != "int32" or scale_dtype != "float32":
        raise ValueError("only int8 inputs, int32 accumulation and float32 scales are supported")
    if out_dtype not in ("float16", "bfloat16", "float32"):
        raise ValueError(f"out_dtype must be float16, bfloat16 or float32, got {out_dtype}")


def w8a8_launch(A, B, scale_a, scale_b, C, batch, M, N, K, n_scale_b, b_layout, out_code, stream):
    """One W8A8 launch with the int32 workspace the library asks for (the reference's workspace_idx buffer,
    example_quant_batch_matmul.py:28,42): allocated per call on A's device like the reference's, and only where the
    library cuts K into slices (one batch, few activation rows); otherwise the rescale stays fused and nothing is
    allocated."""
    lib = _abi.load()
    ws_bytes = lib.tlq_w8a8_workspace_bytes(batch, M, N, K)
    ws = _abi.scratch(ws_bytes, A.device, stream)
    _abi.check(lib.tlq_gemm_w8a8_ws(_abi.ptr(A), _abi.ptr(B), _abi.ptr(scale_a), _abi.ptr(scale_b), _abi.ptr(C), _abi.ptr(ws),
                                    ws_bytes, batch, M, N, K, n_scale_b, b_layout, out_code, stream))


@jit(out_idx=[3], workspace_idx=[4], pass_configs=_PASS_CONFIGS)
def simple_quant_batch_matmul(Batch: int, M: int, N: int, K: int, scale_size: Literal["1", "N"],
                              block_M: int, block_N: int, block_K: int,
                              in_dtype: Literal["int8"] = "int8",
                              out_dtype: Literal["float16", "bfloat16"] = "float16",
                              accum_dtype: Literal["int32"] = "int32",
                              scale_dtype: Literal["float32"] = "float32"):
    """Simple QuantMatmul with per-tensor / per-channel quantization scale (batched)."""
    _check_types(scale_size, in_dtype, out_dtype, accum_dtype, scale_dtype)
    N_scale = N if scale_size == "N" else 1
    tout = ABI_DTYPE[TORCH_DTYPES[out_dtype]]

    def launch(t, sym, stream):
        A, B, scale, C, _ws = t
        w8a8_launch(A, B, None, scale, C, Batch, M, N, K, N_scale, _abi.B_KN, tout, stream)

    return KernelSpec("simple_quant_batch_matmul",
                      [Param("A", (Batch, M, K), in_dtype), Param("B", (Batch, K, N), in_dtype),
                       Param("scale", (N_scale,), scale_dtype), Param("C", (Batch, M, N), out_dtype),
                       Param("workspace_1", (Batch, M, N), accum_dtype)], launch,
                      {"block": (block_M, block_N, block_K), "scale_size": scale_size})


@jit(out_idx=[3], workspace_idx=[4], pass_configs=_PASS_CONFIGS)
def simple_quant_matmul(M: int, N: int, K: int, scale_size: Literal["1", "N"],
                        block_M: int, block_N: int, block_K: int,
                        in_dtype: Literal["int8"] = "int8",
                        out_dtype: Literal["float16", "bfloat16"] = "float16",
                        accum_dtype: Literal["int32"] = "int32",
                        scale_dtype: Literal["float32"] = "float32"):
    """2-D twin (example_quant_matmul.py:8-90)."""
    _check_types(scale_size, in_dtype, out_dtype, accum_dtype, scale_dtype)
    N_scale = N if scale_size == "N" else 1
    tout = ABI_DTYPE[TORCH_DTYPES[out_dtype]]

    def launch(t, sym, stream):
        A, B, scale, C, _ws = t
        w8a8_launch(A, B, None, scale, C, 1, M, N, K, N_scale, _abi.B_KN, tout, stream)

    return KernelSpec("simple_quant_matmul",
                      [Param("A", (M, K), in_dtype), Param("B", (K, N), in_dtype),
                       Param("scale", (N_scale,), scale_dtype), Param("C", (M, N), out_dtype),
                       Param("workspace_1", (M, N), accum_dtype)], launch,
                      {"block": (block_M, block_N, block_K), "scale_size": scale_size})
