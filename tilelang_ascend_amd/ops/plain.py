"""Non-quantised twins of the quantised operators: plain GEMV, split-K GEMM and batched GEMM.

``batch_matmul(B, M, N, K, block_M, block_N, K_L1, dtype="float16", accum_dtype="float")`` ->
``kernel(A [B, M, K], B [B, K, N]) -> C [B, M, N]`` (examples/batch_gemm/batch_gemm.py:28-60, ``out_idx=[-1]``).

``simple_gemv(N, K, block_N, block_K, dtype="float16", accum_dtype="float32")`` ->
``kernel(x [K], A [N, K]) -> y [N]`` (examples/gemv/example_gemv_v.py:17-80 and example_gemv_c.py:16-46,
``out_idx=[-1]``, y = x @ A.T in `dtype`, accumulated in float32).

``gemm_splitk(M, N, K, block_M, block_N, block_K, split_k, dtype="float16", accum_dtype="float")`` ->
``kernel(A [M, K], B [K, N], C [M, N] float32)`` (examples/gemm_splitk/example_tilelang_gemm_splitk.py:16-48):
no output index -- C is accumulated in place by atomic adds and must be zeroed by the caller, as the example does.
"""
from __future__ import annotations

from .. import _abi
from ..jit import ABI_DTYPE, TORCH_DTYPES, KernelSpec, Param, PassConfigKey, jit

_DT = {"float16": "float16", "bfloat16": "bfloat16", "float32": "float32", "float": "float32"}


@jit(out_idx=[-1], pass_configs={PassConfigKey.TIR_MERGE_STATIC_SMEM: True, PassConfigKey.TL_ASCEND_AUTO_SYNC: True})
def simple_gemv(N: int, K: int, block_N: int, block_K: int, dtype: str = "float16", accum_dtype: str = "float32"):
    if dtype not in _DT or _DT[accum_dtype] != "float32":
        raise ValueError("dtype must be float16, bfloat16 or float32 and accum_dtype float32")
    dt = _DT[dtype]
    code = ABI_DTYPE[TORCH_DTYPES[dt]]

    def launch(t, sym, stream):
        x, A, y = t
        _abi.check(_abi.load().tlq_gemv(_abi.ptr(x), _abi.ptr(A), _abi.ptr(y), N, K, code, code, stream))

    return KernelSpec("simple_gemv", [Param("x", (K,), dt), Param("A", (N, K), dt), Param("y", (N,), dt)], launch,
                      {"block": (block_N, block_K)})


@jit(pass_configs={PassConfigKey.TL_ASCEND_AUTO_SYNC: True, PassConfigKey.TL_ASCEND_MEMORY_PLANNING: True})
def gemm_splitk(M: int, N: int, K: int, block_M: int, block_N: int, block_K: int, split_k: int,
                dtype: str = "float16", accum_dtype: str = "float"):
    if dtype not in ("float16", "bfloat16") or _DT[accum_dtype] != "float32":
        raise ValueError("dtype must be float16 or bfloat16 and accum_dtype float")
    if split_k < 1 or K % split_k:
        raise ValueError(f"split_k={split_k} must divide K={K}")
    code = ABI_DTYPE[TORCH_DTYPES[dtype]]

    def launch(t, sym, stream):
        A, B, C = t
        _abi.check(_abi.load().tlq_gemm_f16_splitk(_abi.ptr(A), _abi.ptr(B), _abi.ptr(C), M, N, K, split_k, code, _abi.B_KN,
                                                   stream))

    return KernelSpec("gemm_splitk", [Param("A", (M, K), dtype), Param("B", (K, N), dtype), Param("C", (M, N), "float32")],
                      launch, {"block": (block_M, block_N, block_K), "split_k": split_k})


@jit(out_idx=[-1], pass_configs={PassConfigKey.TL_ASCEND_AUTO_CV_COMBINE: True, PassConfigKey.TL_ASCEND_AUTO_SYNC: True,
                                 PassConfigKey.TL_ASCEND_MEMORY_PLANNING: True})
def batch_matmul(B: int, M: int, N: int, K: int, block_M: int, block_N: int, K_L1: int, dtype: str = "float16",
                 accum_dtype: str = "float"):
    """examples/batch_gemm/batch_gemm.py:28-60: C[b] = A[b] @ B[b] in `dtype`, accumulated in float32, one launch for
    the whole batch.  The block sizes are accepted and recorded; tiling is chosen by the library."""
    if dtype not in ("float16", "bfloat16") or _DT[accum_dtype] != "float32":
        raise ValueError("dtype must be float16 or bfloat16 and accum_dtype float")
    code = ABI_DTYPE[TORCH_DTYPES[dtype]]

    def launch(t, sym, stream):
        A, Bm, C = t
        _abi.check(_abi.load().tlq_gemm_f16_batched(_abi.ptr(A), _abi.ptr(Bm), _abi.ptr(C), B, M, N, K, code, code, _abi.B_KN,
                                                    stream))

    return KernelSpec("batch_matmul", [Param("A_mat", (B, M, K), dtype), Param("B_mat", (B, K, N), dtype),
                                       Param("C_mat", (B, M, N), dtype)], launch, {"block": (block_M, block_N, K_L1)})
