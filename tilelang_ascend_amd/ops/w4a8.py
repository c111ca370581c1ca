"""W4A8: int8 activations x packed signed-int4 weights -> int32.

Surface of examples/dequantize_gemm/example_dequant_gemm_w4a8.py: ``w4a8_gemm_cv(M, N, K)``
(:25-121) -> ``kernel(A, B_packed, workspace[, C]) -> C`` and ``torch_convert`` (:124-145).
The reference unpacks on the vector cores into a caller-supplied int8 [N, K] global workspace
and then runs the cube GEMM; so does this one from 257 activation rows on when the workspace
(third positional, as the reference's callers pass it) is a usable int8 [N, K] buffer: an unpack
kernel at the HBM roofline and the int8 GEMM, which together beat the kernel that unpacks on the
way into LDS.  With fewer rows the unpack pass would cost more than the GEMM: the fused kernel
runs over slices of K and keeps one int32 [M, N] matrix per slice in the workspace.
"""
from __future__ import annotations

import torch

from .. import _abi
from ..jit import KernelSpec, Param, PassConfigKey, jit
from .dequant_gemm import unpack_int4

PASS_CONFIGS = {
    PassConfigKey.TL_ASCEND_AUTO_SYNC: True,
    PassConfigKey.TL_ASCEND_AUTO_CV_SYNC: True,
    PassConfigKey.TL_ASCEND_AUTO_CV_COMBINE: True,
    PassConfigKey.TL_ASCEND_MEMORY_PLANNING: True,
}


@jit(out_idx=[-1], pass_configs=PASS_CONFIGS)
def w4a8_gemm_cv(M, N, K):
    """C[M,N] i32 = A[M,K] i8 . twos_complement_unpack(B_packed)[N,K]^T (exact)."""

    def launch(t, sym, stream):
        A, Bp, workspace, C = t
        ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None and workspace.is_contiguous() else 0
        _abi.check(_abi.load().tlq_gemm_w4a8_ws(_abi.ptr(A), _abi.ptr(Bp), _abi.ptr(workspace) if ws_bytes else None, ws_bytes,
                                                _abi.ptr(C), M, N, K, _abi.S4_TWOS, stream))

    return KernelSpec("w4a8_gemm_cv", [Param("A", (M, K), "int8"), Param("B_packed", (N, K // 2), "uint8"),
                                       Param("workspace", (N, K), "int8"), Param("C", (M, N), "int32")], launch)


def torch_convert(tensor: torch.Tensor) -> torch.Tensor:
    """example_dequant_gemm_w4a8.py:124-145: packed uint8 [N, K/2] -> int8 [N, K], each nibble
    sign-extended (two's complement), low nibble first.  Runs as a HIP kernel; CPU in -> CPU out."""
    assert tensor.dtype == torch.uint8
    if tensor.device.type == "cuda":
        return unpack_int4(tensor, torch.int8, "twos")
    return unpack_int4(tensor.cuda(), torch.int8, "twos").cpu()
