"""Weight-only int4 dequant GEMM / GEMV operators.

Surface of examples/dequantize_gemm/example_dequant_gemm_fine_grained.py: ``fp16_gemm`` (:60-115),
``int8_gemm`` (:118-173), ``dequant_gemm_fp16_wrapper`` (:176-223), ``dequant_gemm_int8_wrapper``
(:226-266) and the two unpack helpers (:10-57), same names and argument order.  The reference
unpacks on the host in Python and runs a plain GEMM on 4x larger weights; here unpack, per-group
scale / zero and the GEMM are one HIP kernel, and the unpack helpers are HIP kernels too.

Extension the reference's example does not have: per-group ``scales`` / ``zeros``
(``tilelang.quantize`` semantics, W = (u - z) * s with one rounding per operation), passed as
additional trailing arguments so that ``wrapper(A, B_packed)`` keeps its meaning.
"""
from __future__ import annotations

from typing import Optional, Union

import torch

from .. import _abi
from ..jit import ABI_DTYPE, TORCH_DTYPES, KernelSpec, Param, PassConfigKey, jit

_PASS_CONFIGS = {
    PassConfigKey.TL_ASCEND_AUTO_CV_COMBINE: True,
    PassConfigKey.TL_ASCEND_AUTO_SYNC: True,
    PassConfigKey.TL_ASCEND_MEMORY_PLANNING: True,
    PassConfigKey.TL_ASCEND_AUTO_CV_SYNC: True,
}
_SIGN_MODES = {"unsigned": _abi.U4, "twos": _abi.S4_TWOS, "offset8": _abi.S4_OFFSET8, "offset7": _abi.S4_OFFSET7}
_ALGOS = {"auto": _abi.ALGO_AUTO, "gemv": _abi.ALGO_GEMV, "mfma": _abi.ALGO_MFMA, "skinny": _abi.ALGO_SKINNY,
          "two_pass": _abi.ALGO_TWO_PASS, "stream": _abi.ALGO_STREAM, "decode": _abi.ALGO_DECODE, "panel": _abi.ALGO_PANEL, "panel256": _abi.ALGO_PANEL256, "panelm": _abi.ALGO_PANELM}
# arrangement of the 4-bit fields in each 32-bit word: general_compress order, or interleave_weight(target float16)
_LAYOUTS = {"plain": _abi.W_PLAIN, "interleaved": _abi.W_INTERLEAVED_F16}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _require_cuda(t: torch.Tensor, what: str) -> None:
    if t.device.type != "cuda":
        raise ValueError(f"{what} must be on a ROCm device (torch device 'cuda'), got {t.device}")


# ------------------------------------------------------------------------------------------
# unpack / dequant helpers (device tensors in, device tensors out)
# ------------------------------------------------------------------------------------------
def unpack_int4(tensor: torch.Tensor, out_dtype: torch.dtype = torch.int8, sign_mode: str = "unsigned") -> torch.Tensor:
    """uint8 [N, K/2] -> [N, K] of out_dtype (int8 / float16 / bfloat16).  Element k of row n is
    nibble k % 2 of byte k // 2, low nibble first.  sign_mode: 'unsigned' (0..15), 'twos'
    (two's complement -8..7), 'offset8' (u-8), 'offset7' (u-7)."""
    if tensor.dtype != torch.uint8 or tensor.dim() != 2:
        raise ValueError(f"packed weights must be a 2-D uint8 tensor, got {tensor.dtype} {tuple(tensor.shape)}")
    if not tensor.is_contiguous():
        raise ValueError("Input tensor at index 0 must be contiguous")
    _require_cuda(tensor, "packed weights")
    N, Kp = tensor.shape
    out = torch.empty(N, Kp * 2, dtype=out_dtype, device=tensor.device)
    with torch.cuda.device(tensor.device):
        _abi.check(_abi.load().tlq_unpack_int4(_abi.ptr(tensor), _abi.ptr(out), N, Kp * 2, ABI_DTYPE[out_dtype],
                                               _SIGN_MODES[sign_mode], _stream()))
    return out


def torch_unpack_uint4_to_fp16(tensor: torch.Tensor) -> torch.Tensor:
    """Same contract as the reference helper (fine_grained.py:10-32): uint8 [N, K/2] -> float16
    [N, K] with values 0..15.  CPU tensor in -> CPU tensor out; the work runs on the GPU."""
    assert tensor.dtype == torch.uint8
    if tensor.device.type == "cuda":
        return unpack_int4(tensor, torch.float16)
    return unpack_int4(tensor.cuda(), torch.float16).cpu()


def torch_unpack_uint4_to_int8(tensor: torch.Tensor) -> torch.Tensor:
    """fine_grained.py:35-57: uint8 [N, K/2] -> int8 [N, K], values 0..15."""
    assert tensor.dtype == torch.uint8
    if tensor.device.type == "cuda":
        return unpack_int4(tensor, torch.int8)
    return unpack_int4(tensor.cuda(), torch.int8).cpu()


def dequantize_w4(B_packed: torch.Tensor, scales: Optional[torch.Tensor] = None,
                  zeros: Union[None, float, int, torch.Tensor] = None, group_size: int = 128,
                  dtype: torch.dtype = torch.float16, weight_layout: str = "plain") -> torch.Tensor:
    """W[n, k] = rn( rn(T(u[n,k]) - z[n, k//g]) * s[n, k//g] ), T = dtype, as a [N, K] tensor.
    scales: [N, K/g] of dtype or None (=1).  zeros: None (=0), a number, or [N, K/g] of dtype.
    weight_layout: "plain", or "interleaved" for words repacked by interleave_weight(target float16)."""
    _require_cuda(B_packed, "B_packed")
    N, Kp = B_packed.shape
    K = Kp * 2
    z_t, z_s = _split_zero(zeros)
    _check_group_tensor(scales, "scales", N, K, group_size, dtype)
    _check_group_tensor(z_t, "zeros", N, K, group_size, dtype)
    out = torch.empty(N, K, dtype=dtype, device=B_packed.device)
    with torch.cuda.device(B_packed.device):
        _abi.check(_abi.load().tlq_dequant_w4_layout(_abi.ptr(B_packed), _abi.ptr(scales), _abi.ptr(z_t), _abi.ptr(out), N, K,
                                                     group_size, float(z_s), ABI_DTYPE[dtype], _LAYOUTS[weight_layout],
                                                     _stream()))
    return out


def _split_zero(zeros):
    if zeros is None:
        return None, 0.0
    if isinstance(zeros, torch.Tensor):
        return zeros, 0.0
    return None, float(zeros)


def _check_group_tensor(t, name, N, K, group, dtype):
    if t is None:
        return
    if t.dtype != dtype:
        raise ValueError(f"Buffer dtype mismatch for parameter {name}: expected {dtype}, got {t.dtype}")
    if tuple(t.shape) != (N, K // group):
        raise ValueError(f"Static shape mismatch for parameter {name}: expected {(N, K // group)}, got {tuple(t.shape)}")
    if not t.is_contiguous():
        raise ValueError(f"Input tensor {name} must be contiguous")
    _require_cuda(t, name)


# ------------------------------------------------------------------------------------------
# plain GEMMs of the reference example
# ------------------------------------------------------------------------------------------
@jit(out_idx=[-1], pass_configs=_PASS_CONFIGS)
def fp16_gemm(M: int, N: int, K: int, block_M: int, block_N: int, block_K: int):
    """fine_grained.py:60-115: C[M,N] f16 = A[M,K] f16 . B[K,N] f16, fp32 accumulate.  The block
    sizes are accepted for signature compatibility; tiling is chosen by the library."""

    def launch(t, sym, stream):
        A, B, C = t
        lib = _abi.load()
        # few activation rows: K slices with their fp32 matrices in a workspace (allocated per call, like the
        # reference's workspace_idx buffers); 0 bytes for every other shape
        ws_bytes = lib.tlq_f16_workspace_bytes(1, M, N, K)
        ws = _abi.scratch(ws_bytes, A.device, stream)
        _abi.check(lib.tlq_gemm_f16_ws(_abi.ptr(A), _abi.ptr(B), _abi.ptr(C), _abi.ptr(ws), ws_bytes, 1, M, N, K, _abi.F16,
                                       _abi.F16, _abi.B_KN, stream))

    return KernelSpec("fp16_gemm", [Param("A", (M, K), "float16"), Param("B", (K, N), "float16"),
                                    Param("C", (M, N), "float16")], launch,
                      {"block": (block_M, block_N, block_K)})


@jit(out_idx=[-1], pass_configs=_PASS_CONFIGS)
def int8_gemm(M: int, N: int, K: int, block_M: int, block_N: int, block_K: int):
    """fine_grained.py:118-173: C[M,N] i32 = A[M,K] i8 . B[K,N] i8, int32 accumulate (exact)."""

    def launch(t, sym, stream):
        A, B, C = t
        _abi.check(_abi.load().tlq_gemm_i8(_abi.ptr(A), _abi.ptr(B), _abi.ptr(C), 1, M, N, K, _abi.B_KN, stream))

    return KernelSpec("int8_gemm", [Param("A", (M, K), "int8"), Param("B", (K, N), "int8"),
                                    Param("C", (M, N), "int32")], launch,
                      {"block": (block_M, block_N, block_K)})


# ------------------------------------------------------------------------------------------
# fused W4A16
# ------------------------------------------------------------------------------------------
@jit(out_idx=[-1], pass_configs=_PASS_CONFIGS)
def w4a16_gemm(M: int, N: int, K: int, block_M: int = 128, block_N: int = 256, block_K: int = 64,
               in_dtype: str = "float16", out_dtype: str = "float16", group_size: int = 128,
               with_scales: bool = True, zeros: Union[None, float, int, str] = None, algo: str = "auto",
               tile: int = 0, gemv_tuning: tuple = None, skinny_tuning: tuple = None, weight_layout: str = "plain"):
    """Device-resident fused kernel: kernel(A, B_packed[, scales][, zeros]) -> C.

    A [M,K] in_dtype; B_packed uint8 [N,K/2]; scales [N,K/group_size] in_dtype when with_scales;
    zeros: None (no zero point), a number (one zero point for the whole matrix) or "tensor"
    (a [N,K/group_size] in_dtype input follows).  C [M,N] out_dtype, fp32 accumulate.
    algo: "auto" | "gemv" (split-K wavefront kernel, M <= 16) | "decode" (M <= 32, K % 256 == 0: persistent work-groups with the
    activations in registers: what "auto" does for 3 <= M <= 16) | "skinny" (M <= 64) | "mfma" (LDS-staged MFMA kernel)
    | "stream" (wavefront-private packed weights dequantised in registers, 17 <= M <= 512: what "auto" does up to
    M = 384) | "panel" (large M in one launch: packed weights copied to LDS as they are and dequantised on the MFMA operand
    read; what "auto" does from 513 to 2048 rows where its work-groups fill the machine) | "two_pass" (dequantise into a
    workspace, then the plain GEMM: what "auto" does otherwise above 512 rows).  "auto" first consults the library's table
    of tuned choices (autotuner.tune_w4a16_choice; the device's persisted choices are installed on the first launch unless
    TLQ_TUNED_CHOICES=0).  A workspace
    (split-K partial sums or the [N, K] dequantised weights) is taken from torch's stream-ordered allocator on every
    call, as the reference allocates its workspace_idx buffers per call, so launches on different streams do not share one;
    when the launch stream (forward(stream=...)) is not torch's current stream the block is recorded on it (_abi.scratch).
    weight_layout: "plain" (general_compress order) or "interleaved" (B_packed went through interleave_weight for the
    float16 target, e.g. quantize.gpu.pack_int4(..., interleave="float16")); interleaved weights are read by the "gemv" (one row,
    two fp16 rows), "decode", "stream" and panel kernels and the two passes, with results bit-identical to the plain layout
    (the GEMV: to the rounding of its fp32 sums).
    tile: rows of activations per work-group of the MFMA kernel (16, 32, 64, 128, 256; 0 = chosen by the
    library); gemv_tuning = (rows_per_wave, waves, blocks_per_cu, depth) and skinny_tuning = (waves,
    row_tiles) select among the pre-built variants of those kernels.  These are the tunable parameters an
    autotuner searches (the role of block_M / block_N / block_K in the reference, which are accepted and
    recorded but do not select a tiling here)."""
    if tile not in (0, 16, 32, 64, 128, 256):
        raise ValueError(f"tile must be one of 0, 16, 32, 64, 128, 256 (got {tile})")
    if in_dtype not in ("float16", "bfloat16"):
        raise ValueError(f"in_dtype must be float16 or bfloat16, got {in_dtype}")
    if out_dtype not in ("float16", "bfloat16", "float32"):
        raise ValueError(f"out_dtype must be float16, bfloat16 or float32, got {out_dtype}")
    zeros_tensor = isinstance(zeros, str)
    if zeros_tensor and zeros != "tensor":
        raise ValueError('zeros must be None, a number or "tensor"')
    zero_scalar = 0.0 if (zeros is None or zeros_tensor) else float(zeros)
    G = K // group_size
    params = [Param("A", (M, K), in_dtype), Param("B_packed", (N, K // 2), "uint8")]
    if with_scales:
        params.append(Param("scales", (N, G), in_dtype))
    if zeros_tensor:
        params.append(Param("zeros", (N, G), in_dtype))
    params.append(Param("C", (M, N), out_dtype))
    tin, tout = ABI_DTYPE[TORCH_DTYPES[in_dtype]], ABI_DTYPE[TORCH_DTYPES[out_dtype]]
    algo_code = _ALGOS[algo]
    layout_code = _LAYOUTS[weight_layout]

    def launch(t, sym, stream):
        A, Bp = t[0], t[1]
        i = 2
        S = Z = None
        if with_scales:
            S = t[i]
            i += 1
        if zeros_tensor:
            Z = t[i]
            i += 1
        C = t[i]
        lib = _abi.load()
        ws = None
        if algo == "auto":
            from ..autotuner import ensure_w4a16_choices_loaded
            ensure_w4a16_choices_loaded()  # (once per process: the device's persisted tuned choices, if any)
        # what the named family asks for ("auto": the rule-based choice and any tuned choice for this shape)
        ws_bytes = lib.tlq_w4a16_workspace_bytes_for(M, N, K, algo_code)
        if layout_code != _abi.W_PLAIN and algo == "auto" and M > 256:
            ws_bytes = max(ws_bytes, N * K * 2)
        if ws_bytes:
            ws = _abi.scratch(ws_bytes, A.device, stream)
        with _abi.tuning(w4a16_tile=tile, gemv=gemv_tuning, skinny=skinny_tuning):
            _abi.check(lib.tlq_gemm_w4a16_layout_ws(_abi.ptr(A), _abi.ptr(Bp), _abi.ptr(S), _abi.ptr(Z), _abi.ptr(C), M, N, K,
                                                    group_size, zero_scalar, tin, tout, algo_code, layout_code, _abi.ptr(ws),
                                                    ws_bytes, stream))

    return KernelSpec("w4a16_gemm", params, launch,
                      {"block": (block_M, block_N, block_K), "group": group_size, "zeros": zeros, "algo": algo,
                       "tile": tile, "gemv_tuning": gemv_tuning, "skinny_tuning": skinny_tuning,
                       "weight_layout": weight_layout})


def dequant_gemm_fp16_wrapper(M: int, N: int, K: int, block_M: int, block_N: int, block_K: int,
                              input_dtype: str = "float16", output_dtype: str = "float16",
                              group_size: int = 128, algo: str = "auto", weight_layout: str = "plain"):
    """fine_grained.py:176-223: returns wrapper(A, B_packed) -> C = A @ unpack(B_packed).T.

    As in the reference the wrapper takes CPU tensors and returns a CPU tensor (it moves data to
    the device itself, :218-220); device tensors are accepted too and then the result stays on
    the device.  Unlike the reference, bfloat16 activations are NOT down-cast to float16
    (:211-214): the kernel multiplies in bfloat16 like the reference's own oracle (:283).
    Extension: wrapper(A, B_packed, scales=None, zeros=None) with per-group scales [N, K/group_size]
    and zeros (number or [N, K/group_size] tensor), W = (u - z) * s."""
    if output_dtype not in ("float16", "bfloat16", "float32"):
        raise KeyError(output_dtype)
    kernels = {}

    def wrapper(A: torch.Tensor, B_packed: torch.Tensor, scales: Optional[torch.Tensor] = None,
                zeros: Union[None, float, int, torch.Tensor] = None):
        on_cpu = A.device.type != "cuda"
        z_is_tensor = isinstance(zeros, torch.Tensor)
        key = (scales is not None, "tensor" if z_is_tensor else zeros)
        if key not in kernels:
            kernels[key] = w4a16_gemm(M, N, K, block_M, block_N, block_K, input_dtype, output_dtype, group_size,
                                      scales is not None, key[1], algo, weight_layout=weight_layout)
        args = [A, B_packed] + ([scales] if scales is not None else []) + ([zeros] if z_is_tensor else [])
        if on_cpu:
            args = [a.cuda() for a in args]
        C = kernels[key](*args)
        return C.cpu() if on_cpu else C

    return wrapper


def dequant_gemm_int8_wrapper(M: int, N: int, K: int, block_M: int, block_N: int, block_K: int,
                              output_dtype: str = "int32"):
    """fine_grained.py:226-266: wrapper(A int8 [M,K], B_packed uint8 [N,K/2]) ->
    (A.i32 @ unpack_unsigned(B_packed).i32.T).to(output_dtype); int32 accumulation is exact.
    The unpack is fused into the int8 MFMA kernel."""
    out_t = {"int32": torch.int32, "float16": torch.float16, "bfloat16": torch.bfloat16}[output_dtype]
    kernel = _w4a8_kernel(M, N, K, "unsigned")

    def wrapper(A: torch.Tensor, B_packed: torch.Tensor):
        on_cpu = A.device.type != "cuda"
        C = kernel(A.cuda() if on_cpu else A, B_packed.cuda() if on_cpu else B_packed)
        C = C.cpu() if on_cpu else C
        return C.to(out_t)

    return wrapper


@jit(out_idx=[-1], pass_configs=_PASS_CONFIGS)
def _w4a8_kernel(M: int, N: int, K: int, sign_mode: str):
    mode = _SIGN_MODES[sign_mode]

    def launch(t, sym, stream):
        A, Bp, C = t
        _abi.check(_abi.load().tlq_gemm_w4a8(_abi.ptr(A), _abi.ptr(Bp), _abi.ptr(C), M, N, K, mode, stream))

    return KernelSpec("w4a8_gemm", [Param("A", (M, K), "int8"), Param("B_packed", (N, K // 2), "uint8"),
                                    Param("C", (M, N), "int32")], launch, {"sign": sign_mode})
