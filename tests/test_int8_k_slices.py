"""K slices of the one-batch int8 kernels (few activation rows: too few output tiles to fill the machine).

tlq_gemm_w8a8_ws cuts K into slices that write int32 matrices into the workspace and sums + rescales them in a second
pass; tlq_gemm_i8 lets the slices add into C with atomic adds.  Integer sums are exact in any order, so every result
must equal the one-pass kernels' bit for bit, and both are checked against the exact-integer oracle.  The slices are
whole 128-byte stages and may be uneven (the last one holds what is left).
"""
import ctypes

import numpy as np
import pytest
import torch

from helpers import assert_bit_equal, gen
from oracle import cref


def _lib():
    from tilelang_ascend_amd import _abi

    return _abi, _abi.load(), _abi.ptr


# ---- host logic (no GPU) -----------------------------------------------------------------------------------------
def test_slice_choice_on_the_host():
    _abi, lib, _ = _lib()
    # few rows on few tiles: cut; many rows: one pass; K that is not whole stages: one pass
    assert lib.tlq_debug_i8_split(16, 4096, 4096, 1) > 1
    assert lib.tlq_debug_i8_split(16, 4096, 4096, 0) > 1
    assert lib.tlq_debug_i8_split(2048, 4096, 4096, 1) == 1
    assert lib.tlq_debug_i8_split(16, 4096, 4096 + 64, 1) == 1
    assert lib.tlq_debug_i8_split(16, 4096, 128, 1) == 1
    # atomic adds cost more than a matrix per slice: never more slices
    for M, N, K in ((16, 4096, 4096), (64, 8192, 8192), (128, 4096, 11008), (256, 5120, 13824)):
        assert lib.tlq_debug_i8_split(M, N, K, 0) <= lib.tlq_debug_i8_split(M, N, K, 1)
    # the workspace the library asks for is one int32 matrix per slice; nothing for several batches
    s = lib.tlq_debug_i8_split(32, 4096, 11008, 1)
    assert lib.tlq_w8a8_workspace_bytes(1, 32, 4096, 11008) == s * 32 * 4096 * 4
    assert lib.tlq_w8a8_workspace_bytes(4, 32, 4096, 11008) == 0
    assert lib.tlq_w8a8_workspace_bytes(1, 2048, 4096, 4096) == 0
    assert lib.tlq_w8a8_workspace_bytes(1, 0, 4096, 4096) == 0
    # a forced count is rounded to a cut that leaves no slice empty: 7 stages in 5 -> slices of 2 stages -> 4 slices
    lib.tlq_tune_i8_split(5)
    try:
        assert lib.tlq_debug_i8_split(16, 512, 128 * 7, 1) == 4
        assert lib.tlq_debug_i8_split(16, 512, 128 * 7, 0) == 4
        assert lib.tlq_debug_i8_split(16, 512, 128 * 2, 1) == 2  # never more slices than stages
    finally:
        lib.tlq_tune_i8_split(0)
    lib.tlq_tune_i8_split(1)
    try:
        assert lib.tlq_debug_i8_split(16, 4096, 4096, 1) == 1
        assert lib.tlq_w8a8_workspace_bytes(1, 16, 4096, 4096) == 0
    finally:
        lib.tlq_tune_i8_split(0)
    # a forced tile means that kernel, unsplit
    lib.tlq_tune_i8_tile(128)
    try:
        assert lib.tlq_debug_i8_split(16, 4096, 4096, 1) == 1
    finally:
        lib.tlq_tune_i8_tile(0)


# ---- GPU ------------------------------------------------------------------------------------------------------
# M ragged against the 32- and 128-row tiles, N ragged against the 128-column tile, K of 2 .. 108 stages
SHAPES = [(1, 256, 512), (16, 4096, 4096), (33, 400, 128 * 7), (5, 512, 384), (64, 1024, 1024), (200, 2064, 4096),
          (7, 11008, 4096), (32, 4096, 11008), (130, 1040, 128 * 13)]


def _run_i8(lib, _abi, P, A, W, M, N, K, lay, slices):
    lib.tlq_tune_i8_split(slices)
    try:
        C = torch.full((M, N), 7, dtype=torch.int32, device="cuda")  # stale contents must not survive
        _abi.check(lib.tlq_gemm_i8(P(A), P(W), P(C), 1, M, N, K, lay, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        return C.cpu()
    finally:
        lib.tlq_tune_i8_split(0)


@pytest.mark.gpu
@pytest.mark.parametrize("lay", [0, 1], ids=["KN", "NK"])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_int32_output_with_atomic_slices(M, N, K, lay):
    _abi, lib, P = _lib()
    g = gen(M + N + K + lay)
    A = torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=g)
    W = torch.randint(-128, 128, (K, N) if lay == _abi.B_KN else (N, K), dtype=torch.int8, generator=g)
    want = torch.from_numpy(cref.gemm_i8(A.numpy(), W.numpy(), lay))
    Ad, Wd = A.cuda(), W.cuda()
    for slices in (1, 0, 2, 3, 5, 64):
        got = _run_i8(lib, _abi, P, Ad, Wd, M, N, K, lay, slices)
        assert_bit_equal(got, want, f"int8 GEMM, {slices} slices asked, {M}x{N}x{K} layout {lay}")


@pytest.mark.gpu
@pytest.mark.parametrize("lay", [0, 1], ids=["KN", "NK"])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_rescaled_output_with_a_matrix_per_slice(M, N, K, lay):
    _abi, lib, P = _lib()
    g = gen(3 * M + N + K + lay)
    st = torch.cuda.current_stream().cuda_stream
    A = torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=g)
    W = torch.randint(-128, 128, (K, N) if lay == _abi.B_KN else (N, K), dtype=torch.int8, generator=g)
    sa = torch.rand(M, generator=g) * 0.04 + 0.01
    sb = torch.rand(N, generator=g) * 0.009 + 0.001
    acc = cref.gemm_i8(A.numpy(), W.numpy(), lay)
    Ad, Wd, sad, sbd = A.cuda(), W.cuda(), sa.cuda(), sb.cuda()
    ws = torch.full((64 * M * N,), 9, dtype=torch.int32, device="cuda")
    cases = [(torch.float16, _abi.F16, 0, sad, sbd, N), (torch.bfloat16, _abi.BF16, 1, None, sbd, N),
             (torch.float32, _abi.F32, 2, sad, sbd[:1].contiguous(), 1), (torch.float16, _abi.F16, 0, sad, None, N)]
    for dt, code, kind, a_s, b_s, nsb in cases:
        want_bits = cref.rescale(acc, None if a_s is None else sa.numpy(), None if b_s is None else sb.numpy()[:nsb], kind)
        want = torch.from_numpy(want_bits if kind == 2 else want_bits.view(np.int16).copy())
        one_pass = torch.empty(M, N, dtype=dt, device="cuda")
        _abi.check(lib.tlq_gemm_w8a8(P(Ad), P(Wd), P(a_s), P(b_s), P(one_pass), 1, M, N, K, nsb, lay, code, st))
        for slices in (0, 2, 3, 5, 64):
            lib.tlq_tune_i8_split(slices)
            try:
                C = torch.full((M, N), float("nan"), dtype=dt, device="cuda")
                _abi.check(lib.tlq_gemm_w8a8_ws(P(Ad), P(Wd), P(a_s), P(b_s), P(C), P(ws), ws.numel() * 4, 1, M, N, K, nsb,
                                                lay, code, st))
            finally:
                lib.tlq_tune_i8_split(0)
            torch.cuda.synchronize()
            what = f"W8A8 {dt} {slices} slices asked, {M}x{N}x{K} layout {lay}"
            assert_bit_equal(C.cpu(), one_pass.cpu(), what + " (against one pass)")
            got = C.cpu()
            assert_bit_equal(got if kind == 2 else got.view(torch.int16), want, what + " (against the oracle)")


@pytest.mark.gpu
def test_a_small_or_missing_workspace_means_fewer_slices_or_one_pass():
    _abi, lib, P = _lib()
    M, N, K = 16, 4096, 4096
    g = gen(77)
    st = torch.cuda.current_stream().cuda_stream
    A = torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=g).cuda()
    W = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=g).cuda()
    sb = (torch.rand(N, generator=g) * 0.01).cuda()
    want = torch.empty(M, N, dtype=torch.float16, device="cuda")
    _abi.check(lib.tlq_gemm_w8a8(P(A), P(W), None, P(sb), P(want), 1, M, N, K, N, _abi.B_NK, _abi.F16, st))
    full = lib.tlq_w8a8_workspace_bytes(1, M, N, K)
    assert full >= 2 * M * N * 4
    ws = torch.empty(full + 16, dtype=torch.uint8, device="cuda")
    for ptr, nbytes in ((P(ws), full), (P(ws), 2 * M * N * 4), (P(ws), M * N * 4), (P(ws), 100), (None, 0), (ctypes.c_void_p(ws.data_ptr() + 4), full)):
        C = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        _abi.check(lib.tlq_gemm_w8a8_ws(P(A), P(W), None, P(sb), P(C), ptr, nbytes, 1, M, N, K, N, _abi.B_NK, _abi.F16, st))
        torch.cuda.synchronize()
        assert_bit_equal(C.cpu(), want.cpu(), f"workspace of {nbytes} bytes")
    # several batches: one pass per batch, the workspace is not touched
    Ab = torch.randint(-128, 128, (3, M, K), dtype=torch.int8, generator=g).cuda()
    Wb = torch.randint(-128, 128, (3, N, K), dtype=torch.int8, generator=g).cuda()
    Cb = torch.empty(3, M, N, dtype=torch.float16, device="cuda")
    Cw = torch.empty(3, M, N, dtype=torch.float16, device="cuda")
    _abi.check(lib.tlq_gemm_w8a8(P(Ab), P(Wb), None, P(sb), P(Cb), 3, M, N, K, N, _abi.B_NK, _abi.F16, st))
    _abi.check(lib.tlq_gemm_w8a8_ws(P(Ab), P(Wb), None, P(sb), P(Cw), P(ws), full, 3, M, N, K, N, _abi.B_NK, _abi.F16, st))
    torch.cuda.synchronize()
    assert_bit_equal(Cw.cpu(), Cb.cpu(), "three batches")


@pytest.mark.gpu
def test_the_operators_take_the_sliced_path_for_few_rows():
    """simple_quant_matmul and int8_gemm_kernel_corrected on a decode-sized problem: the library asks for a workspace
    (so K is cut) and the operators' results equal the oracle's."""
    from oracle import ref
    from tilelang_ascend_amd import ops

    _abi, lib, _ = _lib()
    M, N, K = 24, 2048, 4096
    assert lib.tlq_w8a8_workspace_bytes(1, M, N, K) > 0
    g = gen(78)
    A = torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=g)
    B = torch.randint(-128, 128, (K, N), dtype=torch.int8, generator=g)
    scale = torch.randn(N, generator=g)
    got = ops.simple_quant_matmul(M, N, K, "N", 128, 256, 64, out_dtype="float16")(A.cuda(), B.cuda(), scale.cuda()).cpu()
    assert_bit_equal(got, ref.ref_program_quant(A[None], B[None], scale, torch.float16)[0], "simple_quant_matmul, few rows")
    Bnk = B.t().contiguous()
    sa = torch.rand(M, generator=g) * 0.04 + 0.01
    sb = torch.rand(N, generator=g) * 0.009 + 0.001
    kernel = ops.int8_gemm_kernel_corrected(N, K, out_dtype="bfloat16")
    got = kernel(A.cuda(), Bnk.cuda(), sa.cuda(), sb.cuda()).cpu()
    assert_bit_equal(got, ref.ref_int8_gemm_sequential(A, Bnk, sa, sb, torch.bfloat16), "int8_gemm_kernel_corrected, few rows")


@pytest.mark.gpu
@pytest.mark.parametrize("sign_mode", [0, 1, 2, 3])
@pytest.mark.parametrize("M,N,K", [(1, 260, 512), (16, 4096, 4096), (33, 400, 128 * 7), (200, 2048, 4096), (32, 1024, 11008)])
def test_packed_int4_weights_over_k_slices(M, N, K, sign_mode):
    """tlq_gemm_w4a8 (slices add into C) and tlq_gemm_w4a8_ws (a matrix per slice in the workspace) against the kernel
    without slices and against the exact integer product of the unpacked weights, for every sign convention."""
    from oracle import ref

    _abi, lib, P = _lib()
    g = gen(5 * M + N + K + sign_mode)
    st = torch.cuda.current_stream().cuda_stream
    A = torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=g)
    Wp = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=g)
    lo, hi = (Wp & 15).to(torch.int16), (Wp >> 4).to(torch.int16)
    u = torch.stack([lo, hi], dim=-1).reshape(N, K)
    vals = {0: u, 1: torch.where(u >= 8, u - 16, u), 2: u - 8, 3: u - 7}[sign_mode].to(torch.int8)
    want = ref.int_matmul_exact(A, vals.t().contiguous()).to(torch.int32)
    Ad, Wd = A.cuda(), Wp.cuda()
    ws = torch.empty(max(N * K, 64 * M * N * 4), dtype=torch.int8, device="cuda")
    for slices in (1, 0, 2, 3, 5, 64):
        lib.tlq_tune_i8_split(slices)
        lib.tlq_tune_w4a8_ws(1)
        try:
            C = torch.full((M, N), 7, dtype=torch.int32, device="cuda")
            _abi.check(lib.tlq_gemm_w4a8(P(Ad), P(Wd), P(C), M, N, K, sign_mode, st))
            D = torch.full((M, N), 7, dtype=torch.int32, device="cuda")
            _abi.check(lib.tlq_gemm_w4a8_ws(P(Ad), P(Wd), P(ws), ws.numel(), P(D), M, N, K, sign_mode, st))
        finally:
            lib.tlq_tune_i8_split(0)
            lib.tlq_tune_w4a8_ws(0)
        torch.cuda.synchronize()
        assert_bit_equal(C.cpu(), want, f"W4A8 sign mode {sign_mode}, {slices} slices asked, {M}x{N}x{K} (adds into C)")
        assert_bit_equal(D.cpu(), want, f"W4A8 sign mode {sign_mode}, {slices} slices asked, {M}x{N}x{K} (matrix per slice)")
