"""K slices of the plain 16-bit GEMM (tlq_gemm_f16_ws: one batch, few activation rows).

Every slice of K writes its fp32 tile into its own [M,N] matrix in the workspace and a second pass adds the matrices in
slice order and rounds once: the result is deterministic and meets the float bar against an fp32 product; with no (or
too small a) workspace the call is tlq_gemm_f16, bit for bit.  The two passes of the W4A16 entry point run their
second pass this way when the workspace has room beyond the dequantised matrix.
"""
import pytest
import torch

from helpers import DT, assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference


def _lib():
    from tilelang_ascend_amd import _abi

    return _abi, _abi.load(), _abi.ptr


def test_slice_choice_on_the_host():
    _abi, lib, _ = _lib()
    assert lib.tlq_debug_f16_split(16, 4096, 4096) > 1
    assert lib.tlq_debug_f16_split(4096, 4096, 4096) == 1   # enough output tiles
    assert lib.tlq_debug_f16_split(16, 4096, 4096 + 8) == 1  # K is not whole 128-byte stages
    assert lib.tlq_debug_f16_split(16, 4096, 64) == 1        # one stage
    s = lib.tlq_debug_f16_split(64, 4096, 11008)
    assert s > 1 and lib.tlq_f16_workspace_bytes(1, 64, 4096, 11008) == s * 64 * 4096 * 4
    assert lib.tlq_f16_workspace_bytes(2, 64, 4096, 11008) == 0  # several batches fill the machine by themselves
    assert lib.tlq_f16_workspace_bytes(1, 64, 4100, 11008) == 0  # N % 8 != 0 is not a shape of the GEMM
    lib.tlq_tune_f16_split(5)
    try:
        assert lib.tlq_debug_f16_split(16, 512, 64 * 7) == 4  # 7 stages in 5 -> slices of 2 stages -> 4 slices
    finally:
        lib.tlq_tune_f16_split(0)
    lib.tlq_tune_f16_split(1)
    try:
        assert lib.tlq_f16_workspace_bytes(1, 16, 4096, 4096) == 0
    finally:
        lib.tlq_tune_f16_split(0)
    # the W4A16 workspace: the dequantised matrix plus the slices of its plain GEMM
    # (K = 43 x 64 has no equal cut for the fused tile kernel, so M = 300 takes the two passes)
    # (and, K being no power of two, room for one scale and one zero point per weight row written out per group of 64)
    assert lib.tlq_w4a16_workspace_bytes(300, 256, 2752) == (256 * 2752 * 2 + lib.tlq_f16_workspace_bytes(1, 300, 256, 2752)
                                                             + 2 * 256 * 43 * 2 + 16)
    assert lib.tlq_f16_workspace_bytes(1, 300, 256, 2752) > 0


SHAPES = [(1, 264, 512), (16, 4096, 4096), (33, 1024, 11008), (200, 2048, 4096), (40, 520, 64 * 7), (130, 1032, 64 * 13)]


@pytest.mark.gpu
@pytest.mark.parametrize("in_dtype,out_dtype", [("float16", "float16"), ("bfloat16", "bfloat16"), ("float16", "float32")])
@pytest.mark.parametrize("lay", [0, 1], ids=["KN", "NK"])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_sliced_gemm_against_an_fp32_product(M, N, K, lay, in_dtype, out_dtype):
    _abi, lib, P = _lib()
    dt, odt = DT[in_dtype], DT[out_dtype]
    code = {torch.float16: _abi.F16, torch.bfloat16: _abi.BF16, torch.float32: _abi.F32}
    st = torch.cuda.current_stream().cuda_stream
    A = torch.randn(M, K, generator=gen(M + K)).to(dt)
    W = torch.randn((K, N) if lay == _abi.B_KN else (N, K), generator=gen(N + K + lay)).to(dt)
    want = A.float() @ (W.float() if lay == _abi.B_KN else W.float().t())
    Ad, Wd = A.cuda(), W.cuda()
    ws = torch.empty(64 * M * N, dtype=torch.float32, device="cuda")
    one_pass = torch.empty(M, N, dtype=odt, device="cuda")
    _abi.check(lib.tlq_gemm_f16(P(Ad), P(Wd), P(one_pass), M, N, K, code[dt], code[odt], lay, st))
    for slices in (0, 2, 3, 5, 64):
        lib.tlq_tune_f16_split(slices)
        try:
            outs = []
            for _ in range(2):
                ws.fill_(float("nan"))  # stale contents must not matter
                C = torch.full((M, N), float("nan"), dtype=odt, device="cuda")
                _abi.check(lib.tlq_gemm_f16_ws(P(Ad), P(Wd), P(C), P(ws), ws.numel() * 4, 1, M, N, K, code[dt], code[odt], lay, st))
                torch.cuda.synchronize()
                outs.append(C.cpu())
            # no workspace: the one-pass kernel
            D = torch.full((M, N), float("nan"), dtype=odt, device="cuda")
            _abi.check(lib.tlq_gemm_f16_ws(P(Ad), P(Wd), P(D), None, 0, 1, M, N, K, code[dt], code[odt], lay, st))
            torch.cuda.synchronize()
        finally:
            lib.tlq_tune_f16_split(0)
        what = f"{in_dtype}->{out_dtype} {slices} slices asked, {M}x{N}x{K} layout {lay}"
        check_float_output(outs[0], want, what)
        assert torch.equal(outs[0], outs[1]), what + ": slice order must make the result reproducible"
        assert_bit_equal(D.cpu(), one_pass.cpu(), what + ": without a workspace")


@pytest.mark.gpu
def test_fewer_slices_in_a_smaller_workspace():
    _abi, lib, P = _lib()
    M, N, K = 16, 2048, 4096
    st = torch.cuda.current_stream().cuda_stream
    A = torch.randn(M, K, generator=gen(1)).half()
    W = torch.randn(N, K, generator=gen(2)).half()
    want = A.float() @ W.float().t()
    Ad, Wd = A.cuda(), W.cuda()
    full = lib.tlq_f16_workspace_bytes(1, M, N, K)
    assert full >= 4 * M * N * 4
    ws = torch.empty(full, dtype=torch.uint8, device="cuda")
    for nbytes in (full, 2 * M * N * 4, M * N * 4, 64):
        C = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        _abi.check(lib.tlq_gemm_f16_ws(P(Ad), P(Wd), P(C), P(ws), nbytes, 1, M, N, K, _abi.F16, _abi.F16, _abi.B_NK, st))
        torch.cuda.synchronize()
        check_float_output(C.cpu(), want, f"workspace of {nbytes} bytes")


@pytest.mark.gpu
def test_the_fp16_gemm_operator_and_the_two_passes_use_the_slices():
    from tilelang_ascend_amd import ops

    _abi, lib, P = _lib()
    M, N, K = 24, 1024, 4096
    assert lib.tlq_f16_workspace_bytes(1, M, N, K) > 0
    A = torch.randn(M, K, generator=gen(3)).half()
    B = torch.randn(K, N, generator=gen(4)).half()
    got = ops.fp16_gemm(M, N, K, 128, 256, 64)(A.cuda(), B.cuda()).cpu()
    check_float_output(got, A.float() @ B.float(), "fp16_gemm, few rows")
    # W4A16, forced two passes, with and without room for the slices behind the dequantised matrix
    M, N, K, g = 300, 256, 2752, 64
    for dt, code in ((torch.float16, _abi.F16), (torch.bfloat16, _abi.BF16)):
        A = torch.randn(M, K, generator=gen(5)).to(dt)
        Wp, s, z = make_w4(N, K, g, dt, "int", seed=6)
        want = w4a16_reference(A, Wp, s, z, g)
        need = lib.tlq_w4a16_workspace_bytes(M, N, K)
        assert need > N * K * 2
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        Ad, Wd, sd, zd = A.cuda(), Wp.cuda(), s.cuda(), z.cuda()
        st = torch.cuda.current_stream().cuda_stream
        for nbytes in (need, N * K * 2):
            C = torch.full((M, N), float("nan"), dtype=dt, device="cuda")
            _abi.check(lib.tlq_gemm_w4a16_ws(P(Ad), P(Wd), P(sd), P(zd), P(C), M, N, K, g, 0.0, code, code, _abi.ALGO_TWO_PASS,
                                             P(ws), nbytes, st))
            torch.cuda.synchronize()
            check_float_output(C.cpu(), want, f"two passes {dt}, workspace {nbytes}")
