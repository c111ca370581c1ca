"""tlq_gemm_w4a16_noalloc (the entry point that allocates nothing: its workspace is a device array built into the
library) against tlq_gemm_w4a16_ws with a caller-owned workspace, through the C ABI, bit for bit: the same kernels run
in the same order, only the workspace address differs.  Two calls in a row share the built-in array, the second on a
smaller problem, so stale contents of the first call lie behind and beside what the second one uses.
"""
import pytest
import torch

from helpers import assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference
from oracle import ref

pytestmark = pytest.mark.gpu

SCRATCH = 64 << 20


def _both(M, N, K, group, dtype, zeros_kind, seed):
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    code = _abi.F16 if dtype == torch.float16 else _abi.BF16
    A = torch.randn(M, K, generator=gen(seed)).to(dtype)
    Wp, s, z = make_w4(N, K, group, dtype, zeros_kind, seed + 1)
    zt = z if torch.is_tensor(z) else None
    zs = 0.0 if torch.is_tensor(z) or z is None else float(z)
    dA, dW, dS = A.cuda(), Wp.cuda(), s.cuda()
    dZ = zt.cuda() if zt is not None else None
    st = torch.cuda.current_stream().cuda_stream
    need = lib.tlq_w4a16_workspace_bytes(M, N, K)
    assert 0 < need <= SCRATCH, f"the case must use scratch memory and fit the built-in array (needs {need})"
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    want = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    _abi.check(lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(want), M, N, K, group, zs, code, code, _abi.ALGO_AUTO,
                                     P(ws), need, st))
    got = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    # (a warm-up call first: the one-time look-up of the array's address must not count)
    _abi.check(lib.tlq_gemm_w4a16_noalloc(P(dA), P(dW), P(dS), P(dZ), P(got), M, N, K, group, zs, code, code,
                                          _abi.ALGO_AUTO, st))
    torch.cuda.synchronize()
    got.fill_(float("nan"))
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    _abi.check(lib.tlq_gemm_w4a16_noalloc(P(dA), P(dW), P(dS), P(dZ), P(got), M, N, K, group, zs, code, code,
                                          _abi.ALGO_AUTO, st))
    torch.cuda.synchronize()
    # torch's counter sees its own allocator only; the device's free memory also shows a hipMalloc inside the library
    assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] == free_before
    return got.cpu(), want.cpu(), (A, Wp, s, z)


def test_noalloc_matches_the_workspace_entry_point_twice_in_a_row():
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    assert lib.tlq_gemm_w4a16_noalloc_init() == 0, _abi.last_error()
    # first call: two passes (the dequantised 4096 x 2048 bf16 matrix, 16 MiB of the array)
    got, want, _ = _both(2048, 4096, 2048, 128, torch.bfloat16, "scalar8", 11)
    assert_bit_equal(got, want, "two-pass problem")
    # second call, smaller: K slices whose fp32 partial sums overlay the start of the first call's matrix
    got, want, (A, Wp, s, z) = _both(48, 1024, 2048, 64, torch.float16, "int", 21)
    assert_bit_equal(got, want, "split-K problem after a larger call")
    check_float_output(got, w4a16_reference(A, Wp, s, z, 64), "split-K problem vs the oracle")
    # and once more the first shape with other data: nothing of the second call may leak into it
    got, want, _ = _both(2048, 4096, 2048, 128, torch.bfloat16, "scalar8", 31)
    assert_bit_equal(got, want, "two-pass problem, third call")


def test_noalloc_takes_the_next_best_kernel_when_only_that_fits():
    """M = 300, N = 4096, K = 10240: the two passes would need 80 MiB + the K slices of their GEMM, more than the built-in
    array; the partial sums of the K-slice kernels (46.9 MiB) fit.  The call must then equal tlq_gemm_w4a16_ws with a
    workspace of the array's size, bit for bit, and meet the float bar against the oracle."""
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, N, K, g = 300, 4096, 10240, 128
    assert lib.tlq_w4a16_workspace_bytes(M, N, K) > SCRATCH >= lib.tlq_w4a16_workspace_bytes_min(M, N, K) > 0
    A = torch.randn(M, K, generator=gen(41)).half()
    Wp, s, z = make_w4(N, K, g, torch.float16, "int", 42)
    dA, dW, dS, dZ = A.cuda(), Wp.cuda(), s.cuda(), z.cuda()
    st = torch.cuda.current_stream().cuda_stream
    ws = torch.empty(SCRATCH, dtype=torch.uint8, device="cuda")
    want = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    _abi.check(lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(want), M, N, K, g, 0.0, _abi.F16, _abi.F16, _abi.ALGO_AUTO,
                                     P(ws), SCRATCH, st))
    got = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    before = torch.cuda.memory_allocated()
    _abi.check(lib.tlq_gemm_w4a16_noalloc(P(dA), P(dW), P(dS), P(dZ), P(got), M, N, K, g, 0.0, _abi.F16, _abi.F16,
                                          _abi.ALGO_AUTO, st))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert_bit_equal(got.cpu(), want.cpu(), "next-best kernel in the built-in array")
    check_float_output(got.cpu(), w4a16_reference(A, Wp, s, z, g), "next-best kernel vs the oracle")


def test_noalloc_runs_what_does_not_fit_on_the_kernels_without_scratch():
    """M = 2048, N = 14336, K = 4096: even the least demanding workspace kernel would need more than the built-in array.
    The call then equals tlq_gemm_w4a16_ws without a workspace (the kernels that need no scratch), bit for bit, instead of
    failing for lack of room; a sample of rows is checked against the oracle."""
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, N, K, g = 2048, 14336, 4096, 128
    assert lib.tlq_w4a16_workspace_bytes_min(M, N, K) > SCRATCH
    A = torch.randn(M, K, generator=gen(51)).half()
    Wp, s, _ = make_w4(N, K, g, torch.float16, None, 52)
    dA, dW, dS = A.cuda(), Wp.cuda(), s.cuda()
    st = torch.cuda.current_stream().cuda_stream
    want = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    _abi.check(lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), None, P(want), M, N, K, g, 8.0, _abi.F16, _abi.F16, _abi.ALGO_AUTO, None, 0, st))
    got = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    _abi.check(lib.tlq_gemm_w4a16_noalloc(P(dA), P(dW), P(dS), None, P(got), M, N, K, g, 8.0, _abi.F16, _abi.F16, _abi.ALGO_AUTO, st))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert_bit_equal(got.cpu(), want.cpu(), "problem beyond the built-in array")
    rows = torch.arange(0, M, 37)
    W = ref.dequant_w4(Wp, s, 8, g, torch.float16).float()
    check_float_output(got.cpu()[rows], A[rows].float() @ W.T, "problem beyond the built-in array vs the oracle")
