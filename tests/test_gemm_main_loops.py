"""The two main loops of the 256 x 256 GEMM tiles against each other: the five-slot kernel (csrc/gemm_slots.h, whole
128-byte stages of K; tlq_tune_gemm_slots(2) takes it wherever it can run) and the two-stage kernel (csrc/gemm_core.h,
tlq_tune_gemm_slots(0)).  Every case
runs the same inputs through both: integer GEMMs and the rescaled outputs must agree bit for bit, and so must the
16-bit GEMMs (same tiling, same order of accumulation inside a tile; the kernels only differ in when data is fetched).
The default path is also checked against an exact / fp32 evaluation.
"""
import pytest
import torch

from helpers import assert_bit_equal, gen

pytestmark = pytest.mark.gpu

HOOKS = [("slots", 0)]


def _with_hook(name, value, fn):
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    hook = getattr(lib, f"tlq_tune_gemm_{name}")
    hook(value)
    try:
        return fn()
    finally:
        hook(1)  # the default


# K in 16-bit values: one, two, three stages (64 values each), odd stage counts, a partial last stage (falls back /
# register tail), long rows; M, N ragged against the 256 x 256 tile
# (the 256 x 256 kernels are chosen from 128 output tiles on: M, N around 2900)
SHAPES_16 = [(256, 256, 64), (300, 520, 192), (1000, 1288, 4160), (4096, 4096, 4096), (260, 264, 96), (2048, 2304, 72),
             (2900, 2904, 64), (2900, 2824, 128), (3000, 2824, 192), (2816, 3072, 320), (2820, 2904, 72)]


@pytest.mark.parametrize("hook,value", HOOKS)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", SHAPES_16)
def test_plain_gemm_same_bits_on_both_main_loops(hook, value, dtype, M, N, K):
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    A = torch.randn(M, K, generator=gen(1)).to(dtype).cuda()
    B = torch.randn(N, K, generator=gen(2)).to(dtype).cuda()
    code = _abi.F16 if dtype == torch.float16 else _abi.BF16
    st = torch.cuda.current_stream().cuda_stream

    def run():
        C = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
        _abi.check(lib.tlq_gemm_f16(P(A), P(B), P(C), M, N, K, code, code, _abi.B_NK, st))
        torch.cuda.synchronize()
        return C.cpu()

    want = _with_hook(hook, 2, run)  # the five-slot kernel wherever it can run
    ref32 = A.float().cpu() @ B.float().cpu().t()
    assert float((want.float() - ref32).norm() / ref32.norm()) < 3e-3
    got = _with_hook(hook, value, run)
    assert_bit_equal(got, want, f"{hook}={value} {dtype} {M}x{N}x{K}")


@pytest.mark.parametrize("hook,value", HOOKS)
@pytest.mark.parametrize("layout", ["KN", "NK"])
@pytest.mark.parametrize("B,M,N,K", [(1, 256, 256, 128), (2, 300, 528, 384), (1, 2048, 4096, 4096), (3, 512, 272, 640),
                                     (1, 260, 512, 144)])
def test_w8a8_same_bits_on_both_main_loops(hook, value, layout, B, M, N, K):
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    A = torch.randint(-127, 128, (B, M, K), dtype=torch.int8, generator=gen(3)).cuda()
    W = torch.randint(-127, 128, (B, K, N) if layout == "KN" else (B, N, K), dtype=torch.int8, generator=gen(4)).cuda()
    sa = (torch.rand(B, M, generator=gen(5)) * 0.04 + 0.01).cuda()
    sb = (torch.rand(N, generator=gen(6)) * 0.009 + 0.001).cuda()
    st = torch.cuda.current_stream().cuda_stream
    lay = _abi.B_KN if layout == "KN" else _abi.B_NK

    def run():
        lib.tlq_tune_i8_tile(256)  # the 256 x 256 kernels, whatever the number of tiles
        try:
            C = torch.full((B, M, N), float("nan"), dtype=torch.float16, device="cuda")
            _abi.check(lib.tlq_gemm_w8a8(P(A), P(W), P(sa), P(sb), P(C), B, M, N, K, N, lay, _abi.F16, st))
            Ci = torch.full((B, M, N), -1, dtype=torch.int32, device="cuda")
            _abi.check(lib.tlq_gemm_i8(P(A), P(W), P(Ci), B, M, N, K, lay, st))
            torch.cuda.synchronize()
        finally:
            lib.tlq_tune_i8_tile(0)
        return C.cpu(), Ci.cpu()

    want, want_i = _with_hook(hook, 2, run)  # the five-slot kernel wherever it can run
    Wt = W.cpu() if layout == "KN" else W.cpu().transpose(1, 2)
    exact = torch.matmul(A.cpu().double(), Wt.double()).to(torch.int64)
    assert torch.equal(want_i.to(torch.int64), exact)
    got, got_i = _with_hook(hook, value, run)
    assert torch.equal(got_i, want_i), f"{hook}={value} int32 accumulators differ"
    assert_bit_equal(got, want, f"{hook}={value} {layout} {B}x{M}x{N}x{K}")
