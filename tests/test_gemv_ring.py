"""The ring kernel of the single decode GEMV (M = 1, rows of up to 4096 values: every global read a direct
global -> LDS load) against the register-resident kernel it replaces -- same sums in the same order, so the outputs
must be the same bits -- and against the oracle (examples/gemv/example_gemv_c.py:27-46 for the shape convention)."""
import pytest
import torch

from helpers import DT, assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference

pytestmark = pytest.mark.gpu


def run_gemv(A, Wp, s, z, group, ring, out_dtype=None):
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, K = A.shape
    N = Wp.shape[0]
    code = {torch.float16: _abi.F16, torch.float32: _abi.F32, torch.bfloat16: _abi.BF16}
    out_dtype = out_dtype or A.dtype
    zt = z if torch.is_tensor(z) else None
    zs = 0.0 if (torch.is_tensor(z) or z is None) else float(z)
    dA, dW = A.cuda(), Wp.cuda()
    dS = s.cuda() if s is not None else None
    dZ = zt.cuda() if zt is not None else None
    C = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    print(f"gemv ring={ring} M={M} N={N} K={K} g={group} {A.dtype} out={out_dtype}", flush=True)
    lib.tlq_tune_gemv_ring(ring)
    try:
        _abi.check(lib.tlq_gemm_w4a16(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, code[A.dtype], code[out_dtype],
                                      _abi.ALGO_GEMV, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
    finally:
        lib.tlq_tune_gemv_ring(1)
    return C.cpu()


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("zeros_kind", [None, "scalar8", "int", "frac"])
@pytest.mark.parametrize("N,K,group", [
    (11008, 4096, 128), (14336, 4096, 64), (77, 1024, 32), (1000, 2048, 64), (4096, 4096, 32), (16, 256, 32), (1, 512, 64),
    (5000, 2560, 64), (513, 3072, 128), (32000, 1024, 128),
])
def test_ring_kernel_equals_the_register_resident_kernel_and_the_oracle(N, K, group, zeros_kind, in_dtype):
    from tilelang_ascend_amd import _abi

    plan = (torch.zeros(6, dtype=torch.int64)).numpy()
    assert _abi.load().tlq_debug_gemv_ring_plan(1, N, K, group, 256, plan.ctypes.data) == 1, "this shape is meant to take the ring kernel"
    dt = DT[in_dtype]
    A = torch.randn(1, K, generator=gen(80)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=81)
    ring = run_gemv(A, Wp, s, z, group, 1)
    rows = run_gemv(A, Wp, s, z, group, 0)
    assert_bit_equal(ring, rows, f"ring vs register-resident kernel {in_dtype} N={N} K={K} g={group} zeros={zeros_kind}")
    check_float_output(ring, w4a16_reference(A, Wp, s, z, group), "ring kernel vs oracle")


def test_ring_kernel_float32_output_and_absent_scales():
    N, K, group = 3000, 4096, 128
    A = torch.randn(1, K, generator=gen(82)).to(torch.float16)
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=83)
    for ss, zz in ((s, z), (None, z), (s, None), (None, None)):
        ring = run_gemv(A, Wp, ss, zz, group, 1, torch.float32)
        rows = run_gemv(A, Wp, ss, zz, group, 0, torch.float32)
        assert_bit_equal(ring, rows, "ring vs register-resident kernel, fp32 output")
        want = w4a16_reference(A, Wp, ss, zz, group)
        if ss is None:  # unscaled weights: sums of several hundred, judged by their relative error
            assert ((ring - want).norm() / want.norm()).item() <= 1e-4
        else:
            check_float_output(ring, want, "ring kernel vs oracle, fp32 output")


def test_misaligned_scales_fall_back_to_the_register_resident_kernel():
    """Scale / zero tensors that do not start on a 16-byte boundary cannot feed 16-byte direct loads."""
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    N, K, group = 256, 1024, 32
    A = torch.randn(1, K, generator=gen(84)).to(torch.float16)
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=85)
    pad_s = torch.zeros(s.numel() + 8, dtype=torch.float16, device="cuda")
    pad_z = torch.zeros(z.numel() + 8, dtype=torch.float16, device="cuda")
    ds, dz = pad_s[1:1 + s.numel()].view_as(s), pad_z[1:1 + z.numel()].view_as(z)
    ds.copy_(s)
    dz.copy_(z)
    dA, dW = A.cuda(), Wp.cuda()
    C = torch.full((1, N), float("nan"), dtype=torch.float16, device="cuda")
    _abi.check(lib.tlq_gemm_w4a16(P(dA), P(dW), P(ds), P(dz), P(C), 1, N, K, group, 0.0, _abi.F16, _abi.F16, _abi.ALGO_GEMV,
                                  torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    check_float_output(C.cpu(), w4a16_reference(A, Wp, s, z, group), "misaligned scales")


@pytest.mark.parametrize("zeros_kind", [None, "scalar8", "int", "frac"])
@pytest.mark.parametrize("N,K,group", [(11008, 4096, 128), (77, 1024, 32), (1000, 2048, 64), (5000, 2560, 64), (16, 256, 32), (14336, 4096, 64)])
def test_ring_kernel_with_two_activation_rows(N, K, group, zeros_kind):
    """fp16, two activation rows: each weight row is expanded once and multiplied with both.  Against the oracle; and each
    activation row must come out exactly as it does when it is the only one (the rows do not mix)."""
    from tilelang_ascend_amd import _abi

    M = 2
    plan = (torch.zeros(6, dtype=torch.int64)).numpy()
    assert _abi.load().tlq_debug_gemv_ring_plan(M, N, K, group, 256, plan.ctypes.data) == 1
    A = torch.randn(M, K, generator=gen(88)).to(torch.float16)
    Wp, s, z = make_w4(N, K, group, torch.float16, zeros_kind, seed=89)
    got = run_gemv(A, Wp, s, z, group, 1)
    check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"ring kernel M={M} vs oracle")
    for m in (0, M - 1):
        alone = run_gemv(A[m:m + 1].contiguous(), Wp, s, z, group, 1)
        assert_bit_equal(got[m:m + 1], alone, f"activation row {m} of {M} vs the same row alone")


@pytest.mark.parametrize("per_cu", [2, 3])
@pytest.mark.parametrize("N,K,group", [(11008, 4096, 128), (5000, 2560, 64), (14336, 4096, 64), (600, 1024, 32)])
def test_ring_kernel_with_several_work_groups_per_cu(N, K, group, per_cu):
    """tlq_tune_gemv_unroll sizes the grid for that many work-groups per CU (fewer rows per work-group): the same rows,
    each summed in the same order, so the same bits as the default grid."""
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    A = torch.randn(1, K, generator=gen(70)).half()
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=71)
    want = run_gemv(A, Wp, s, z, group, 1)
    lib.tlq_tune_gemv_unroll(per_cu)
    try:
        got = run_gemv(A, Wp, s, z, group, 1)
    finally:
        lib.tlq_tune_gemv_unroll(0)
    assert_bit_equal(got, want, f"{per_cu} work-groups per CU, N={N} K={K} g={group}")
    check_float_output(got, w4a16_reference(A, Wp, s, z, group), "against the oracle")
