"""Non-quantised twins: plain GEMV (examples/gemv), split-K GEMM (examples/gemm_splitk), batched GEMM
(examples/batch_gemm) and the plain fp16 GEMM of the dequant example with the second operand stored [K, N]."""
import pytest
import torch

from oracle import ref

DT = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32}


def test_oracles_closed_forms():
    A = torch.arange(24, dtype=torch.float32).view(4, 6)
    x = torch.zeros(6)
    x[2] = 1.0
    assert torch.equal(ref.ref_program_gemv(x, A), A[:, 2])                  # one-hot picks a column
    assert torch.equal(ref.ref_program_gemv(torch.ones(6), A), A.sum(dim=1))  # constant vector: row sums
    a = torch.randn(5, 8, generator=torch.Generator().manual_seed(1)).half()
    b = torch.eye(8).half()
    assert torch.equal(ref.ref_program_splitk(a, b), a.float())              # identity


def _rel_l2(got, want):
    return float((got.double() - want.double()).norm() / want.double().norm().clamp_min(1e-30))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32"])
@pytest.mark.parametrize("N,K", [(1024, 1024), (64, 64), (3, 8), (1, 4096), (257, 11008), (11008, 4096), (77, 40000)])
def test_gemv_matches_reference(dtype, N, K):
    from tilelang_ascend_amd.ops import simple_gemv

    g = torch.Generator().manual_seed(N + K)
    x = torch.randn(K, generator=g).to(DT[dtype])
    A = torch.randn(N, K, generator=g).to(DT[dtype])
    y = simple_gemv(N, K, 128, 128, dtype=dtype)(x.cuda(), A.cuda()).cpu()
    assert y.dtype == DT[dtype] and y.shape == (N,)
    want = ref.ref_program_gemv(x, A)
    exact = A.double() @ x.double()
    # fp32 accumulation: relative L2 <= 1e-3 of the exact product on top of the output rounding; the
    # reference's own criterion (example_gemv_v.py:97) is assert_close(rtol=atol=1e-2) scaled by sqrt(K) magnitudes
    assert _rel_l2(y, exact) <= (1e-5 if dtype == "float32" else 3e-3), _rel_l2(y, exact)
    torch.testing.assert_close(y.float(), want.float(), rtol=1e-2, atol=1e-2 * max(1.0, (K / 1024) ** 0.5))


@pytest.mark.gpu
def test_gemv_one_hot_and_row_sums_are_exact():
    from tilelang_ascend_amd.ops import simple_gemv

    N, K = 130, 2048
    A = torch.randint(-8, 8, (N, K), generator=torch.Generator().manual_seed(3)).half()
    k = simple_gemv(N, K, 64, 64)
    for j in (0, 7, 8, 1023, 2047):
        x = torch.zeros(K, dtype=torch.float16)
        x[j] = 1.0
        assert torch.equal(k(x.cuda(), A.cuda()).cpu(), A[:, j])
    ones = torch.ones(K, dtype=torch.float16)
    assert torch.equal(k(ones.cuda(), A.cuda()).cpu().float(), A.float().sum(dim=1))  # small integers: exact in fp32


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,split_k", [(128, 128, 128, 2), (1024, 1024, 1024, 4), (16, 4096, 14336, 16), (100, 72, 960, 3),
                                           (300, 264, 512, 1), (64, 128, 8192, 64)])
def test_splitk_matches_reference(dtype, M, N, K, split_k):
    from tilelang_ascend_amd.ops import gemm_splitk

    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, K, generator=g).to(DT[dtype])
    b = torch.randn(K, N, generator=g).to(DT[dtype])
    c = torch.zeros(M, N, dtype=torch.float32, device="cuda")
    out = gemm_splitk(M, N, K, 128, 128, 32, split_k, dtype=dtype)(a.cuda(), b.cuda(), c)
    assert out == [] or out is None
    want = ref.ref_program_splitk(a, b)
    assert _rel_l2(c.cpu(), want) <= 1e-5
    torch.testing.assert_close(c.cpu(), want, rtol=1e-2, atol=1e-2)
    # accumulation in place: a second call doubles the result
    gemm_splitk(M, N, K, 128, 128, 32, split_k, dtype=dtype)(a.cuda(), b.cuda(), c)
    assert _rel_l2(c.cpu(), 2 * want) <= 1e-5


@pytest.mark.gpu
def test_splitk_integer_inputs_are_exact_for_any_split():
    """Small-integer operands make every partial sum exact in fp32, so all splits must agree bit for bit."""
    from tilelang_ascend_amd.ops import gemm_splitk

    M, N, K = 48, 136, 1536
    g = torch.Generator().manual_seed(9)
    a = torch.randint(-4, 5, (M, K), generator=g).half()
    b = torch.randint(-4, 5, (K, N), generator=g).half()
    want = ref.ref_program_splitk(a, b)
    for split_k in (1, 2, 3, 6, 12, 24):
        c = torch.zeros(M, N, dtype=torch.float32, device="cuda")
        gemm_splitk(M, N, K, 128, 128, 32, split_k)(a.cuda(), b.cuda(), c)
        assert torch.equal(c.cpu(), want), split_k


@pytest.mark.gpu
def test_plain_twins_reject_bad_arguments():
    from tilelang_ascend_amd import _abi
    from tilelang_ascend_amd.ops import gemm_splitk

    lib, P = _abi.load(), _abi.ptr
    x = torch.zeros(64, device="cuda", dtype=torch.float16)
    A = torch.zeros(4, 64, device="cuda", dtype=torch.float16)
    y = torch.zeros(4, device="cuda", dtype=torch.float16)
    assert lib.tlq_gemv(P(x), P(A), P(y), 4, 60, _abi.F16, _abi.F16, None) != 0 and "16 bytes" in _abi.last_error()
    assert lib.tlq_gemv(P(x), P(A), P(y), 4, 64, _abi.I8, _abi.F16, None) != 0
    assert lib.tlq_gemv(P(x), P(A), P(y), 0, 64, _abi.F16, _abi.F16, None) == 0
    c = torch.zeros(4, 8, device="cuda")
    assert lib.tlq_gemm_f16_splitk(P(A), P(A), P(c), 4, 8, 64, 3, _abi.F16, _abi.B_KN, None) != 0
    assert "slices" in _abi.last_error()
    with pytest.raises(ValueError):
        gemm_splitk(4, 8, 64, 128, 128, 32, 5)


@pytest.mark.gpu
def test_plain_twin_examples(capsys):
    from tilelang_ascend_amd.examples.gemm_splitk import example_gemm_splitk as exs
    from tilelang_ascend_amd.examples.gemv import example_gemv as exg

    exg.main(["--n", "512", "--k", "768"])
    out = capsys.readouterr().out
    assert out.rstrip().splitlines()[-2:] == ["GEMV example passed!", "Kernel Output Match!"]
    exs.main([])
    out = capsys.readouterr().out
    assert "Test passed: M=128, N=128, K=128, split_k=2" in out and "Test passed: M=1024, N=1024, K=1024, split_k=4" in out
    assert out.rstrip().endswith("Kernel Output Match!")
    exs.main(["--M", "64", "--N", "256", "--K", "2048", "--split-k", "8"])
    assert "Test passed: M=64, N=256, K=2048, split_k=8" in capsys.readouterr().out


def _ternary(shape, seed):
    return torch.randint(-1, 2, shape, generator=torch.Generator().manual_seed(seed)).to(torch.float16)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(2300, 4104, 328), (4096, 2048, 72), (130, 264, 200), (2048, 4096, 1024)])
def test_fp16_gemm_kn_operand_large_tiles_and_k_tails(M, N, K):
    """B stored [K, N] is transposed on the way into LDS: shapes that take the 256 x 256 instance (ragged M and N, K not a
    multiple of the 64-element stage) and the 128 x 128 one.  Ternary inputs make every sum an exact small integer, so the
    comparison with the integer product is bit for bit; random inputs are checked at the float-output bar."""
    from helpers import check_float_output
    from tilelang_ascend_amd.ops import fp16_gemm

    kernel = fp16_gemm(M, N, K, 128, 256, 64)
    A, B = _ternary((M, K), 60), _ternary((K, N), 61)
    got = kernel(A.cuda(), B.cuda()).cpu()
    assert torch.equal(got, (A.float() @ B.float()).half())
    g = torch.Generator().manual_seed(62)
    A, B = torch.randn(M, K, generator=g).half(), torch.randn(K, N, generator=g).half()
    check_float_output(kernel(A.cuda(), B.cuda()).cpu(), A.float() @ B.float(), f"fp16_gemm [K,N] {M}x{N}x{K}")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("B,M,N,K", [(1, 2048, 4096, 1024), (1, 1024, 2056, 512), (1, 4096, 4096, 64), (2, 1000, 1288, 192), (3, 300, 264, 128), (1, 257, 8, 64)])
def test_kn_operand_on_the_five_slot_kernel(dtype, B, M, N, K):
    """[K, N] weights copied global -> LDS as they are and transposed by the operand read (ds_read_b64_tr_b16): whole 64-value
    stages of K, N a multiple of 8, forced onto the 256 x 256 tiles so that small, ragged and batched problems take this
    loader too.  Exact on ternary inputs; random inputs at the float-output bar; and the same bits as the two-stage kernel
    that reads [K, N] weights through registers (tlq_tune_gemm_slots(0))."""
    from helpers import check_float_output
    from tilelang_ascend_amd import _abi
    from tilelang_ascend_amd.ops import batch_matmul

    lib = _abi.load()
    kernel = batch_matmul(B, M, N, K, 128, 256, 64, dtype=dtype)
    lib.tlq_tune_gemm_tile(256)
    lib.tlq_tune_gemm_slots(2)  # the five-slot kernel wherever it can run
    try:
        a, b = _ternary((B, M, K), 66).to(DT[dtype]), _ternary((B, K, N), 67).to(DT[dtype])
        got = kernel(a.cuda(), b.cuda()).cpu()
        assert torch.equal(got, torch.matmul(a.float(), b.float()).to(DT[dtype]))
        g = torch.Generator().manual_seed(68)
        a, b = torch.randn(B, M, K, generator=g).to(DT[dtype]), torch.randn(B, K, N, generator=g).to(DT[dtype])
        got = kernel(a.cuda(), b.cuda()).cpu()
        want = torch.matmul(a.float(), b.float())
        for i in range(B):
            check_float_output(got[i], want[i], f"[K,N] five-slot {dtype} batch {i}")
        lib.tlq_tune_gemm_slots(0)
        two_stage = kernel(a.cuda(), b.cuda()).cpu()
        assert torch.equal(got, two_stage), "five-slot vs two-stage kernel on [K, N] weights"
    finally:
        lib.tlq_tune_gemm_slots(1)
        lib.tlq_tune_gemm_tile(0)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("B,M,N,K", [(8, 1024, 1024, 1024), (3, 100, 72, 40), (2, 520, 264, 136), (20, 256, 512, 64), (1, 64, 64, 64)])
def test_batch_matmul_matches_reference(dtype, B, M, N, K):
    from helpers import check_float_output
    from tilelang_ascend_amd.ops import batch_matmul

    kernel = batch_matmul(B, M, N, K, 128, 256, 64, dtype=dtype)
    a, b = _ternary((B, M, K), 63).to(DT[dtype]), _ternary((B, K, N), 64).to(DT[dtype])
    got = kernel(a.cuda(), b.cuda()).cpu()
    assert got.shape == (B, M, N) and got.dtype == DT[dtype]
    assert torch.equal(got, torch.matmul(a.float(), b.float()).to(DT[dtype]))  # exact small integers, batch by batch
    g = torch.Generator().manual_seed(65)
    a, b = torch.randn(B, M, K, generator=g).to(DT[dtype]), torch.randn(B, K, N, generator=g).to(DT[dtype])
    got = kernel(a.cuda(), b.cuda()).cpu()
    want = torch.matmul(a.float(), b.float())
    for i in range(B):
        check_float_output(got[i], want[i], f"batch_matmul {dtype} batch {i}")
    torch.testing.assert_close(got, want.to(DT[dtype]), rtol=1e-2, atol=1e-2)  # the example's own criterion (batch_gemm.py:77)


@pytest.mark.gpu
def test_batch_matmul_example_and_bad_arguments(capsys):
    from tilelang_ascend_amd import _abi
    from tilelang_ascend_amd.examples.batch_gemm import batch_gemm as ex
    from tilelang_ascend_amd.ops import batch_matmul

    ex.main(["--b", "4", "--m", "256", "--n", "512", "--k", "128"])
    assert capsys.readouterr().out.rstrip().splitlines()[-2:] == ["init successful!", "Batch Kernel Output Match!"]
    with pytest.raises(ValueError):
        batch_matmul(2, 64, 64, 64, 128, 256, 64, dtype="float32")
    lib, P = _abi.load(), _abi.ptr
    t = torch.zeros(4096, device="cuda", dtype=torch.float16)
    assert lib.tlq_gemm_f16_batched(P(t), P(t), P(t), 2, 3, 8, 8, _abi.F16, _abi.F16, _abi.B_KN, None) == 0  # 3*8 % 8 == 0
    assert lib.tlq_gemm_f16_batched(P(t), P(t), P(t), 2, 3, 8, 12, _abi.F16, _abi.F16, _abi.B_KN, None) != 0
    assert lib.tlq_gemm_f16_batched(P(t), P(t), P(t), -1, 8, 8, 8, _abi.F16, _abi.F16, _abi.B_KN, None) != 0
    assert "batch" in _abi.last_error()
    assert lib.tlq_gemm_f16_batched(P(t), P(t), P(t), 0, 8, 8, 8, _abi.F16, _abi.F16, _abi.B_KN, None) == 0
