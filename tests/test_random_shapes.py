"""Seeded random shapes through the automatic kernel choice (tlq_gemm_w4a16_ws with the workspace its query asks for, and
tlq_gemm_w4a16 without one) against the oracle: ragged M and N, K any multiple of 64, every group size that divides K, all
zero-point kinds, both activation types.  Whatever kernel the choice lands on must accept the shape and agree with
ref_program_fp16 extended by scales / zero points (examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:269-289)."""
import random

import pytest
import torch

from helpers import DT, check_float_output, gen, make_w4, w4a16_reference

pytestmark = pytest.mark.gpu


def random_case(seed):
    rnd = random.Random(seed)
    M = rnd.choice([1, 2, 3, 5, 8, 16, 17, 24, 32, 33, 48, 64, 65, 100, 128, 200, 256, 300, 512, 513, 700, 1024])
    N = rnd.choice([4, 8, 16, 20, 64, 100, 256, 260, 1000, 1024, 2048, 3000, 4096, 5120, 8192, 11008])
    K = 64 * rnd.choice([1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 40, 64, 86, 128])
    while M * N * K > 1 << 31:  # keep the oracle's matmul in seconds
        N = max(4, N // 2 // 4 * 4)
    groups = [g for g in (32, 64, 128, 256, 512) if K % g == 0]
    group = rnd.choice(groups)
    zeros_kind = rnd.choice([None, "scalar8", "int", "frac"])
    in_dtype = rnd.choice(["float16", "bfloat16"])
    return M, N, K, group, zeros_kind, in_dtype


@pytest.mark.parametrize("seed", range(72))
def test_automatic_choice_on_random_shapes(seed):
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, N, K, group, zeros_kind, in_dtype = random_case(seed)
    dt = DT[in_dtype]
    code = _abi.F16 if dt == torch.float16 else _abi.BF16
    A = torch.randn(M, K, generator=gen(1000 + seed)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=2000 + seed)
    zt = z if torch.is_tensor(z) else None
    zs = 0.0 if (torch.is_tensor(z) or z is None) else float(z)
    dA, dW, dS = A.cuda(), Wp.cuda(), s.cuda()
    dZ = zt.cuda() if zt is not None else None
    want = w4a16_reference(A, Wp, s, z, group)
    need = lib.tlq_w4a16_workspace_bytes(M, N, K)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    for with_ws in (True, False):
        C = torch.full((M, N), float("nan"), dtype=dt, device="cuda")
        print(f"random shape seed={seed} M={M} N={N} K={K} g={group} zeros={zeros_kind} {in_dtype} workspace={need if with_ws else 'none'}", flush=True)
        if with_ws:
            rc = lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, code, code, _abi.ALGO_AUTO, P(ws), need, st)
        else:
            rc = lib.tlq_gemm_w4a16(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, code, code, _abi.ALGO_AUTO, st)
        torch.cuda.synchronize()
        if rc != 0:
            # the only shapes no kernel takes: more than 16 activation rows with N not a multiple of 4 (MFMA tile stores)
            assert M > 16 and N % 4 != 0, _abi.last_error()
            continue
        check_float_output(C.cpu(), want, f"seed {seed} {'with' if with_ws else 'without'} workspace")


# ---- the other entry points of the path, same idea: seeded random shapes, the reference's own operator signatures ----
from helpers import assert_bit_equal  # noqa: E402
from oracle import ref  # noqa: E402


@pytest.fixture(scope="module")
def ops():
    from tilelang_ascend_amd import _abi, ops

    _abi.load()
    return ops


def _i8(shape, seed):
    return torch.randint(-128, 128, shape, dtype=torch.int8, generator=gen(seed))


@pytest.mark.parametrize("seed", range(40))
def test_int8_family_on_random_shapes(ops, seed):
    """int8_gemm (fine_grained.py:118-173), simple_quant_batch_matmul (example_quant_batch_matmul.py:8-91),
    int8_gemm_kernel_corrected (deepseek_v4/int8_gemm.py:25-104) and w4a8_gemm_cv (example_dequant_gemm_w4a8.py:25-121):
    exact integers, and the rescaled outputs bit for bit."""
    rnd = random.Random(5000 + seed)
    M = rnd.choice([1, 7, 16, 32, 33, 100, 128, 129, 256, 300, 513, 1024, 2048])
    N = rnd.choice([16, 64, 128, 144, 256, 272, 1024, 2064, 4096])
    K = rnd.choice([16, 64, 128, 400, 512, 1024, 2048, 4096])
    while M * N * K > 1 << 31:
        M = max(1, M // 2)
    which = seed % 4
    print(f"int8 family seed={seed} kind={which} M={M} N={N} K={K}", flush=True)
    if which == 0:
        A, B = _i8((M, K), 6000 + seed), _i8((K, N), 7000 + seed)
        got = ops.int8_gemm(M, N, K, 128, 128, 64)(A.cuda(), B.cuda()).cpu()
        assert_bit_equal(got, ref.int_matmul_exact(A, B).to(torch.int32), "int8_gemm")
    elif which == 1:
        Bt = rnd.choice([1, 2, 3, 5])
        M = min(M, 512)
        scale_size = rnd.choice(["1", "N"])
        out_dtype = rnd.choice(["float16", "bfloat16"])
        A, B = _i8((Bt, M, K), 6000 + seed), _i8((Bt, K, N), 7000 + seed)
        scale = torch.randn(N if scale_size == "N" else 1, generator=gen(8000 + seed))
        got = ops.simple_quant_batch_matmul(Bt, M, N, K, scale_size, 128, 256, 64, out_dtype=out_dtype)(A.cuda(), B.cuda(), scale.cuda()).cpu()
        assert_bit_equal(got, ref.ref_program_quant(A, B, scale, DT[out_dtype]), "quant_batch_matmul")
    elif which == 2:
        out_dtype = rnd.choice(["float32", "bfloat16", "float16"])
        A, B = _i8((M, K), 6000 + seed), _i8((N, K), 7000 + seed)
        g = gen(8000 + seed)
        sa = torch.rand(M, generator=g) * 0.04 + 0.01
        sb = torch.rand(N, generator=g) * 0.009 + 0.001
        got = ops.int8_gemm_kernel_corrected(N, K, block_M=64, block_N=64, block_K=64, out_dtype=out_dtype)(A.cuda(), B.cuda(), sa.cuda(), sb.cuda()).cpu()
        assert_bit_equal(got, ref.ref_int8_gemm_sequential(A, B, sa, sb, DT[out_dtype]), "per-token x per-channel")
    else:
        K = max(K, 64) // 64 * 64
        A = torch.randint(-8, 8, (M, K), dtype=torch.int8, generator=gen(6000 + seed))
        qB, _ = ref.generate_quantized_weight(N, K, gen(7000 + seed))
        out = ops.w4a8_gemm_cv(M, N, K)(A.cuda(), qB.cuda(), torch.zeros(N, K, dtype=torch.int8).cuda(), torch.zeros(M, N, dtype=torch.int32).cuda())
        assert_bit_equal(out.cpu().transpose(0, 1).contiguous(), ref.ref_program_w4a8(A, qB).contiguous(), "w4a8")


@pytest.mark.parametrize("seed", range(24))
def test_dequant_unpack_and_activation_quantiser_on_random_shapes(ops, seed):
    """tlq_dequant_w4 / torch_unpack_uint4_to_* (fine_grained.py:10-57) and the per-token quantiser
    (deepseek_v4/act_quant.py:93-142): bit exact."""
    rnd = random.Random(9000 + seed)
    N = rnd.choice([1, 3, 16, 100, 513, 1024, 4096, 11008])
    K = 64 * rnd.choice([1, 2, 3, 8, 16, 33, 64, 172])
    group = rnd.choice([g for g in (32, 64, 128, 256) if K % g == 0])
    dt_name = rnd.choice(["float16", "bfloat16"])
    dt = DT[dt_name]
    zeros_kind = rnd.choice([None, "scalar8", "int", "frac"])
    print(f"dequant / unpack / act-quant seed={seed} N={N} K={K} g={group} {dt_name} zeros={zeros_kind}", flush=True)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=9100 + seed)
    cz = z.cuda() if torch.is_tensor(z) else z
    assert_bit_equal(ops.dequantize_w4(Wp.cuda(), s.cuda(), cz, group, dt).cpu(), ref.dequant_w4(Wp, s, z, group, dt), "dequant_w4")
    assert_bit_equal(ops.torch_unpack_uint4_to_fp16(Wp), ref.torch_unpack_uint4_to_fp16(Wp), "unpack to fp16")
    assert_bit_equal(ops.torch_unpack_uint4_to_int8(Wp), ref.torch_unpack_uint4_to_int8(Wp), "unpack to int8")
    M = rnd.choice([1, 5, 64, 300])
    x = (torch.randn(M, K, generator=gen(9200 + seed)) * rnd.choice([0.01, 1.0, 30.0])).to(torch.bfloat16)
    q, sc = ops.act_quant_kernel_int8_optimized(K)(x.cuda())
    wq, wsc = ref.act_quant_torch(x)
    assert_bit_equal(q.cpu(), wq, "act_quant values")
    assert_bit_equal(sc.cpu().reshape(-1), wsc.reshape(-1), "act_quant scales")


@pytest.mark.parametrize("seed", range(24))
def test_plain_16_bit_gemm_on_random_shapes(ops, seed):
    """fp16_gemm (fine_grained.py:60-115) through the operator, which cuts K into slices for few activation rows and takes
    the tile kernels otherwise: the float-output bar against an fp32 product, and the same bits on a second call."""
    rnd = random.Random(9000 + seed)
    M = rnd.choice([1, 7, 16, 32, 33, 100, 128, 129, 256, 300, 513, 1024, 2048])
    N = rnd.choice([8, 64, 128, 136, 256, 264, 1024, 2056, 4096])
    K = rnd.choice([8, 64, 128, 192, 448, 512, 1024, 2048, 4096, 11008])
    while M * N * K > 1 << 31:
        M = max(1, M // 2)
    print(f"fp16_gemm seed={seed} M={M} N={N} K={K}", flush=True)
    A = torch.randn(M, K, generator=gen(9100 + seed)).half()
    B = torch.randn(K, N, generator=gen(9200 + seed)).half()
    kernel = ops.fp16_gemm(M, N, K, 128, 256, 64)
    got = kernel(A.cuda(), B.cuda()).cpu()
    check_float_output(got, A.float() @ B.float(), f"fp16_gemm {M}x{N}x{K}")
    assert torch.equal(got, kernel(A.cuda(), B.cuda()).cpu()), "the result must be reproducible"
