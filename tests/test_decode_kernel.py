"""The decode kernel (TLQ_ALGO_DECODE: 1 <= M <= 32 activation rows, persistent work-groups, activations resident in
registers, one pass over the packed weights).  CPU part: the launch geometry and every address the kernel would form,
walked on the host with the kernel's own address functions.  GPU part: against the oracle, and with one-hot
activations the outputs must be the dequantised weights bit for bit."""
import ctypes

import pytest
import torch

from helpers import DT, assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference
from oracle import ref

SHAPES = [  # M, N, K, group
    (1, 16, 256, 32), (3, 40, 512, 64), (16, 14336, 4096, 128), (16, 14336, 4096, 64), (16, 4096, 14336, 128), (16, 4096, 14336, 64),
    (7, 11008, 4096, 128), (16, 1000, 2304, 256), (17, 520, 1024, 1024), (32, 14336, 4096, 128), (32, 4096, 14336, 64), (25, 72, 11008, 32),
]


def _plan(M, N, K, group, cus=256):
    from tilelang_ascend_amd import _abi

    out = (ctypes.c_int64 * 5)()
    ok = _abi.load().tlq_debug_decode_plan(M, N, K, group, cus, ctypes.cast(out, ctypes.c_void_p))
    return ok, dict(mt=out[0], chunks=out[1], waves=out[2], grid_x=out[3], lds=out[4])


@pytest.mark.parametrize("M,N,K,group", SHAPES)
def test_decode_plan_and_every_address_on_the_host(M, N, K, group):
    from tilelang_ascend_amd import _abi

    ok, p = _plan(M, N, K, group)
    assert ok, (M, N, K, group)
    assert p["mt"] == (1 if M <= 16 else 2) and 1 <= p["waves"] <= 16 and p["lds"] <= 160 * 1024
    assert p["chunks"] * p["waves"] >= K // 256 > (p["chunks"] - 1) * p["waves"]
    assert p["grid_x"] * p["chunks"] <= 256 and p["grid_x"] <= (N + 15) // 16
    rc = _abi.load().tlq_debug_check_decode_addressing(M, N, K, group, p["mt"], p["chunks"], p["waves"], p["grid_x"])
    assert rc == 0, _abi.last_error()


def test_decode_plan_rejects_what_the_kernel_cannot_do_and_the_check_catches_a_wrong_geometry():
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    for M, N, K, group in ((33, 64, 256, 64), (0, 64, 256, 64), (4, 64, 384, 64), (4, 64, 256, 96), (4, 64, 256, 16), (4, 3, 256, 256),
                           (24, 100, 256, 64)):  # (two activation tiles on rows of 256 values: one wavefront, nobody adds up the second)
        assert not _plan(M, N, K, group)[0], (M, N, K, group)
    assert _plan(24, 100, 512, 64)[0] and _plan(16, 100, 256, 64)[0]
    assert lib.tlq_debug_check_decode_addressing(24, 128, 256, 64, 2, 1, 1, 8) != 0 and "add up" in _abi.last_error()
    # a launch that does not cover K, or leaves tiles out, fails the walk
    assert lib.tlq_debug_check_decode_addressing(16, 512, 4096, 128, 1, 1, 8, 32) != 0 and "slices" in _abi.last_error()
    assert lib.tlq_debug_check_decode_addressing(16, 512, 4096, 128, 1, 1, 16, 64) != 0 and "work-groups" in _abi.last_error()
    assert lib.tlq_debug_check_decode_addressing(20, 512, 4096, 128, 1, 1, 16, 32) != 0
    assert lib.tlq_debug_check_decode_addressing(16, 512, 4096, 128, 1, 1, 16, 32) == 0


def run_decode(A, Wp, s, z, group, out_dtype=None, algo=None, layout=0):
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, K = A.shape
    N = Wp.shape[0]
    code = {torch.float16: _abi.F16, torch.bfloat16: _abi.BF16, torch.float32: _abi.F32}
    out_dtype = out_dtype or A.dtype
    zt = z if torch.is_tensor(z) else None
    zs = 0.0 if (torch.is_tensor(z) or z is None) else float(z)
    dA, dW = A.cuda(), Wp.cuda()
    dS = s.cuda() if s is not None else None
    dZ = zt.cuda() if zt is not None else None
    need = lib.tlq_w4a16_workspace_bytes(M, N, K)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    print(f"decode M={M} N={N} K={K} g={group} {A.dtype} workspace={need}", flush=True)
    _abi.check(lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, code[A.dtype], code[out_dtype],
                                     _abi.ALGO_DECODE if algo is None else algo, P(ws), need, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return C.cpu()


@pytest.mark.gpu
@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,zeros_kind", [
    (1, 16, 256, 32, "int"), (3, 40, 512, 64, "frac"), (16, 14336, 4096, 128, "int"), (16, 4096, 14336, 64, "int"),
    (7, 11008, 4096, 128, "scalar8"), (16, 1000, 2304, 256, None), (17, 520, 1024, 1024, "int"), (32, 14336, 4096, 128, "frac"),
    (32, 4096, 14336, 64, "int"), (25, 72, 11008, 32, "int"), (9, 4100, 4096, 128, "int"), (16, 8200, 1024, 64, "scalar8"),
])
def test_decode_against_the_oracle(in_dtype, M, N, K, group, zeros_kind):
    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(80)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=81)
    got = run_decode(A, Wp, s, z, group)
    check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"decode {in_dtype} {M}x{N}x{K} g{group} {zeros_kind}")


@pytest.mark.gpu
@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("zeros_kind", [None, "scalar8", "int", "frac"])
@pytest.mark.parametrize("M,K", [(16, 512), (32, 4096), (13, 8192)])
def test_decode_one_hot_rows_return_the_dequantised_weights(in_dtype, zeros_kind, M, K):
    """A = rows of the identity: C[m, n] = W[n, col(m)] exactly, for 16-bit and fp32 outputs, one and several chunks of K."""
    dt = DT[in_dtype]
    N, group = 1048, 64
    A = torch.eye(K, dtype=dt)[torch.randperm(K, generator=gen(82))[:M]]
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=83)
    W = ref.dequant_w4(Wp, s, z, group, dt)
    cols = A.float().argmax(dim=1)
    want = W[:, cols].T.contiguous()
    assert_bit_equal(run_decode(A, Wp, s, z, group), want, f"one-hot {in_dtype} zeros={zeros_kind}")
    assert_bit_equal(run_decode(A, Wp, s, z, group, torch.float32), want.float(), f"one-hot f32 out {in_dtype} zeros={zeros_kind}")


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,group", [(24, 100, 256, 64), (32, 64, 256, 128), (20, 48, 512, 32), (17, 1000, 768, 256)])
def test_short_rows_with_more_than_sixteen_activation_rows(M, N, K, group):
    """Rows of 256 values are one wavefront's slice: with two activation tiles the decode kernel does not apply (the
    automatic choice without a workspace takes another kernel); from 512 values on it does."""
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    A = torch.randn(M, K, generator=gen(64)).to(torch.float16)
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=65)
    dA, dW, dS, dZ = A.cuda(), Wp.cuda(), s.cuda(), z.cuda()
    want = w4a16_reference(A, Wp, s, z, group)
    for algo in (_abi.ALGO_AUTO, _abi.ALGO_DECODE):
        C = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        print(f"short rows M={M} N={N} K={K} g={group} algo={algo}", flush=True)
        rc = lib.tlq_gemm_w4a16(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, 0.0, _abi.F16, _abi.F16, algo,
                                torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        if algo == _abi.ALGO_DECODE and K == 256:
            assert rc != 0 and "decode kernel" in _abi.last_error()
            continue
        assert rc == 0, _abi.last_error()
        check_float_output(C.cpu(), want, f"short rows algo {algo}")


@pytest.mark.gpu
def test_automatic_choice_takes_the_decode_kernel_and_no_workspace_is_needed_for_short_rows():
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, N, K, group = 16, 2048, 4096, 128
    A = torch.randn(M, K, generator=gen(84)).to(torch.float16)
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=85)
    a = run_decode(A, Wp, s, z, group)
    b = run_decode(A, Wp, s, z, group, algo=_abi.ALGO_AUTO)
    assert_bit_equal(a, b, "auto vs decode")
    C = torch.empty(M, N, dtype=torch.float16, device="cuda")
    dA, dW, dS, dZ = A.cuda(), Wp.cuda(), s.cuda(), z.cuda()
    _abi.check(lib.tlq_gemm_w4a16(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, 0.0, _abi.F16, _abi.F16, _abi.ALGO_DECODE, None))
    torch.cuda.synchronize()
    assert_bit_equal(C.cpu(), a, "no-workspace entry point")
    # rows of 8192 values need the workspace: the entry point without one says so
    t = torch.zeros(64, dtype=torch.float16, device="cuda")
    rc = lib.tlq_gemm_w4a16(P(t), P(t), None, None, P(t), 4, 16, 8192, 128, 8.0, _abi.F16, _abi.F16, _abi.ALGO_DECODE, None)
    assert rc != 0 and "decode kernel" in _abi.last_error()
    # and the skinny kernel still serves whoever switches the decode kernel off
    lib.tlq_tune_w4a16_decode(0)
    try:
        c = run_decode(A, Wp, s, z, group, algo=_abi.ALGO_AUTO)
    finally:
        lib.tlq_tune_w4a16_decode(1)
    check_float_output(c, w4a16_reference(A, Wp, s, z, group), "skinny kernel with the decode kernel off")
