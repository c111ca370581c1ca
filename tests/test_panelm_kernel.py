"""The middle-M panel kernel (TLQ_ALGO_PANELM through tlq_gemm_w4a16_ws: 64 or 128 activation rows x 256 weight rows per
work-group of four wavefronts, a ring of four / three LDS slots, scales and zero points through LDS windows, a zero-point
tensor handled inside the one launch -- the fused form of the reference's unpack-then-GEMM wrapper,
examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:176-223, for tens to hundreds of activation rows).

Without a GPU: its plan, the host walk over every direct load, LDS cell and operand read of a launch, and its schedule of
loads, waits, barriers and LDS reads played through on the host (with wait counts one too loose it must fail).  On the GPU:
against the oracle for both tile heights, all zero-point kinds (fractional zero points that start in a later window make
the kernel change dequantiser on the way), groups of 64 to 1024 values, one and many K slices, both activation types;
with one-hot activations the outputs must be the dequantised weights bit for bit."""
import ctypes

import pytest
import torch

from helpers import DT, assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference
from oracle import ref

CODE = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}


def plan_of(M, N, K, group, cus=256):
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    out = (ctypes.c_int64 * 5)()
    ok = lib.tlq_debug_panelm_plan(M, N, K, group, cus, out)
    return bool(ok), dict(tiles_m=out[0], tiles_n=out[1], split=out[2], slice_steps=out[3], rows=out[4])


def window_of(group):
    return 8 * group // 128 if group >= 128 else 8 // (128 // group)


@pytest.mark.parametrize("M,N,K,group", [
    (256, 14336, 4096, 128), (64, 14336, 4096, 128), (512, 4096, 14336, 64), (132, 1040, 2048, 64), (100, 272, 8192, 1024),
    (48, 1024, 4096, 128), (384, 8192, 8192, 256), (4, 16, 1024, 128), (192, 528, 4096, 128),
])
def test_plan_and_host_walk(M, N, K, group):
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    ok, p = plan_of(M, N, K, group)
    assert ok, (M, N, K, group)
    steps, window = K // 128, window_of(group)
    assert p["rows"] in (64, 128)
    assert p["tiles_m"] == -(-M // p["rows"]) and p["tiles_n"] == -(-N // 256)
    assert p["split"] == -(-steps // p["slice_steps"])
    assert p["split"] == 1 or p["slice_steps"] % window == 0  # slices are whole windows of eight groups
    assert window >= (4 if p["rows"] == 64 else 3)            # a window spans the ring
    assert lib.tlq_debug_check_panelm_addressing(M, N, K, group, p["rows"], p["slice_steps"]) == 0, _abi.last_error()
    if steps > window:  # the shortest slices
        assert lib.tlq_debug_check_panelm_addressing(M, N, K, group, p["rows"], window) == 0, _abi.last_error()


def test_plan_refuses_what_the_kernel_does_not_take():
    for M, N, K, group in [(258, 4096, 4096, 128),    # M % 4
                           (256, 4104, 4096, 128),    # N % 16
                           (256, 4096, 4160, 128),    # K % 128
                           (256, 4096, 4096, 96),     # group not a power of two
                           (256, 4096, 2048, 512),    # four groups per row: no whole window of eight
                           (256, 4096, 11008, 128),   # 86 groups per row
                           (256, 4096, 4096, 32)]:    # windows of two steps: shorter than the ring
        assert not plan_of(M, N, K, group)[0], (M, N, K, group)
    # groups of 64 values give windows of four steps: the ring of three slots (128 rows) and of four (64 rows) both fit
    assert plan_of(64, 4096, 4096, 64)[0] and plan_of(256, 4096, 4096, 64)[0]


def test_schedule_on_the_host():
    """The kernel's own wait counts pass for both tile heights and for windows as short as the ring; a wait that leaves one
    load more outstanding than the data it guards allows must fail, and so must a window shorter than the ring."""
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    for rows, depth, wait_w, wait_a in ((64, 4, 20, 20), (128, 3, 20, 16)):
        for steps in (1, 2, 5, 32):
            for window in (depth, 8, 16):
                assert lib.tlq_debug_check_panelm_schedule(rows, steps, window, -1, -1) == 0, _abi.last_error()
        assert lib.tlq_debug_check_panelm_schedule(rows, 16, 8, wait_w, wait_a) == 0  # what the kernel's constants come to
        assert lib.tlq_debug_check_panelm_schedule(rows, 16, 8, wait_w + 1, wait_a) != 0 and "packed weights" in _abi.last_error()
        assert lib.tlq_debug_check_panelm_schedule(rows, 16, 8, wait_w, wait_a + 1) != 0 and "activation tile" in _abi.last_error()
        assert lib.tlq_debug_check_panelm_schedule(rows, 16, 8, wait_w - 4, wait_a - 4) == 0  # (stricter waits only cost time)
        assert lib.tlq_debug_check_panelm_schedule(rows, 16, depth - 1, -1, -1) != 0


def run_panelm(A, Wp, s, z, group, out_dtype=None, rows=0, slice_steps=0, algo=None):
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, K = A.shape
    N = Wp.shape[0]
    out_dtype = out_dtype or A.dtype
    zt = z if torch.is_tensor(z) else None
    zs = 0.0 if (torch.is_tensor(z) or z is None) else float(z)
    dA, dW = A.cuda(), Wp.cuda()
    dS = s.cuda() if s is not None else None
    dZ = zt.cuda() if zt is not None else None
    lib.tlq_tune_w4a16_panel_slice(slice_steps)
    lib.tlq_tune_w4a16_panelm_rows(rows)
    try:
        ok, p = plan_of(M, N, K, group)
        assert ok
        assert lib.tlq_debug_check_panelm_addressing(M, N, K, group, p["rows"], p["slice_steps"]) == 0, _abi.last_error()
        need = (p["split"] * M * N * 4 if p["split"] > 1 else 0) + 16
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        C = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
        st = torch.cuda.current_stream().cuda_stream
        print(f"panelm M={M} N={N} K={K} g={group} {A.dtype} plan={p}", flush=True)
        _abi.check(lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, CODE[A.dtype], CODE[out_dtype],
                                         _abi.ALGO_PANELM if algo is None else algo, P(ws), need, st))
        torch.cuda.synchronize()
    finally:
        lib.tlq_tune_w4a16_panel_slice(0)
        lib.tlq_tune_w4a16_panelm_rows(0)
    return C.cpu()


def make_case(N, K, group, dt, zeros_kind, seed):
    if isinstance(zeros_kind, float):  # a fractional scalar zero point: the unfolded dequantiser without a tensor
        Wp, s, _ = make_w4(N, K, group, dt, None, seed=seed)
        return Wp, s, zeros_kind
    if zeros_kind == "latefrac":  # integral windows first, fractions from the middle of a row on
        Wp, s, z = make_w4(N, K, group, dt, "int", seed=seed)
        z[:, (K // group) // 2 + 1:] += 0.25
        return Wp, s, z
    return make_w4(N, K, group, dt, zeros_kind, seed=seed)


@pytest.mark.gpu
@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,zeros_kind,rows", [
    (64, 256, 1024, 128, "int", 0), (128, 512, 1024, 128, "int", 0), (200, 528, 2048, 64, "scalar8", 0), (132, 1040, 2048, 64, "frac", 0),
    (300, 704, 4096, 128, "frac", 0), (64, 512, 4096, 256, None, 0), (48, 1024, 4096, 128, "int", 0), (260, 512, 8192, 128, "int", 0),
    (512, 1024, 2048, 128, None, 0), (256, 512, 2048, 64, "int", 64), (64, 768, 4096, 128, "int", 128), (100, 272, 8192, 1024, "latefrac", 0),
    (192, 512, 4096, 128, 7.5, 0), (96, 512, 4096, 128, "latefrac", 0), (256, 256, 4096, 64, "latefrac", 64), (4, 16, 1024, 128, "scalar8", 0),
])
def test_panelm_against_the_oracle(in_dtype, M, N, K, group, zeros_kind, rows):
    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(70)).to(dt)
    Wp, s, z = make_case(N, K, group, dt, zeros_kind, 71)
    # (a handful of outputs rounded to bfloat16 are too few for a relative L2 bar of 1e-3: one flipped last bit among 64
    # values is 2e-3 of the norm; the smallest case is checked in fp32)
    out_dtype = torch.float32 if M * N < 1024 else dt
    got = run_panelm(A, Wp, s, z, group, rows=rows, out_dtype=out_dtype)
    check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"panelm {in_dtype} {M}x{N}x{K} g{group} {zeros_kind} rows {rows}")


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [64, 128])
@pytest.mark.parametrize("group,windows", [(128, 1), (64, 1), (64, 3), (256, 1), (128, 2)])
def test_panelm_k_slices_of_whole_windows(rows, group, windows):
    """Forced slice lengths from one window up, with a ragged last slice; fractional zero points in the later windows only,
    so that a work-group changes dequantiser part of the way through its slice or starts with the unfolded one."""
    M, N, K = 196, 528, 4096 + 128 * window_of(group)
    for dt in (torch.float16, torch.bfloat16):
        A = torch.randn(M, K, generator=gen(72)).to(dt)
        Wp, s, z = make_case(N, K, group, dt, "latefrac", 73)
        got = run_panelm(A, Wp, s, z, group, rows=rows, slice_steps=windows * window_of(group))
        check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"panelm slices g{group} x{windows} rows {rows} {dt}")


@pytest.mark.gpu
@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("zeros_kind", [None, "scalar8", "int", "frac", "latefrac"])
@pytest.mark.parametrize("rows", [64, 128])
def test_panelm_one_hot_rows_return_the_dequantised_weights(in_dtype, zeros_kind, rows):
    """A = rows of the identity: C[m, n] = W[n, m] exactly (one non-zero product per output), for 16-bit and fp32 outputs."""
    dt = DT[in_dtype]
    N, K, group, M = 528, 2048, 64, 320
    A = torch.eye(K, dtype=dt)[torch.randperm(K, generator=gen(74))[:M]]
    Wp, s, z = make_case(N, K, group, dt, zeros_kind, 75)
    W = ref.dequant_w4(Wp, s, z, group, dt)
    want = (A.float() @ W.float().T)
    for out_dtype in (dt, torch.float32):
        got = run_panelm(A, Wp, s, z, group, out_dtype=out_dtype, rows=rows)
        assert_bit_equal(got, want.to(out_dtype), f"panelm one-hot {in_dtype} {zeros_kind} rows {rows} -> {out_dtype}")


@pytest.mark.gpu
def test_automatic_choice_takes_the_middle_m_kernel_on_large_matrices_and_agrees():
    """tlq_gemm_w4a16_ws with the automatic choice and a workspace of tlq_w4a16_workspace_bytes at 256 rows on a matrix of
    2^25 weights or more: equal, bit for bit, to the explicit call (same kernel), and within the bar of the oracle."""
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, N, K, group = 256, 8192, 4096, 128
    dt = torch.float16
    A = torch.randn(M, K, generator=gen(76)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, "int", seed=77)
    need = lib.tlq_w4a16_workspace_bytes(M, N, K)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=dt, device="cuda")
    dA, dW, dS, dZ = A.cuda(), Wp.cuda(), s.cuda(), z.cuda()
    st = torch.cuda.current_stream().cuda_stream
    _abi.check(lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, 0.0, _abi.F16, _abi.F16, _abi.ALGO_AUTO, P(ws), need, st))
    torch.cuda.synchronize()
    explicit = run_panelm(A, Wp, s, z, group)
    assert_bit_equal(C.cpu(), explicit, "automatic choice vs explicit middle-M panel kernel")
    check_float_output(explicit, w4a16_reference(A, Wp, s, z, group), "middle-M panel kernel via the automatic choice")
