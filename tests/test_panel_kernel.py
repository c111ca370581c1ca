"""The panel kernels (TLQ_ALGO_PANEL256 and TLQ_ALGO_PANEL through tlq_gemm_w4a16_ws / tlq_gemm_w4a16_layout_ws: large M in
one launch, 256 activation rows x 256 weight rows on four wavefronts or 128 x 512 on eight per work-group, packed weights
copied global -> LDS as they are and dequantised on the MFMA operand read -- the fused form of the reference's
unpack-then-GEMM wrapper, examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:176-223).

Without a GPU: their plans, the host walk over every direct load, gather, LDS cell and operand read of a launch, and for
the 256-row kernel its schedule of loads, waits and barriers played through on the host (with wrong wait counts it must
fail).  On the GPU: against the oracle on ragged shapes, all zero-point kinds (a zero-point tensor with fractional values
makes the 256-row kernel change dequantiser on the way and the 128-row kernel take a second, unfolded launch), every group size, one and many K slices, both activation types and both word layouts;
with one-hot activations the outputs must be the dequantised weights bit for bit."""
import ctypes

import pytest
import torch

from helpers import DT, assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference
from oracle import ref

CODE = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}


KERNELS = ["panel256", "panel"]
TILE = {"panel256": (256, 256), "panel": (128, 512)}


def algo_of(kernel):
    from tilelang_ascend_amd import _abi

    return {"panel256": _abi.ALGO_PANEL256, "panel": _abi.ALGO_PANEL}[kernel]


def plan_of(M, N, K, group, cus=256, kernel="panel"):
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    out = (ctypes.c_int64 * 4)()
    ok = (lib.tlq_debug_panel256_plan if kernel == "panel256" else lib.tlq_debug_panel_plan)(M, N, K, group, cus, out)
    return bool(ok), dict(tiles_m=out[0], tiles_n=out[1], split=out[2], slice_steps=out[3])


def walk(kernel, M, N, K, group, slice_steps):
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    fn = lib.tlq_debug_check_panel256_addressing if kernel == "panel256" else lib.tlq_debug_check_panel_addressing
    assert fn(M, N, K, group, slice_steps) == 0, _abi.last_error()


@pytest.mark.parametrize("M,N,K,group", [
    (4096, 4096, 4096, 128), (1000, 1040, 1024, 32), (132, 528, 2048, 64), (8192, 14336, 4096, 128), (1024, 4096, 14336, 64),
    (260, 4096, 8192, 256), (128, 512, 8192, 1024), (4, 16, 1024, 128), (516, 16, 128 * 24, 64),
])
@pytest.mark.parametrize("kernel", KERNELS)
def test_plan_and_host_walk(kernel, M, N, K, group):
    ok, p = plan_of(M, N, K, group, kernel=kernel)
    assert ok, (M, N, K, group)
    steps = K // 128
    # slices are whole windows of eight groups (128-row kernel: its scale windows) or whole groups (256-row kernel)
    if kernel == "panel":
        unit = 8 * group // 128 if group >= 128 else 8 // (128 // group)
    else:
        unit = max(group // 128, 1)
    bm, bn = TILE[kernel]
    assert p["tiles_m"] == -(-M // bm) and p["tiles_n"] == -(-N // bn)
    assert p["split"] == -(-steps // p["slice_steps"])
    assert p["split"] == 1 or p["slice_steps"] % unit == 0 or (kernel == "panel256" and unit % p["slice_steps"] == 0)
    walk(kernel, M, N, K, group, p["slice_steps"])
    if steps > unit:  # the shortest slices the plan may take
        walk(kernel, M, N, K, group, unit)


def test_256_row_kernel_cuts_k_inside_a_group_that_is_longer_than_a_slice():
    """One scale per weight row (group = K) and few tiles: the plan of the 256-row kernel cuts K into power-of-two parts of
    the group (every step takes its group from its position in K), the host walk covers such slices, and a part that does
    not divide the group is refused by the walk."""
    from tilelang_ascend_amd import _abi

    ok, p = plan_of(768, 4096, 8192, 8192, kernel="panel256")
    assert ok and p["split"] > 1 and 64 % p["slice_steps"] == 0 and p["slice_steps"] >= 16, p
    walk("panel256", 768, 4096, 8192, 8192, p["slice_steps"])
    walk("panel256", 260, 528, 4096, 4096, 8)
    assert _abi.load().tlq_debug_check_panel256_addressing(260, 528, 4096, 4096, 12) != 0 and "even part" in _abi.last_error()


def test_schedule_of_the_256_row_kernel_on_the_host():
    """The kernel's own wait counts pass for any number of steps; a wait that leaves one load more outstanding than the
    data it guards allows must fail (stricter waits only cost time)."""
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    for steps in (1, 2, 3, 5, 32):
        assert lib.tlq_debug_check_panel256_schedule(steps, -1, -1) == 0, _abi.last_error()
    assert lib.tlq_debug_check_panel256_schedule(4, 24, 0) == 0  # what the kernel's constants must come to
    assert lib.tlq_debug_check_panel256_schedule(4, 25, 0) != 0 and "packed weights" in _abi.last_error()
    assert lib.tlq_debug_check_panel256_schedule(4, 24, 1) != 0 and "barrier" in _abi.last_error()
    assert lib.tlq_debug_check_panel256_schedule(4, 20, 0) == 0


def test_plan_refuses_what_the_kernel_does_not_take():
    for M, N, K, group in [(4098, 4096, 4096, 128),   # M % 4
                           (4096, 4104, 4096, 128),   # N % 16
                           (4096, 4096, 4160, 128),   # K % 128
                           (4096, 4096, 4096, 96)]:   # group not a power of two
        for kernel in KERNELS:
            assert not plan_of(M, N, K, group, kernel=kernel)[0], (kernel, M, N, K, group)
    for M, N, K, group in [(4096, 4096, 2048, 512),   # four groups per row: no whole window of eight
                           (4096, 4096, 11008, 128)]:  # 86 groups per row
        assert not plan_of(M, N, K, group, kernel="panel")[0], (M, N, K, group)
        assert plan_of(M, N, K, group, kernel="panel256")[0], (M, N, K, group)  # (its scales do not pass through windows)


def test_few_tiles_cut_k_into_whole_windows():
    ok, p = plan_of(1024, 4096, 14336, 128)
    assert ok and p["split"] > 1 and p["slice_steps"] % 8 == 0
    ok, p = plan_of(4096, 4096, 4096, 128)
    assert ok and p["split"] == 1 and p["slice_steps"] == 32
    ok, p = plan_of(1024, 4096, 14336, 128, kernel="panel256")  # 4 x 16 tiles on 256 CUs
    assert ok and p["split"] > 1 and p["slice_steps"] >= 16
    ok, p = plan_of(4096, 4096, 4096, 128, kernel="panel256")
    assert ok and p["split"] == 1 and p["slice_steps"] == 32 and p["tiles_m"] * p["tiles_n"] == 256


def run_panel(A, Wp, s, z, group, out_dtype=None, layout=0, kernel="panel256", slice_steps=0):
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
    try:
        ok, p = plan_of(M, N, K, group, kernel=kernel)
        assert ok
        walk(kernel, M, N, K, group, p["slice_steps"])
        need = (p["split"] * M * N * 4 if p["split"] > 1 else 0) + 16
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        C = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
        st = torch.cuda.current_stream().cuda_stream
        print(f"{kernel} M={M} N={N} K={K} g={group} {A.dtype} layout={layout} plan={p}", flush=True)
        _abi.check(lib.tlq_gemm_w4a16_layout_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, CODE[A.dtype], CODE[out_dtype],
                                                algo_of(kernel), layout, P(ws), need, st))
        torch.cuda.synchronize()
    finally:
        lib.tlq_tune_w4a16_panel_slice(0)
    return C.cpu()


@pytest.mark.gpu
@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,zeros_kind", [
    (128, 512, 1024, 128, "int"), (200, 528, 2048, 64, "scalar8"), (132, 1040, 1024, 32, "frac"), (300, 704, 4096, 128, "frac"),
    (64, 512, 2048, 256, None), (1024, 1024, 4096, 128, "int"), (260, 512, 8192, 128, "int"), (4, 16, 1024, 128, "scalar8"),
    (516, 2064, 1024, 128, 7.5), (1536, 4096, 4096, 128, "int"), (640, 1024, 8192, 1024, "int"),
])
def test_panel_against_the_oracle(kernel, in_dtype, M, N, K, group, zeros_kind):
    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(60)).to(dt)
    if isinstance(zeros_kind, float):  # a fractional scalar zero point: the unfolded kernel without a tensor
        Wp, s, _ = make_w4(N, K, group, dt, None, seed=61)
        z = zeros_kind
    else:
        Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=61)
    got = run_panel(A, Wp, s, z, group, kernel=kernel)
    check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"{kernel} {in_dtype} {M}x{N}x{K} g{group} {zeros_kind}")


@pytest.mark.gpu
@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,slice_steps,zeros_kind", [
    (768, 2048, 8192, 8192, 0, "int"), (1024, 1024, 4096, 4096, 16, "frac"), (260, 528, 4096, 4096, 8, "scalar8"), (516, 1040, 8192, 2048, 4, "int"),
])
def test_256_row_kernel_with_slices_inside_one_group(in_dtype, M, N, K, group, slice_steps, zeros_kind):
    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(67)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=68)
    got = run_panel(A, Wp, s, z, group, kernel="panel256", slice_steps=slice_steps)
    check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"panel256 {in_dtype} {M}x{N}x{K} g{group} slices of {slice_steps} {zeros_kind}")


@pytest.mark.gpu
@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("group,slice_steps", [(128, 8), (64, 4), (32, 2), (32, 6), (256, 16), (128, 24)])
def test_panel_k_slices_of_whole_windows(kernel, group, slice_steps):
    """Forced slice lengths from one window up, with a ragged last slice; fractional zero points in the later windows only,
    so that the folded launch gives up part of the way through."""
    M, N, K = 260, 1040, 4096
    for dt in (torch.float16, torch.bfloat16):
        A = torch.randn(M, K, generator=gen(62)).to(dt)
        Wp, s, z = make_w4(N, K, group, dt, "int", seed=63)
        z[:, (K // group) // 2 + 1:] += 0.25  # integral windows first
        got = run_panel(A, Wp, s, z, group, kernel=kernel, slice_steps=slice_steps)
        check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"{kernel} slices g{group} s{slice_steps} {dt}")


@pytest.mark.gpu
@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("zeros_kind", [None, "scalar8", "int", "frac"])
@pytest.mark.parametrize("layout", [0, 1])
def test_panel_one_hot_rows_return_the_dequantised_weights(kernel, in_dtype, zeros_kind, layout):
    """A = rows of the identity: C[m, n] = W[n, m] exactly (one non-zero product per output), in both word layouts, for
    16-bit and fp32 outputs."""
    dt = DT[in_dtype]
    N, K, group, M = 528, 1024, 64, 320
    A = torch.eye(K, dtype=dt)[torch.randperm(K, generator=gen(64))[:M]]
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=65)
    W = ref.dequant_w4(Wp, s, z, group, dt)
    words = Wp
    if layout == 1:
        words = ref.interleave_weight(Wp.view(torch.int8), 4, "float16").view(torch.uint8).contiguous()
    want = (A.float() @ W.float().T)
    for out_dtype in (dt, torch.float32):
        got = run_panel(A, words, s, z, group, out_dtype=out_dtype, layout=layout, kernel=kernel)
        assert_bit_equal(got, want.to(out_dtype), f"{kernel} one-hot {in_dtype} {zeros_kind} layout {layout} -> {out_dtype}")


@pytest.mark.gpu
@pytest.mark.parametrize("kernel", KERNELS)
def test_tiny_scales_round_like_the_reference(kernel):
    """Scales so small that products are subnormal in the activation type: the folded dequantiser forms (u - z) s in fp32
    and rounds once, which must give what the reference's multiplication in the activation type gives."""
    N, K, group, M = 512, 1024, 128, 128
    for dt in (torch.float16, torch.bfloat16):
        A = torch.eye(K, dtype=dt)[:M]
        Wp, s, z = make_w4(N, K, group, dt, "int", seed=66)
        tiny = 2.0 ** -20 if dt == torch.float16 else 2.0 ** -100
        s = (s.float() * tiny / 0.01).to(dt)
        W = ref.dequant_w4(Wp, s, z, group, dt)
        got = run_panel(A, Wp, s, z, group, out_dtype=dt, kernel=kernel)
        assert_bit_equal(got, (A.float() @ W.float().T).to(dt), f"{kernel} tiny scales {dt}")


@pytest.mark.gpu
def test_automatic_choice_takes_the_256_row_panel_kernel_above_512_rows_and_agrees():
    """tlq_gemm_w4a16_ws with the automatic choice and a workspace of tlq_w4a16_workspace_bytes on a shape whose 256-row
    tiles fill the machine: equal, bit for bit, to the explicit call (same kernel), and within the bar of the oracle."""
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, N, K, group = 1024, 16384, 1024, 128  # 4 x 64 tiles of 256 x 256: one full round
    dt = torch.float16
    A = torch.randn(M, K, generator=gen(67)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, "int", seed=68)
    need = lib.tlq_w4a16_workspace_bytes(M, N, K)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=dt, device="cuda")
    dA, dW, dS, dZ = A.cuda(), Wp.cuda(), s.cuda(), z.cuda()
    st = torch.cuda.current_stream().cuda_stream
    _abi.check(lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, 0.0, _abi.F16, _abi.F16, _abi.ALGO_AUTO, P(ws), need, st))
    torch.cuda.synchronize()
    explicit = run_panel(A, Wp, s, z, group, kernel="panel256")
    assert_bit_equal(C.cpu(), explicit, "automatic choice vs explicit 256-row panel kernel")
    check_float_output(explicit, w4a16_reference(A, Wp, s, z, group), "panel via the automatic choice")
