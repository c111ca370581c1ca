"""The streaming W4A16 kernel (TLQ_ALGO_STREAM through tlq_gemm_w4a16_ws: 17 <= M <= 512, weights streamed once per 128
activation rows, packed words dequantised in registers) against the oracle: ragged M and N, every ring depth, one and many
K slices, all zero-point kinds and group sizes, both activation types; and with one-hot activations the outputs must be
the dequantised weights bit for bit."""
import pytest
import torch

from helpers import DT, assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference
from oracle import ref

pytestmark = pytest.mark.gpu


def run_stream(A, Wp, s, z, group, out_dtype=None, algo=None):
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
    st = torch.cuda.current_stream().cuda_stream
    print(f"stream M={M} N={N} K={K} g={group} {A.dtype} workspace={need}", flush=True)
    _abi.check(lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, code[A.dtype], code[out_dtype],
                                     _abi.ALGO_STREAM if algo is None else algo, P(ws), need, st))
    torch.cuda.synchronize()
    return C.cpu()


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,zeros_kind", [
    (17, 256, 128, 128, "int"), (32, 260, 256, 32, "frac"), (33, 1000, 512, 64, "scalar8"), (64, 2048, 4096, 128, "int"),
    (65, 520, 1152, 128, None), (100, 4096, 2048, 256, "int"), (128, 3072, 1024, 64, "frac"), (200, 516, 640, 128, "int"),
    (512, 1024, 2048, 128, "scalar8"), (48, 14336, 4096, 128, "int"), (96, 4096, 14336, 64, "int"),
    # one scale per weight row (group = K) and other groups longer than a K slice: the slices are parts of one group
    (64, 2048, 4096, 4096, "int"), (200, 1024, 2048, 1024, "frac"), (48, 4096, 8192, 8192, "scalar8"), (300, 512, 4096, 2048, "int"),
    (128, 3072, 4096, 4096, None),
])
def test_stream_against_the_oracle(in_dtype, M, N, K, group, zeros_kind):
    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(50)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=51)
    got = run_stream(A, Wp, s, z, group)
    check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"stream {in_dtype} {M}x{N}x{K} g{group} {zeros_kind}")


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("zeros_kind", [None, "scalar8", "int", "frac"])
def test_stream_one_hot_rows_return_the_dequantised_weights(in_dtype, zeros_kind):
    """A = rows of the identity: C[m, n] = W[n, m] exactly (one non-zero product per output), for fp32 and 16-bit outputs."""
    dt = DT[in_dtype]
    N, K, group, M = 528, 512, 64, 320
    A = torch.eye(K, dtype=dt)[torch.randperm(K, generator=gen(52))[:M]]
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=53)
    W = ref.dequant_w4(Wp, s, z, group, dt)
    cols = A.float().argmax(dim=1)
    want = W[:, cols].T.contiguous()
    assert_bit_equal(run_stream(A, Wp, s, z, group), want, f"one-hot {in_dtype} zeros={zeros_kind}")
    assert_bit_equal(run_stream(A, Wp, s, z, group, torch.float32), want.float(), f"one-hot f32 out {in_dtype} zeros={zeros_kind}")


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,slice_steps,zeros_kind", [
    # a slice longer than the 16 groups whose scales a wavefront holds runs in windows (4 / 8 / 16 steps of 128 values for
    # groups of 32 / 64 / 128): whole and ragged last windows, one and several slices, every activation tile count
    (20, 300, 128 * 11, 32, 11, "int"), (50, 516, 128 * 11, 32, 6, "frac"), (130, 260, 128 * 9, 32, 9, "scalar8"),
    (40, 264, 128 * 19, 64, 19, "int"), (200, 512, 128 * 19, 64, 10, None), (300, 256, 128 * 16, 64, 16, "mixed"),
    (64, 256, 128 * 35, 128, 35, "int"), (48, 1028, 128 * 35, 128, 18, "mixed"), (24, 256, 128 * 12, 32, 12, "mixed"),
    (256, 2048, 4096, 64, 0, "int"), (256, 14336, 4096, 64, 0, "int"),
    # large groups: windows of 32 and 64 steps
    (64, 256, 128 * 80, 256, 80, "int"), (40, 260, 128 * 72, 512, 72, "frac"),
    # slices that are a part of one group (4, 8 and 16 steps of groups of 32 steps; 2 steps of groups of 4)
    (64, 256, 128 * 32, 4096, 8, "int"), (100, 516, 128 * 64, 4096, 4, "frac"), (200, 260, 128 * 32, 4096, 16, "mixed"), (24, 256, 128 * 8, 512, 2, "int"),
])
def test_stream_windows_of_a_long_slice(in_dtype, M, N, K, group, slice_steps, zeros_kind):
    from tilelang_ascend_amd import _abi

    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(56)).to(dt)
    mixed = zeros_kind == "mixed"  # integral zero points in the first windows, fractional ones later: the dequantiser changes on the way
    Wp, s, z = make_w4(N, K, group, dt, "int" if mixed else zeros_kind, seed=57)
    if mixed:
        _, _, zf = make_w4(N, K, group, dt, "frac", seed=58)
        z = z.clone()
        z[:, 20:] = zf[:, 20:]
    lib = _abi.load()
    lib.tlq_tune_w4a16_stream_slice(slice_steps)
    try:
        got = run_stream(A, Wp, s, z, group)
    finally:
        lib.tlq_tune_w4a16_stream_slice(0)
    check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"windows {in_dtype} {M}x{N}x{K} g{group} slice {slice_steps} {zeros_kind}")


def test_stream_rejects_what_it_cannot_do():
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    t = torch.zeros(64, dtype=torch.float16, device="cuda")
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    for M, N, K, group in ((16, 256, 128, 128), (600, 256, 128, 128), (64, 256, 192, 64), (64, 256, 256, 96), (64, 254, 256, 128)):
        rc = lib.tlq_gemm_w4a16_ws(P(t), P(t), None, None, P(t), M, N, K, group, 8.0, _abi.F16, _abi.F16, _abi.ALGO_STREAM,
                                   P(ws), 1 << 20, None)
        assert rc != 0 and "streaming kernel" in _abi.last_error(), (M, N, K, group)


def test_automatic_choice_takes_the_streaming_kernel_and_agrees_with_it():
    from tilelang_ascend_amd import _abi

    M, N, K, group = 64, 4096, 4096, 128  # (small problems and short rows at this M -- K <= 2048 on up to 2^24 weights -- go to single-launch kernels instead)
    A = torch.randn(M, K, generator=gen(54)).to(torch.float16)
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=55)
    a = run_stream(A, Wp, s, z, group)
    b = run_stream(A, Wp, s, z, group, algo=_abi.ALGO_AUTO)
    assert_bit_equal(a, b, "auto vs stream")
