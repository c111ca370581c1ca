"""GPU parity tests: every HIP kernel, called through the C ABI (via the operator layer), against
the CPU oracle on identical seeded inputs.

Bars: integer / byte results and dequantised weights bit exact; float GEMM outputs within
relative L2 1e-3, max-abs 1e-2 (on top of the output type's own rounding) and
assert_close(rtol=atol=1e-2) of the fp32-accumulated reference.
"""
import numpy as np
import pytest
import torch

from helpers import DT, assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference
from oracle import ref

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from tilelang_ascend_amd import _abi, ops

    _abi.load()  # fail loudly if the HIP library is missing
    return ops


@pytest.fixture(autouse=True)
def _name_case(request):
    print(f"[case] {request.node.nodeid}", flush=True)
    yield
    torch.cuda.synchronize()


# ------------------------------------------------------------------------------------------
# unpack
# ------------------------------------------------------------------------------------------
def test_unpack_known_answer(ops):
    # the reference's own vector: examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:384-401
    kat = torch.tensor([[0x12, 0x34]], dtype=torch.uint8)
    f = ops.torch_unpack_uint4_to_fp16(kat)
    i = ops.torch_unpack_uint4_to_int8(kat)
    assert f.shape == (1, 4) and f.dtype == torch.float16 and f.tolist() == [[2.0, 1.0, 4.0, 3.0]]
    assert i.shape == (1, 4) and i.dtype == torch.int8 and i.tolist() == [[2, 1, 4, 3]]


@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (7, 12), (64, 128), (333, 516), (1024, 2048)])
@pytest.mark.parametrize("mode", ["unsigned", "twos", "offset8", "offset7"])
def test_unpack_modes(ops, shape, mode):
    Wp = torch.randint(0, 256, shape, dtype=torch.uint8, generator=gen(1))
    u = ref.unpack_uint4(Wp).astype(np.int16)
    want = {"unsigned": u, "twos": np.where(u >= 8, u - 16, u), "offset8": u - 8, "offset7": u - 7}[mode]
    for dt in (torch.int8, torch.float16, torch.bfloat16):
        got = ops.unpack_int4(Wp.cuda(), dt, mode).cpu()
        assert_bit_equal(got, torch.from_numpy(want.astype(np.float32)).to(dt), f"unpack {mode} {dt}")


def test_unpack_all_bytes_and_empty(ops):
    Wp = torch.arange(256, dtype=torch.uint8).reshape(1, 256)
    assert_bit_equal(ops.torch_unpack_uint4_to_int8(Wp), ref.torch_unpack_uint4_to_int8(Wp), "all bytes")
    assert_bit_equal(ops.torch_convert(Wp), ref.torch_convert(Wp), "all bytes signed")
    empty = torch.empty(0, 8, dtype=torch.uint8)
    assert ops.torch_unpack_uint4_to_fp16(empty).shape == (0, 16)


# ------------------------------------------------------------------------------------------
# per-group dequantisation: bit exact
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("zeros_kind", [None, "scalar8", "int", "frac"])
@pytest.mark.parametrize("N,K,group", [(16, 64, 32), (256, 256, 128), (100, 384, 64), (64, 512, 512), (8, 12, 4)])
def test_dequant_bit_exact(ops, dtype, zeros_kind, N, K, group):
    dt = DT[dtype]
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=2)
    want = ref.dequant_w4(Wp, s, z, group, dt)
    zd = z.cuda() if isinstance(z, torch.Tensor) else z
    got = ops.dequantize_w4(Wp.cuda(), s.cuda(), zd, group, dt).cpu()
    assert_bit_equal(got, want, f"dequant {dtype} zeros={zeros_kind}")


def test_dequant_headline_shape_bit_exact(ops):
    # decode-GEMV weights of the headline configuration: N=11008, K=4096, group 128, fp16 scales + zeros
    Wp, s, z = make_w4(11008, 4096, 128, torch.float16, "int", seed=3)
    got = ops.dequantize_w4(Wp.cuda(), s.cuda(), z.cuda(), 128, torch.float16).cpu()
    assert_bit_equal(got, ref.dequant_w4(Wp, s, z, 128, torch.float16), "dequant 11008x4096")


# ------------------------------------------------------------------------------------------
# W4A16 GEMV (split-K wavefront kernel)
# ------------------------------------------------------------------------------------------
def _run_w4a16(ops, A, Wp, s, z, group, out_dtype, algo, in_dtype):
    M, K = A.shape
    N = Wp.shape[0]
    wrapper = ops.dequant_gemm_fp16_wrapper(M, N, K, 128, 256, 64, in_dtype, out_dtype, group_size=group, algo=algo)
    zd = z.cuda() if isinstance(z, torch.Tensor) else z
    return wrapper(A.cuda(), Wp.cuda(), None if s is None else s.cuda(), zd).cpu()


@pytest.mark.parametrize("rows,waves", [(0, 0), (1, 1), (1, 4), (2, 2), (4, 4), (-1, 4), (-2, 2), (0, 7), (0, 16)])
def test_gemv_headline(ops, rows, waves):
    """M=1, N=11008, K=4096, group 128, fp16 scales U[0.005,0.02], fp16 zeros U{6..9}, fp16 out."""
    from tilelang_ascend_amd import _abi

    M, N, K, group = 1, 11008, 4096, 128
    A = torch.randn(M, K, generator=gen(4)).to(torch.float16)
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=5)
    want = w4a16_reference(A, Wp, s, z, group)
    _abi.load().tlq_tune_gemv(rows, waves)
    try:
        got = _run_w4a16(ops, A, Wp, s, z, group, "float16", "gemv", "float16")
    finally:
        _abi.load().tlq_tune_gemv(0, 0)
    check_float_output(got, want, f"gemv rows={rows} waves={waves}")


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("N,K,group", [
    (49152, 8192, 128), (8192, 16384, 64), (1031, 16384, 32),
    # 28 and 86 groups per row (no multiples of eight: the scales of a work-group's rows are still whole 16-byte pieces), more
    # rows per CU than LDS holds scales for (several equal work-groups per CU), and a row count with which they are no whole pieces
    (152064, 3584, 128), (16384, 11008, 128), (12000, 8192, 32), (10001, 3584, 128),
])
def test_gemv_long_rows_and_many_rows(ops, in_dtype, N, K, group):
    """Output-projection-sized decode shapes: rows of 8192 and 16384 values, whose activations alone take 18 - 36 KB of
    the GEMV's LDS, so that the rows a work-group may own are limited by what is left of 64 KB (or the streaming kernel
    takes over).  The kernel runs on all rows; 384 seeded rows plus the first and last ones are compared with the oracle."""
    dt = DT[in_dtype]
    A = torch.randn(1, K, generator=gen(40)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, "int", seed=41)
    got = _run_w4a16(ops, A, Wp, s, z, group, in_dtype, "auto", in_dtype)
    assert torch.isfinite(got.float()).all()
    rows = torch.cat([torch.arange(0, min(N, 48)), torch.arange(max(0, N - 48), N),
                      torch.randperm(N, generator=gen(42))[:384]]).unique()
    want = w4a16_reference(A, Wp[rows], s[rows], z[rows], group)
    check_float_output(got[:, rows], want, f"gemv {in_dtype} N={N} K={K} g={group}")


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,zeros_kind", [
    (1, 64, 64, 32, None), (1, 250, 2048, 128, "frac"), (2, 1000, 4096, 64, "int"), (3, 77, 1024, 1024, "scalar8"),
    (5, 130, 8192, 128, "int"), (16, 512, 14336, 128, "int"),
])
def test_gemv_shapes(ops, in_dtype, M, N, K, group, zeros_kind):
    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(6)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=7)
    for out_dtype in ("float32", in_dtype):
        got = _run_w4a16(ops, A, Wp, s, z, group, out_dtype, "gemv", in_dtype)
        check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"gemv {in_dtype}->{out_dtype}")


@pytest.mark.parametrize("N,K,group,zeros_kind", [
    (11008, 4096, 128, "int"), (1000, 4096, 32, "int"), (250, 2048, 128, "frac"), (77, 1088, 64, "int"),
    (5, 64, 32, None), (4097, 1024, 1024, "scalar8"), (333, 3136, 64, "frac"), (64, 4096, 4096, "int"),
    # long rows: 3 .. 8 chunks per lane, work-groups of 8 wavefronts
    (4096, 11008, 128, "int"), (520, 14336, 128, "frac"), (300, 6144, 64, "int"), (130, 8192, 32, "scalar8"),
    (77, 16384, 256, "int"), (1000, 4160, 64, "int"), (64, 9984, 128, None),
])
@pytest.mark.parametrize("waves,blocks_per_cu,depth", [(0, 0, 0), (16, 1, 3), (5, 3, 2), (2, 8, 6), (16, 2, 1)])
@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
def test_gemv_register_resident_kernel(ops, in_dtype, N, K, group, zeros_kind, waves, blocks_per_cu, depth):
    """M = 1, K <= 16384: the kernel that keeps the activations in registers and stages the scales and
    zero points of a work-group's rows in LDS, over its grid shapes and queue depths (fp16: biased dot and
    chunk sums; bf16: element-wise dequantisation and the packed dot)."""
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    dt = DT[in_dtype]
    A = torch.randn(1, K, generator=gen(40)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=41)
    want = w4a16_reference(A, Wp, s, z, group)
    lib.tlq_tune_gemv(0, waves)
    lib.tlq_tune_gemv_unroll(blocks_per_cu)
    lib.tlq_tune_gemv_depth(depth)
    try:
        for out_dtype in (in_dtype, "float32"):
            got = _run_w4a16(ops, A, Wp, s, z, group, out_dtype, "gemv", in_dtype)
            check_float_output(got, want, f"gemv rows kernel {in_dtype} -> {out_dtype}")
    finally:
        lib.tlq_tune_gemv(0, 0)
        lib.tlq_tune_gemv_unroll(0)
        lib.tlq_tune_gemv_depth(0)


@pytest.mark.parametrize("M,N,K,group", [(1, 1000, 4096, 128), (1, 130, 8192, 128), (2, 257, 2048, 64)])
def test_gemv_batched_entry_point(M, N, K, group):
    """tlq_gemv_w4a16_batched: several independent problems (own activations, weights, scales, zeros) per launch."""
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    batch = 3
    sets = [make_w4(N, K, group, torch.float16, "int", seed=50 + b) for b in range(batch)]
    A = torch.randn(batch, M, K, generator=gen(49)).to(torch.float16)
    Wp = torch.stack([x[0] for x in sets]).cuda()
    S = torch.stack([x[1] for x in sets]).cuda()
    Z = torch.stack([x[2] for x in sets]).cuda()
    C = torch.empty(batch, M, N, dtype=torch.float16, device="cuda")
    Ad = A.cuda()
    rc = lib.tlq_gemv_w4a16_batched(P(Ad), P(Wp), P(S), P(Z), P(C), batch, M, N, K, group, 0.0, _abi.F16, _abi.F16,
                                    torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _abi.last_error()
    for b in range(batch):
        check_float_output(C[b].cpu(), w4a16_reference(A[b], *sets[b], group), f"batched set {b}")


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,zeros_kind,algo", [
    (2048, 256, 512, 128, "int", "auto"), (100, 136, 256, 64, "frac", "two_pass"), (2304, 72, 192, 32, None, "auto"),
    (16, 64, 128, 128, "scalar8", "two_pass"), (256, 264, 8192, 128, "int", "two_pass"), (2100, 72, 14336, 64, "frac", "auto"),
])
def test_w4a16_two_pass_with_workspace(ops, in_dtype, M, N, K, group, zeros_kind, algo):
    """Dequantise into the kernel object's workspace, then the plain GEMM: what auto does from M = 256 up."""
    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(60)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=61)
    want = w4a16_reference(A, Wp, s, z, group)
    for out_dtype in ("float32", in_dtype):
        got = _run_w4a16(ops, A, Wp, s, z, group, out_dtype, algo, in_dtype)
        check_float_output(got, want, f"two-pass {in_dtype}->{out_dtype}")


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,zeros_kind", [
    (64, 4096, 14336, 128, "int"), (17, 136, 2048, 64, "frac"), (255, 520, 4096, 32, None), (48, 14336, 4096, 128, "scalar8"),
    (130, 64, 8192, 1024, "int"), (32, 4, 1024, 128, "int"), (512, 264, 8192, 128, "int"), (1500, 72, 14336, 64, "frac"),
])
def test_w4a16_mid_m_split_k_with_workspace(ops, in_dtype, M, N, K, group, zeros_kind):
    """Small and middle M with a workspace: the tile kernel over K slices, fp32 partial sums added in slice order."""
    from tilelang_ascend_amd import _abi

    assert _abi.load().tlq_w4a16_workspace_bytes(M, N, K) > 0
    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(70)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=71)
    want = w4a16_reference(A, Wp, s, z, group)
    for out_dtype in ("float32", in_dtype):
        got = _run_w4a16(ops, A, Wp, s, z, group, out_dtype, "auto", in_dtype)
        check_float_output(got, want, f"mid-M split-K {in_dtype}->{out_dtype}")
        again = _run_w4a16(ops, A, Wp, s, z, group, out_dtype, "auto", in_dtype)
        assert torch.equal(got, again), "slice order must make the result reproducible"


def test_w4a16_workspace_entry_point_rules():
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    assert lib.tlq_w4a16_workspace_bytes(2048, 256, 512) == 256 * 512 * 2       # two passes: the dequantised matrix
    assert lib.tlq_w4a16_workspace_bytes(255, 256, 512) == 0                     # K too short to cut, M below the two passes
    assert lib.tlq_w4a16_workspace_bytes(16, 4096, 4096) == 0                    # decode sizes use no workspace
    # 16 K slices of fp32 partial sums, and (rows of 14336 = 7 x 2048 values are no power of two) room for one scale and
    # one zero point per weight row written out per group of 1024: two tensors of 4096 x 14 16-bit values, plus 16 bytes
    assert lib.tlq_w4a16_workspace_bytes(64, 4096, 14336) == 16 * 64 * 4096 * 4 + 2 * 4096 * 14 * 2 + 16
    assert lib.tlq_w4a16_workspace_bytes(64, 4096, 16384) == 16 * 64 * 4096 * 4
    M, N, K, g = 64, 128, 256, 128
    A = torch.randn(M, K, generator=gen(62)).half()
    Wp, s, z = make_w4(N, K, g, torch.float16, "int", seed=63)
    Ad, Wd, sd, zd = A.cuda(), Wp.cuda(), s.cuda(), z.cuda()
    C = torch.empty(M, N, dtype=torch.float16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    args = (P(Ad), P(Wd), P(sd), P(zd), P(C), M, N, K, g, 0.0, _abi.F16, _abi.F16)
    # forced two-pass without (or with a short) workspace is an error, auto falls back to the fused kernels
    assert lib.tlq_gemm_w4a16_ws(*args, _abi.ALGO_TWO_PASS, None, 0, st) != 0 and "workspace" in _abi.last_error()
    ws = torch.empty(N * K * 2, dtype=torch.uint8, device="cuda")
    assert lib.tlq_gemm_w4a16_ws(*args, _abi.ALGO_TWO_PASS, P(ws), N * K * 2 - 1, st) != 0
    assert lib.tlq_gemm_w4a16_ws(*args, _abi.ALGO_AUTO, None, 0, st) == 0
    fused = C.clone()
    assert lib.tlq_gemm_w4a16_ws(*args, _abi.ALGO_TWO_PASS, P(ws), N * K * 2, st) == 0
    want = w4a16_reference(A, Wp, s, z, g)
    check_float_output(fused.cpu(), want, "auto without workspace")
    check_float_output(C.cpu(), want, "forced two-pass")
    # the workspace holds the dequantised matrix, bit for bit
    assert_bit_equal(ws.view(torch.float16).view(N, K).cpu(), ref.dequant_w4(Wp, s, z, g, torch.float16), "workspace")
    assert lib.tlq_gemm_w4a16(*args, _abi.ALGO_TWO_PASS, st) != 0          # not an algo of the plain entry point


def test_gemv_one_hot_reads_back_dequantised_rows(ops):
    """A one-hot activation row makes the output equal one column of the dequantised matrix:
    pins nibble order, group indexing and zero / scale handling inside the fused kernel."""
    N, K, group = 96, 512, 64
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=8)
    W = ref.dequant_w4(Wp, s, z, group, torch.float16)
    for k in (0, 1, 4, 5, 63, 64, 255, 511):
        A = torch.zeros(1, K, dtype=torch.float16)
        A[0, k] = 1.0
        got = _run_w4a16(ops, A, Wp, s, z, group, "float16", "gemv", "float16")
        assert_bit_equal(got[0], W[:, k], f"one-hot k={k}")


# ------------------------------------------------------------------------------------------
# W4A16 MFMA GEMM
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("tile", [0, 16, 32, 64, 128, 256])
@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
def test_gemm_w4a16_tiles(ops, tile, in_dtype):
    from tilelang_ascend_amd import _abi

    dt = DT[in_dtype]
    M, N, K, group = 300, 520, 512, 128  # ragged M and N tails
    A = torch.randn(M, K, generator=gen(9)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, "int", seed=10)
    want = w4a16_reference(A, Wp, s, z, group)
    _abi.load().tlq_tune_w4a16_tile(tile)
    try:
        got = _run_w4a16(ops, A, Wp, s, z, group, "float32", "mfma", in_dtype)
        got16 = _run_w4a16(ops, A, Wp, s, z, group, in_dtype, "mfma", in_dtype)
    finally:
        _abi.load().tlq_tune_w4a16_tile(0)
    check_float_output(got, want, f"w4a16 mfma tile={tile} {in_dtype} f32 out")
    check_float_output(got16, want, f"w4a16 mfma tile={tile} {in_dtype}")


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("zeros_kind", [None, "scalar8", "int", "frac"])
def test_gemm_w4a16_identity_is_dequant(ops, in_dtype, zeros_kind):
    """A = identity => C equals the dequantised weight matrix transposed, bit for bit: the
    'dequantised weights bit exact' requirement checked through the fused GEMM."""
    dt = DT[in_dtype]
    N, K, group = 272, 256, 64
    A = torch.eye(K, dtype=dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=11)
    W = ref.dequant_w4(Wp, s, z, group, dt)
    got = _run_w4a16(ops, A, Wp, s, z, group, in_dtype, "mfma", in_dtype)
    assert_bit_equal(got, W.T.contiguous(), f"identity {in_dtype} zeros={zeros_kind}")


def test_gemm_w4a16_config1_reference_loops(ops):
    """M=N=K=256, fp16, group 128, zero = 8: the reference's own CPU-runnable case, checked against
    the literal per-element unpack loop."""
    M = N = K = 256
    A = torch.randn(M, K, generator=gen(12)).to(torch.float16)
    Wp, s, _ = make_w4(N, K, 128, torch.float16, None, seed=13)
    u = ref.unpack_uint4_loop(Wp, torch.float16)
    W = (u - torch.tensor(8.0, dtype=torch.float16)) * s.repeat_interleave(128, dim=1)
    want = A.float() @ W.float().T
    for algo in ("mfma",):
        got = _run_w4a16(ops, A, Wp, s, 8, 128, "float16", algo, "float16")
        check_float_output(got, want, f"config 1 {algo}")
    # no scales, no zeros: exactly the reference example's wrapper(A, B_packed)
    wrapper = ops.dequant_gemm_fp16_wrapper(M, N, K, 128, 256, 64)
    got = wrapper(A, Wp)
    assert got.device.type == "cpu" and got.dtype == torch.float16
    check_float_output(got, ref.ref_program_fp16_loop(A, Wp, "float32"), "reference wrapper")


@pytest.mark.parametrize("M", [1024, 4096])
def test_gemm_w4a16_prefill_bf16(ops, M):
    """bf16 prefill shape (N=K=4096, group 128, zero = 8, bf16 out): the fused kernel, and what the automatic
    choice does with a workspace (K slices at M = 1024, two passes at M = 4096)."""
    N = K = 4096
    A = torch.randn(M, K, generator=gen(14)).to(torch.bfloat16)
    Wp, s, _ = make_w4(N, K, 128, torch.bfloat16, None, seed=15)
    want = w4a16_reference(A, Wp, s, 8, 128)
    for algo in ("mfma", "auto"):
        got = _run_w4a16(ops, A, Wp, s, 8, 128, "bfloat16", algo, "bfloat16")
        check_float_output(got, want, f"prefill bf16 M={M} {algo}")


@pytest.mark.parametrize("M,N,K,group", [(16, 14336, 4096, 64), (64, 4096, 14336, 128), (256, 14336, 4096, 128)])
def test_gemm_w4a16_mlp_shapes(ops, M, N, K, group):
    A = torch.randn(M, K, generator=gen(16)).to(torch.float16)
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=17)
    got = _run_w4a16(ops, A, Wp, s, z, group, "float16", "auto", "float16")
    check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"mlp {M}x{N}x{K} g{group}")


# ------------------------------------------------------------------------------------------
# int8 paths: bit exact
# ------------------------------------------------------------------------------------------
def _i8(shape, seed, lo=-128, hi=128):
    return torch.randint(lo, hi, shape, dtype=torch.int8, generator=gen(seed))


@pytest.mark.parametrize("tile", [0, 32, 128, 256])
@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (100, 272, 400), (1, 16, 16), (513, 1040, 1024)])
def test_int8_gemm_exact(ops, tile, M, N, K):
    from tilelang_ascend_amd import _abi

    A, B = _i8((M, K), 18), _i8((K, N), 19)
    want = ref.int_matmul_exact(A, B).to(torch.int32)
    _abi.load().tlq_tune_i8_tile(tile)
    try:
        got = ops.int8_gemm(M, N, K, 128, 128, 64)(A.cuda(), B.cuda()).cpu()
    finally:
        _abi.load().tlq_tune_i8_tile(0)
    assert_bit_equal(got, want, f"int8 gemm tile={tile}")


def test_int8_extreme_values(ops):
    # A = B = -128 everywhere, K = 4096: every accumulator is 4096 * 16384 = 67 108 864
    M, N, K = 64, 64, 4096
    A = torch.full((M, K), -128, dtype=torch.int8)
    B = torch.full((K, N), -128, dtype=torch.int8)
    got = ops.int8_gemm(M, N, K, 128, 128, 64)(A.cuda(), B.cuda()).cpu()
    assert (got == 67108864).all()


@pytest.mark.parametrize("out_dtype", ["int32", "float16"])
def test_dequant_gemm_int8_wrapper(ops, out_dtype):
    M = N = K = 256
    A = _i8((M, K), 20, -128, 127)
    Wp = torch.randint(0, 255, (N, K // 2), dtype=torch.uint8, generator=gen(21))
    got = ops.dequant_gemm_int8_wrapper(M, N, K, 128, 128, 64, out_dtype)(A, Wp)
    want = ref.ref_program_int8(A, Wp, out_dtype)
    assert_bit_equal(got, want, "dequant_gemm_int8_wrapper")


@pytest.mark.parametrize("M,N,K", [(64, 64, 256), (128, 128, 512), (256, 256, 1024), (40, 20, 64)])
def test_w4a8(ops, M, N, K):
    g = gen(22)
    A = torch.randint(-8, 8, (M, K), dtype=torch.int8, generator=g)
    qB, B_ref = ref.generate_quantized_weight(N, K, g)
    kernel = ops.w4a8_gemm_cv(M, N, K)
    workspace = torch.zeros(N, K, dtype=torch.int8).cuda()
    C_out = torch.zeros(M, N, dtype=torch.int32).cuda()
    result = kernel(A.cuda(), qB.cuda(), workspace, C_out)  # four positionals, like the reference's caller
    expected = ref.ref_program_w4a8(A, qB)
    assert_bit_equal(result.cpu().transpose(0, 1).contiguous(), expected.contiguous(), "w4a8")
    assert torch.equal(ref.torch_convert(qB), B_ref)


@pytest.mark.parametrize("M,N,K", [(64, 256, 256), (300, 1040, 512), (1024, 4096, 1024), (7, 48, 96), (16, 1024, 2048),
                                   (200, 512, 128 * 9)])
def test_w4a8_with_and_without_the_reference_workspace(ops, M, N, K):
    """tlq_gemm_w4a8_ws uses the reference's int8 [N, K] workspace in one of two ways: unpack into it (it then holds
    torch_convert(B_packed), example_dequant_gemm_w4a8.py:69-106) and run the int8 GEMM on it, or -- few activation
    rows -- keep the unpack fused and cut K into slices whose int32 matrices live in the workspace.  Without a
    workspace the fused kernel runs (its slices add into C).  Integers: every result is the oracle's, bit for bit."""
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    g = gen(27)
    A = torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=g)
    qB, B_ref = ref.generate_quantized_weight(N, K, g)
    want = ref.int_matmul_exact(A, B_ref.t().contiguous()).to(torch.int32)
    dA, dB = A.cuda(), qB.cuda()
    st = torch.cuda.current_stream().cuda_stream
    for mode in (0, 1, 2):  # automatic, K slices in the workspace, unpack + int8 GEMM
        for ws_bytes in (N * K, 0, N * K - 16, M * N * 8):
            ws = torch.full((max(N * K, M * N * 8),), 99, dtype=torch.int8, device="cuda")
            C = torch.full((M, N), -1, dtype=torch.int32, device="cuda")
            print(f"w4a8 M={M} N={N} K={K} mode={mode} workspace={ws_bytes}", flush=True)
            lib.tlq_tune_w4a8_ws(mode)
            try:
                _abi.check(lib.tlq_gemm_w4a8_ws(P(dA), P(dB), P(ws) if ws_bytes else None, ws_bytes, P(C), M, N, K, _abi.S4_TWOS, st))
            finally:
                lib.tlq_tune_w4a8_ws(0)
            torch.cuda.synchronize()
            assert_bit_equal(C.cpu(), want, f"w4a8 mode={mode} workspace={ws_bytes}")
            if mode == 2:
                if ws_bytes >= N * K and N % 16 == 0 and K % 16 == 0:
                    assert_bit_equal(ws.cpu()[:N * K].view(N, K), B_ref, "the workspace holds the unpacked weights")
                else:
                    assert (ws == 99).all(), "a workspace that is not used stays untouched"


@pytest.mark.parametrize("scale_size,out_dtype", [("1", "float16"), ("N", "bfloat16"), ("N", "float16")])
@pytest.mark.parametrize("Batch,M,N,K", [(2, 256, 256, 256), (3, 100, 272, 400), (8, 1024, 1024, 1024)])
def test_quant_batch_matmul(ops, scale_size, out_dtype, Batch, M, N, K):
    g = gen(23)
    A = torch.randint(-128, 128, (Batch, M, K), dtype=torch.int8, generator=g)
    B = torch.randint(-128, 128, (Batch, K, N), dtype=torch.int8, generator=g)
    scale = torch.randn(N if scale_size == "N" else 1, generator=g)
    kernel = ops.simple_quant_batch_matmul(Batch, M, N, K, scale_size, 128, 256, 64, out_dtype=out_dtype)
    got = kernel(A.cuda(), B.cuda(), scale.cuda()).cpu()
    want = ref.ref_program_quant(A, B, scale, DT[out_dtype])
    assert_bit_equal(got, want, "quant_batch_matmul")
    # 2-D twin
    k2 = ops.simple_quant_matmul(M, N, K, scale_size, 128, 256, 64, out_dtype=out_dtype)
    assert_bit_equal(k2(A[0].cuda(), B[0].cuda(), scale.cuda()).cpu(), want[0], "quant_matmul")


@pytest.mark.parametrize("out_dtype", ["float32", "bfloat16", "float16"])
def test_int8_gemm_per_token_per_channel(ops, out_dtype):
    M, N, K = 333, 272, 512
    g = gen(24)
    A, B = _i8((M, K), 25), _i8((N, K), 26)
    sa = torch.rand(M, generator=g) * 0.04 + 0.01
    sb = torch.rand(N, generator=g) * 0.009 + 0.001
    kernel = ops.int8_gemm_kernel_corrected(N, K, block_M=64, block_N=64, block_K=64, out_dtype=out_dtype)
    got = kernel(A.cuda(), B.cuda(), sa.cuda(), sb.cuda()).cpu()
    assert_bit_equal(got, ref.ref_int8_gemm_sequential(A, B, sa, sb, DT[out_dtype]), "per-token x per-channel")
    gold = ref.int8_gemm_torch_optimized(A, sa, B, sb, DT[out_dtype])
    torch.testing.assert_close(got.float(), gold.float(), rtol=1e-2, atol=1e-2)  # the reference's own check


def test_w8a8_headline_shape(ops):
    """B=8, M=2048, N=K=4096, int8 U[-127,127], per-token x per-channel scales, fp16 out: bit exact
    against the exact-integer oracle, batch by batch."""
    Batch, M, N, K = 8, 2048, 4096, 4096
    g = gen(27)
    A = torch.randint(-127, 128, (Batch, M, K), dtype=torch.int8, generator=g)
    W = torch.randint(-127, 128, (Batch, K, N), dtype=torch.int8, generator=g)
    sa = torch.rand(Batch, M, generator=g) * 0.04 + 0.01
    sb = torch.rand(N, generator=g) * 0.009 + 0.001
    kernel = ops.quant_batch_matmul_per_token(Batch, M, N, K, out_dtype="float16")
    got = kernel(A.cuda(), W.cuda(), sa.cuda(), sb.cuda()).cpu()
    for b in range(Batch):
        want = ref.ref_int8_gemm_sequential(A[b], W[b].T.contiguous(), sa[b], sb, torch.float16)
        assert_bit_equal(got[b], want, f"w8a8 headline batch {b}")


def test_fp16_gemm_plain(ops):
    M, N, K = 256, 512, 256
    A = torch.randn(M, K, generator=gen(28)).to(torch.float16)
    B = torch.randn(K, N, generator=gen(29)).to(torch.float16)
    got = ops.fp16_gemm(M, N, K, 128, 256, 64)(A.cuda(), B.cuda()).cpu()
    check_float_output(got, A.float() @ B.float(), "fp16_gemm")


# ------------------------------------------------------------------------------------------
# committed fixtures (tests/golden/*.npz): frozen inputs and outputs of the two oracles
# ------------------------------------------------------------------------------------------
GOLDEN = __import__("os").path.join(__import__("os").path.dirname(__import__("os").path.abspath(__file__)), "golden")


def _from_bits(a, kind):
    t = torch.from_numpy(a.view(np.int16).copy())
    return t.view(torch.float16 if kind == 0 else torch.bfloat16)


@pytest.mark.parametrize("name", ["f16_g128_tensorz", "f16_g32_scalar8", "bf16_g64_tensorz", "bf16_g128_scalar8", "f16_plain"])
@pytest.mark.parametrize("algo", ["gemv", "mfma"])
def test_golden_w4a16(ops, name, algo):
    with np.load(f"{GOLDEN}/w4a16_small.npz") as f:
        d = {k[len(name) + 1:]: f[k] for k in f.files if k.startswith(name + ".")}
    M, N, K, g, kind, zs = (int(v) if i < 5 else float(v) for i, v in enumerate(d["meta"]))
    if algo == "gemv" and M > 16:
        pytest.skip("the GEMV kernel handles M <= 16")
    dt = torch.float16 if kind == 0 else torch.bfloat16
    A, Wp = _from_bits(d["A"], kind), torch.from_numpy(d["Wp"])
    S = _from_bits(d["S"], kind) if "S" in d else None
    Z = _from_bits(d["Z"], kind) if "Z" in d else (zs if zs else None)
    W = ops.dequantize_w4(Wp.cuda(), None if S is None else S.cuda(), Z.cuda() if isinstance(Z, torch.Tensor) else Z, g, dt)
    assert_bit_equal(W.cpu(), _from_bits(d["W"], kind), f"golden dequant {name}")
    got = _run_w4a16(ops, A, Wp, S, Z, g, "float32", algo, "float16" if kind == 0 else "bfloat16")
    check_float_output(got, torch.from_numpy(d["C"]), f"golden w4a16 {name} {algo}")


def test_golden_int8(ops):
    from tilelang_ascend_amd import _abi

    with np.load(f"{GOLDEN}/int8_small.npz") as f:
        d = {k: f[k] for k in f.files}
    A, W = torch.from_numpy(d["i8.A"]), torch.from_numpy(d["i8.W_kn"])
    B_, M, K = A.shape
    N = W.shape[2]
    lib, P = _abi.load(), _abi.ptr
    st = torch.cuda.current_stream().cuda_stream
    Ad, Wd = A.cuda(), W.cuda()
    Wnk = W.transpose(1, 2).contiguous().cuda()
    for layout, Bm in ((_abi.B_KN, Wd), (_abi.B_NK, Wnk)):
        C = torch.empty(B_, M, N, dtype=torch.int32, device="cuda")
        _abi.check(lib.tlq_gemm_i8(P(Ad), P(Bm), P(C), B_, M, N, K, layout, st))
        assert_bit_equal(C.cpu(), torch.from_numpy(d["i8.acc"]), f"golden i8 layout {layout}")
    sa, sb = torch.from_numpy(d["i8.scale_a"]).cuda(), torch.from_numpy(d["i8.scale_b"]).cuda()
    got = ops.simple_quant_batch_matmul(B_, M, N, K, "N", 128, 256, 64)(Ad, Wd, sb).cpu()
    assert_bit_equal(got, _from_bits(d["i8.C_scale_b_f16"], 0), "golden per-channel f16")
    got = ops.simple_quant_batch_matmul(B_, M, N, K, "1", 128, 256, 64, out_dtype="bfloat16")(Ad, Wd, sb[:1].contiguous()).cpu()
    assert_bit_equal(got, _from_bits(d["i8.C_scale_1_bf16"], 1), "golden per-tensor bf16")
    got = ops.quant_batch_matmul_per_token(B_, M, N, K, out_dtype="float16")(Ad, Wd, sa, sb).cpu()
    assert_bit_equal(got, _from_bits(d["i8.C_token_channel_f16"], 0), "golden per-token x per-channel")
    Wp = torch.from_numpy(d["w4.Wp"])
    assert_bit_equal(ops.torch_unpack_uint4_to_int8(Wp), torch.from_numpy(d["w4.unsigned"]), "golden unpack")
    assert_bit_equal(ops.torch_convert(Wp), torch.from_numpy(d["w4.signed"]), "golden signed unpack")
    got = ops.dequant_gemm_int8_wrapper(M, N, K, 128, 128, 64, "int32")(A[0], Wp)
    assert_bit_equal(got, torch.from_numpy(d["w4.C_unsigned"]), "golden u4 x i8")
    workspace = torch.empty(N, K, dtype=torch.int8, device="cuda")  # a caller-supplied input in the reference
    got = ops.w4a8_gemm_cv(M, N, K)(Ad[0].contiguous(), Wp.cuda(), workspace).cpu()
    assert_bit_equal(got.T.contiguous(), torch.from_numpy(d["w4.C_signed_t"]), "golden s4 x i8")


# ------------------------------------------------------------------------------------------
# skinny kernel (M <= 64, weights streamed from HBM straight into MFMA operands)
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,zeros_kind", [
    (5, 64, 128, 32, None), (16, 1000, 4096, 128, "int"), (17, 130, 2048, 64, "scalar8"), (32, 512, 1024, 1024, "frac"),
    (33, 272, 1536, 96, "int"), (64, 4096, 1024, 128, "scalar8"), (48, 14336, 4096, 64, "int"),
])
def test_skinny_shapes(ops, in_dtype, M, N, K, group, zeros_kind):
    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(40)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=41)
    want = w4a16_reference(A, Wp, s, z, group)
    for out_dtype in ("float32", in_dtype):
        got = _run_w4a16(ops, A, Wp, s, z, group, out_dtype, "skinny", in_dtype)
        check_float_output(got, want, f"skinny {in_dtype}->{out_dtype}")


@pytest.mark.parametrize("waves,row_tiles", [(1, 1), (3, 1), (16, 1), (4, 2), (16, 2)])
def test_skinny_tunings_and_one_hot(ops, waves, row_tiles):
    """One-hot activations return dequantised weight columns bit-exactly through the MFMA path, whatever
    the split of K between wavefronts."""
    from tilelang_ascend_amd import _abi

    N, K, group = 200, 1024, 128
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=42)
    W = ref.dequant_w4(Wp, s, z, group, torch.float16)
    A = torch.zeros(16, K, dtype=torch.float16)
    cols = [0, 1, 31, 32, 127, 128, 500, 1023, 640, 77, 900, 255, 256, 511, 512, 1000]
    for m, k in enumerate(cols):
        A[m, k] = 1.0
    _abi.load().tlq_tune_w4a16_skinny(waves, row_tiles)
    try:
        got = _run_w4a16(ops, A, Wp, s, z, group, "float16", "skinny", "float16")
    finally:
        _abi.load().tlq_tune_w4a16_skinny(0, 0)
    assert_bit_equal(got, W[:, cols].T.contiguous(), f"skinny one-hot waves={waves} rt={row_tiles}")


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("N,K,group", [(256, 1024, 128), (48, 8192, 64), (40, 448, 64)])
def test_auto_picks_a_kernel_for_every_m(ops, in_dtype, N, K, group):
    """The automatic choice (GEMV, skinny or tile kernel by M, K and type; K = 448 admits no skinny kernel)."""
    dt = DT[in_dtype]
    Wp, s, z = make_w4(N, K, group, dt, "int", seed=43)
    for M in (1, 2, 3, 4, 5, 16, 64, 65, 200):
        A = torch.randn(M, K, generator=gen(44)).to(dt)
        got = _run_w4a16(ops, A, Wp, s, z, group, in_dtype, "auto", in_dtype)
        check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"auto {in_dtype} M={M} K={K}")


@pytest.mark.parametrize("M,N,K,algo", [(64, 4096, 4096, "auto"), (256, 2048, 4096, "panelm"), (16, 2048, 8192, "decode"),
                                        (1024, 1024, 1024, "panel256")])
def test_profiler_assert_consistent_on_kernels_that_add_partial_sums(ops, M, N, K, algo):
    """The reference's race check (tilelang/profiler/__init__.py:188-205) on the kernels whose K slices or wavefronts add
    partial sums: every repeat must reproduce the first run bit for bit."""
    kernel = ops.w4a16_gemm(M, N, K, group_size=128, zeros="tensor", algo=algo)
    Wp, s, z = make_w4(N, K, 128, torch.float16, "int", seed=M)
    A = torch.randn(M, K, generator=gen(N)).half()
    print(f"assert_consistent M={M} N={N} K={K} algo={algo}", flush=True)
    kernel.get_profiler().assert_consistent(repeat=5, input_tensors=[A.cuda(), Wp.cuda(), s.cuda(), z.cuda()])
