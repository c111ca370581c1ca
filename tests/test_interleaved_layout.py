"""Kernels that read weights repacked by interleave_weight for the float16 target (tilelang/quantize/utils.py:73-101; the
layout the reference's fast decoders consume, tilelang/quantize/lop3.py:17-24): the dequantisation pass, the streaming
W4A16 kernel, the decode kernel and the two passes.  The repacking only moves 4-bit fields inside each 32-bit word, so every result must be
bit-identical to the plain layout on the same logical weights, and the dequantised matrix must equal the oracle's."""
import numpy as np
import pytest
import torch

from helpers import DT, assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference
from oracle import ref

pytestmark = pytest.mark.gpu
CODE = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}


def interleaved(Wp: torch.Tensor) -> torch.Tensor:
    """The oracle's interleave_weight on the packed bytes (int8 storage as in the reference), back as uint8."""
    out = ref.interleave_weight(Wp.view(torch.int8), 4, "float16")
    return out.view(torch.uint8).contiguous()


def test_the_oracle_interleave_moves_fields_as_the_header_says():
    """Field j of each interleaved word holds element (0, 2, 4, 6, 1, 3, 5, 7)[j]."""
    vals = torch.arange(8, dtype=torch.uint8).reshape(1, 8)
    packed = (vals[:, 0::2] | (vals[:, 1::2] << 4)).contiguous()
    word = int(np.ascontiguousarray(interleaved(packed).numpy()).view(np.uint32)[0, 0])
    assert [(word >> (4 * j)) & 15 for j in range(8)] == [0, 2, 4, 6, 1, 3, 5, 7]


def run_layout(A, Wp, s, z, group, layout, algo, out_dtype=None, workspace_bytes=None):
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
    need = max(lib.tlq_w4a16_workspace_bytes(M, N, K), N * K * 2) if workspace_bytes is None else workspace_bytes
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    print(f"layout={layout} algo={algo} M={M} N={N} K={K} g={group} {A.dtype} workspace={need}", flush=True)
    rc = lib.tlq_gemm_w4a16_layout_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, CODE[A.dtype], CODE[out_dtype], algo,
                                      layout, P(ws), need, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return rc, C.cpu()


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("zeros_kind", [None, "scalar8", "int", "frac"])
@pytest.mark.parametrize("N,K,group", [(64, 128, 32), (513, 1024, 128), (96, 4096, 64)])
def test_dequant_of_interleaved_words_is_the_oracle_matrix(in_dtype, zeros_kind, N, K, group):
    from tilelang_ascend_amd.ops import dequant_gemm as ops

    dt = DT[in_dtype]
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=70)
    want = ref.dequant_w4(Wp, s, z, group, dt)
    cz = z.cuda() if torch.is_tensor(z) else z
    plain = ops.dequantize_w4(Wp.cuda(), s.cuda(), cz, group, dt).cpu()
    inter = ops.dequantize_w4(interleaved(Wp).cuda(), s.cuda(), cz, group, dt, weight_layout="interleaved").cpu()
    assert_bit_equal(plain, want, "plain layout")
    assert_bit_equal(inter, want, "interleaved layout")


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,zeros_kind", [
    (17, 256, 128, 128, "int"), (33, 1000, 512, 64, "frac"), (64, 2048, 4096, 128, "scalar8"), (100, 520, 1152, 128, None),
    (256, 14336, 4096, 128, "int"), (500, 1024, 2048, 32, "int"),
])
def test_streaming_kernel_on_interleaved_words(in_dtype, M, N, K, group, zeros_kind):
    from tilelang_ascend_amd import _abi

    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(71)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=72)
    rc, plain = run_layout(A, Wp, s, z, group, _abi.W_PLAIN, _abi.ALGO_STREAM)
    assert rc == 0, _abi.last_error()
    rc, inter = run_layout(A, interleaved(Wp), s, z, group, _abi.W_INTERLEAVED_F16, _abi.ALGO_STREAM)
    assert rc == 0, _abi.last_error()
    assert_bit_equal(inter, plain, f"stream interleaved vs plain {in_dtype} {M}x{N}x{K}")
    if M * N * K <= 1 << 31:
        check_float_output(inter, w4a16_reference(A, Wp, s, z, group), "stream interleaved vs oracle")


@pytest.mark.parametrize("in_dtype,out_dtype", [("float16", "float16"), ("bfloat16", "float32")])
@pytest.mark.parametrize("M,N,K,group", [(300, 1024, 512, 128), (1024, 2048, 1024, 64), (448, 5120, 13824, 128), (80, 81920, 1024, 128)])
def test_two_passes_and_automatic_choice_on_interleaved_words(in_dtype, out_dtype, M, N, K, group):
    from tilelang_ascend_amd import _abi

    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(73)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, "int", seed=74)
    # what the automatic choice takes for interleaved words: the streaming kernel for 300 rows on 1024 weight rows (the
    # tile kernels of the two passes would leave most of the machine idle), the two passes for 1024 rows
    # (448 rows on 5120 x 13824: two tiles of the 256-row kernel against four streaming blocks, by estimate)
    # (80 rows on 81920 weight rows: 160 work-groups of the 128-row panel kernel in one round)
    taken = {300: _abi.ALGO_STREAM, 1024: _abi.ALGO_TWO_PASS, 448: _abi.ALGO_PANEL256, 80: _abi.ALGO_PANEL}[M]
    for algo, plain_algo in ((_abi.ALGO_TWO_PASS, _abi.ALGO_TWO_PASS), (_abi.ALGO_AUTO, taken)):
        rc, plain = run_layout(A, Wp, s, z, group, _abi.W_PLAIN, plain_algo, DT[out_dtype])
        assert rc == 0, _abi.last_error()
        rc, inter = run_layout(A, interleaved(Wp), s, z, group, _abi.W_INTERLEAVED_F16, algo, DT[out_dtype])
        assert rc == 0, _abi.last_error()
        assert_bit_equal(inter, plain, f"interleaved (algo {algo}) vs plain {in_dtype} {M}x{N}x{K}")
        check_float_output(plain, w4a16_reference(A, Wp, s, z, group), "vs oracle")


def test_operator_with_interleaved_weights_packed_on_the_gpu():
    """w4a16_gemm(weight_layout="interleaved") on weights packed by quantize.gpu.pack_int4(interleave="float16")."""
    from tilelang_ascend_amd.ops import dequant_gemm as ops
    from tilelang_ascend_amd.quantize import gpu

    M, N, K, group = 96, 768, 1024, 128
    A = torch.randn(M, K, generator=gen(75)).to(torch.float16)
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=76)
    vals = torch.from_numpy(ref.unpack_uint4(Wp)).to(torch.uint8)
    Wi = gpu.pack_int4(vals.cuda(), "float16", torch.uint8)
    assert_bit_equal(Wi.cpu(), interleaved(Wp), "GPU packer vs oracle interleave")
    plain = ops.w4a16_gemm(M, N, K, group_size=group, zeros="tensor")(A.cuda(), Wp.cuda(), s.cuda(), z.cuda()).cpu()
    inter = ops.w4a16_gemm(M, N, K, group_size=group, zeros="tensor", weight_layout="interleaved")(A.cuda(), Wi, s.cuda(), z.cuda()).cpu()
    assert_bit_equal(inter, plain, "operator interleaved vs plain")
    check_float_output(inter, w4a16_reference(A, Wp, s, z, group), "operator interleaved vs oracle")


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,zeros_kind", [(1, 64, 256, 64, "int"), (16, 1000, 4096, 128, "frac"), (32, 520, 8192, 64, "int"), (7, 2048, 1024, 32, None)])
def test_decode_kernel_on_interleaved_words(in_dtype, M, N, K, group, zeros_kind):
    from tilelang_ascend_amd import _abi

    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(77)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=78)
    rc, plain = run_layout(A, Wp, s, z, group, _abi.W_PLAIN, _abi.ALGO_DECODE)
    assert rc == 0, _abi.last_error()
    for algo in (_abi.ALGO_DECODE, _abi.ALGO_AUTO):
        rc, inter = run_layout(A, interleaved(Wp), s, z, group, _abi.W_INTERLEAVED_F16, algo)
        assert rc == 0, _abi.last_error()
        assert_bit_equal(inter, plain, f"decode interleaved vs plain {in_dtype} {M}x{N}x{K} algo {algo}")
    check_float_output(inter, w4a16_reference(A, Wp, s, z, group), "decode interleaved vs oracle")


@pytest.mark.parametrize("in_dtype,M,N,K,group,zeros_kind", [
    ("float16", 1, 1024, 4096, 128, "int"), ("float16", 1, 520, 1024, 32, "frac"), ("float16", 2, 8192, 2048, 64, "int"),
    ("float16", 2, 300, 4096, 128, None), ("bfloat16", 1, 1024, 4096, 128, "int"), ("bfloat16", 1, 264, 2048, 64, "frac")])
def test_ring_gemv_on_interleaved_words(in_dtype, M, N, K, group, zeros_kind):
    """One or two activation rows: the ring GEMV reads the repacked words too.  Its sums pair other elements than with plain
    words, so the two layouts agree to rounding, not bit for bit -- except on one-hot activations, where a single product
    is summed."""
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(81)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=82)
    want = w4a16_reference(A, Wp, s, z, group)
    rc, plain = run_layout(A, Wp, s, z, group, _abi.W_PLAIN, _abi.ALGO_GEMV)
    assert rc == 0, _abi.last_error()
    for algo in (_abi.ALGO_GEMV,) + ((_abi.ALGO_AUTO,) if (M == 1 or N >= 8192) else ()):
        lib.tlq_debug_launch_log(1)
        rc, inter = run_layout(A, interleaved(Wp), s, z, group, _abi.W_INTERLEAVED_F16, algo)
        log = lib.tlq_debug_launch_log_text().decode()
        lib.tlq_debug_launch_log(0)
        assert rc == 0, _abi.last_error()
        assert "interleaved words" in log, log
        check_float_output(inter, want, f"ring GEMV on interleaved words, algo {algo}")
        assert torch.allclose(inter.float(), plain.float(), rtol=2e-3, atol=2e-3)
    hot = torch.zeros(M, K, dtype=dt)
    hot[0, 5] = 1.0
    hot[M - 1, K - 3] = 1.0 if M > 1 else hot[M - 1, K - 3]
    rc, plain_hot = run_layout(hot, Wp, s, z, group, _abi.W_PLAIN, _abi.ALGO_GEMV)
    rc2, inter_hot = run_layout(hot, interleaved(Wp), s, z, group, _abi.W_INTERLEAVED_F16, _abi.ALGO_GEMV)
    assert rc == 0 and rc2 == 0
    assert_bit_equal(inter_hot, plain_hot, "one-hot activations: the dequantised weights themselves")


def test_interleaved_layout_rejects_what_no_kernel_reads():
    from tilelang_ascend_amd import _abi

    A = torch.zeros(16, 128, dtype=torch.float16)  # K = 128: not a shape of the decode kernel
    Wp = torch.zeros(256, 64, dtype=torch.uint8)
    rc, _ = run_layout(A, Wp, None, None, 128, _abi.W_INTERLEAVED_F16, _abi.ALGO_AUTO)
    assert rc != 0 and "plain layout" in _abi.last_error()
    rc, _ = run_layout(A, Wp, None, None, 128, _abi.W_INTERLEAVED_F16, _abi.ALGO_DECODE)
    assert rc != 0 and "decode kernel" in _abi.last_error()
    rc, _ = run_layout(A, Wp, None, None, 128, _abi.W_INTERLEAVED_F16, _abi.ALGO_GEMV)
    assert rc != 0 and "M <= 2" in _abi.last_error()
    rc, _ = run_layout(A, Wp, None, None, 128, _abi.W_INTERLEAVED_F16, _abi.ALGO_MFMA)
    assert rc != 0 and "interleaved weights are read by" in _abi.last_error()
    rc, _ = run_layout(A, Wp, None, None, 128, 7, _abi.ALGO_AUTO)
    assert rc != 0 and "bad weight layout" in _abi.last_error()
