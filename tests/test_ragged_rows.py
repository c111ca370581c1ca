"""Weight-row counts that are no multiple of four (vocabularies of 50257 or 32001 rows) with more than 32 activation rows, and
multiples of four that are no multiples of eight above 512 rows:
tlq_gemm_w4a16_ws runs the first N - N % 16 rows through its usual choice into a packed result behind the workspace, copies
that into C and computes the last rows straight into C.  The first columns must be, bit for bit, what the same call returns
for those weight rows alone, and the whole must agree with the oracle (ref_program_fp16 extended by scales / zero points,
examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:269-289)."""
import pytest
import torch

from helpers import DT, assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference

pytestmark = pytest.mark.gpu
CODE = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}


def run(A, Wp, s, z, group, out_dtype=None, workspace_bytes=None):
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
    need = lib.tlq_w4a16_workspace_bytes(M, N, K) if workspace_bytes is None else workspace_bytes
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    print(f"ragged rows M={M} N={N} K={K} g={group} {A.dtype}->{out_dtype} workspace={need}", flush=True)
    lib.tlq_debug_launch_log(1)
    rc = lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, CODE[A.dtype], CODE[out_dtype], _abi.ALGO_AUTO,
                               P(ws) if need else None, need, torch.cuda.current_stream().cuda_stream)
    run.log = lib.tlq_debug_launch_log_text().decode().strip()
    lib.tlq_debug_launch_log(0)
    torch.cuda.synchronize()
    return rc, C.cpu()


@pytest.mark.parametrize("in_dtype,out_dtype", [("float16", "float16"), ("bfloat16", "bfloat16"), ("float16", "float32")])
@pytest.mark.parametrize("M,N,K,group,zeros_kind", [
    (40, 1001, 512, 128, "int"), (64, 5001, 1024, 64, "frac"), (100, 1003, 512, 128, "scalar8"), (300, 2050, 1024, 128, "int"),
    (700, 1037, 2048, 128, None), (601, 1029, 1024, 32, "int"), (129, 8207, 256, 256, "frac"), (33, 31, 512, 128, "int"),
    (256, 4099, 1408, 1408, "int"),  # with one scale per row on rows that are no power of two as well
    (100, 7, 512, 128, "int"), (600, 1036, 1024, 128, "int"), (1024, 4100, 512, 64, "scalar8"),  # a multiple of four that is no multiple of eight, above 512 rows
])
def test_row_counts_that_are_no_multiple_of_four(in_dtype, out_dtype, M, N, K, group, zeros_kind):
    from tilelang_ascend_amd import _abi

    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(1000 + M)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=1001 + M)
    rc, got = run(A, Wp, s, z, group, DT[out_dtype])
    assert rc == 0, _abi.last_error()
    log = run.log
    head = N - N % 16
    assert ("packed result into C" in log or head == 0) and "last weight rows" in log, log
    if head == 0:  # fewer than 16 weight rows: the last-rows kernel alone
        check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"{N} weight rows")
        return
    cut = lambda t: t[:head].contiguous() if torch.is_tensor(t) else t  # noqa: E731
    rc, first = run(A, Wp[:head].contiguous(), cut(s), cut(z), group, DT[out_dtype])
    assert rc == 0, _abi.last_error()
    assert log.startswith(run.log), (log, run.log)
    assert_bit_equal(got[:, :head].contiguous(), first, f"columns 0 .. {head - 1}")
    check_float_output(got, w4a16_reference(A, Wp, s, z, group),
                       f"ragged {M}x{N}x{K} g{group} {in_dtype}->{out_dtype} {zeros_kind}")


def test_without_room_for_the_packed_result_the_call_answers_as_before():
    """A workspace without room for the packed result: up to 64 rows the skinny kernel takes the count as it is; more rows are
    refused with the tile kernel's message, as they were."""
    from tilelang_ascend_amd import _abi

    A = torch.randn(48, 512, generator=gen(1100)).half()
    Wp, s, z = make_w4(1001, 512, 128, torch.float16, "int", seed=1101)
    rc, got = run(A, Wp, s, z, 128, workspace_bytes=0)
    assert rc == 0 and "packed result" not in run.log, (_abi.last_error(), run.log)
    check_float_output(got, w4a16_reference(A, Wp, s, z, 128), "no workspace, 48 rows")
    A = torch.randn(200, 512, generator=gen(1102)).half()
    rc, _ = run(A, Wp, s, z, 128, workspace_bytes=0)
    assert rc != 0 and "N" in _abi.last_error()


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,group,zeros_kind", [(40, 1001, 512, 128, "int"), (300, 2050, 1024, 64, "frac"), (700, 1037, 2048, 128, "scalar8"), (100, 7, 512, 128, "int")])
def test_interleaved_words_with_ragged_row_counts(in_dtype, M, N, K, group, zeros_kind):
    """tlq_gemm_w4a16_layout_ws takes the same route for words repacked by interleave_weight: against the oracle, and the last
    columns (the last-rows kernel puts each word back in plain order) bit for bit those of the plain layout."""
    from oracle import ref
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(1200 + M)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=1201 + M)
    rc, plain = run(A, Wp, s, z, group)
    assert rc == 0, _abi.last_error()
    Wi = ref.interleave_weight(Wp.view(torch.int8), 4, "float16").view(torch.uint8).contiguous()
    zt = z if torch.is_tensor(z) else None
    zs = 0.0 if (torch.is_tensor(z) or z is None) else float(z)
    dA, dW, dS = A.cuda(), Wi.cuda(), s.cuda()
    dZ = zt.cuda() if zt is not None else None
    need = max(lib.tlq_w4a16_workspace_bytes(M, N, K), 16)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=dt, device="cuda")
    print(f"ragged rows, interleaved words M={M} N={N} K={K} g={group} {in_dtype} workspace={need}", flush=True)
    lib.tlq_debug_launch_log(1)
    rc = lib.tlq_gemm_w4a16_layout_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, CODE[dt], CODE[dt], _abi.ALGO_AUTO,
                                      _abi.W_INTERLEAVED_F16, P(ws), need, torch.cuda.current_stream().cuda_stream)
    log = lib.tlq_debug_launch_log_text().decode()
    lib.tlq_debug_launch_log(0)
    torch.cuda.synchronize()
    assert rc == 0, _abi.last_error()
    assert "last weight rows" in log, log
    got = C.cpu()
    head = N - N % 16
    assert_bit_equal(got[:, head:].contiguous(), plain[:, head:].contiguous(), f"columns {head} .. {N - 1}")
    check_float_output(got, w4a16_reference(A, Wp, s, z, group), f"interleaved, ragged {M}x{N}x{K} {in_dtype}")
