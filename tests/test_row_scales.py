"""One scale / zero point per weight row (group = K) on rows whose length is no power of two: tlq_gemm_w4a16_ws writes the
row's values out per power-of-two group into the tail of the workspace and runs with that group size.  The result must be,
bit for bit, what the same call returns for scales and zero points replicated by the caller, and agree with the oracle
(ref_program_fp16 extended by scales / zero points, examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:269-289)."""
import pytest
import torch

from helpers import DT, assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference

pytestmark = pytest.mark.gpu


def run(A, Wp, s, z, group, algo=0, workspace_bytes=None):
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, K = A.shape
    N = Wp.shape[0]
    code = _abi.F16 if A.dtype == torch.float16 else _abi.BF16
    zt = z if torch.is_tensor(z) else None
    zs = 0.0 if (torch.is_tensor(z) or z is None) else float(z)
    dA, dW = A.cuda(), Wp.cuda()
    dS = s.cuda() if s is not None else None
    dZ = zt.cuda() if zt is not None else None
    need = lib.tlq_w4a16_workspace_bytes(M, N, K) if workspace_bytes is None else workspace_bytes
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=A.dtype, device="cuda")
    print(f"row scales M={M} N={N} K={K} g={group} {A.dtype} algo={algo} workspace={need}", flush=True)
    lib.tlq_debug_launch_log(1)
    rc = lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, code, code, algo, P(ws) if need else None, need,
                               torch.cuda.current_stream().cuda_stream)
    run.log = lib.tlq_debug_launch_log_text().decode().strip()
    lib.tlq_debug_launch_log(0)
    _abi.check(rc)
    torch.cuda.synchronize()
    return C.cpu()


@pytest.mark.parametrize("in_dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("M,N,K,zeros_kind", [
    (1, 1024, 1408, "int"), (4, 520, 1408, "frac"), (24, 1024, 2816, "scalar8"), (64, 2048, 1408, "int"), (200, 1024, 3584, "frac"),
    (300, 4096, 1408, None), (640, 1024, 2816, "int"), (1001, 512, 1408, "int"),
])
def test_one_group_per_row_on_rows_that_are_no_power_of_two(in_dtype, M, N, K, zeros_kind):
    dt = DT[in_dtype]
    A = torch.randn(M, K, generator=gen(900 + M)).to(dt)
    Wp, s, z = make_w4(N, K, K, dt, zeros_kind, seed=901 + M)   # scales / zeros [N, 1]
    got = run(A, Wp, s, z, K)
    log = run.log
    assert "written out per group" in log, log
    g_eff = min(K & -K, 1024)
    rep = lambda t: t.repeat(1, K // g_eff).contiguous() if torch.is_tensor(t) else t  # noqa: E731
    same = run(A, Wp, rep(s), rep(z), g_eff)
    assert log.split(" + ", 1 if z is None or not torch.is_tensor(z) else 2)[-1] == run.log, (log, run.log)  # the same kernels behind the expansion
    assert_bit_equal(got, same, f"one group per row vs replicated values at groups of {g_eff}")
    check_float_output(got, w4a16_reference(A, Wp, s, z, K), f"group = K = {K} {in_dtype} {zeros_kind}")


def test_without_room_for_the_values_the_call_still_answers():
    """No workspace (or one too small for the written-out values): the kernels that take any group run, as before."""
    A = torch.randn(48, 1408, generator=gen(950)).half()
    Wp, s, z = make_w4(512, 1408, 1408, torch.float16, "int", seed=951)
    got = run(A, Wp, s, z, 1408, workspace_bytes=0)
    assert "written out per group" not in run.log
    check_float_output(got, w4a16_reference(A, Wp, s, z, 1408), "no workspace")


@pytest.mark.parametrize("M,N,K,zeros_kind", [(16, 512, 2816, "int"), (64, 1024, 1408, "frac"), (300, 1024, 2816, "int")])
def test_interleaved_words_with_one_group_per_row(M, N, K, zeros_kind):
    """tlq_gemm_w4a16_layout_ws writes the values out the same way: the bits of the plain layout on the same logical weights."""
    from oracle import ref
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    A = torch.randn(M, K, generator=gen(960 + M)).half()
    Wp, s, z = make_w4(N, K, K, torch.float16, zeros_kind, seed=961 + M)
    # (the kernel that reads interleaved words at this size, by name on the plain ones: the sums must be added in the same order)
    plain = run(A, Wp, s, z, K, algo=_abi.ALGO_DECODE if M <= 32 else _abi.ALGO_STREAM)
    Wi = ref.interleave_weight(Wp.view(torch.int8), 4, "float16").view(torch.uint8).contiguous()
    dA, dW, dS, dZ = A.cuda(), Wi.cuda(), s.cuda(), z.cuda()
    need = max(lib.tlq_w4a16_workspace_bytes(M, N, K), 16)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    print(f"row scales, interleaved words M={M} N={N} K={K} workspace={need}", flush=True)
    lib.tlq_debug_launch_log(1)
    rc = lib.tlq_gemm_w4a16_layout_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, K, 0.0, _abi.F16, _abi.F16, _abi.ALGO_AUTO,
                                      _abi.W_INTERLEAVED_F16, P(ws), need, torch.cuda.current_stream().cuda_stream)
    log = lib.tlq_debug_launch_log_text().decode()
    lib.tlq_debug_launch_log(0)
    _abi.check(rc)
    torch.cuda.synchronize()
    assert "written out per group" in log and "dequant" not in log, log
    assert_bit_equal(C.cpu(), plain, "interleaved vs plain words, one group per row")
