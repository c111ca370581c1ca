"""The automatic kernel choice of tlq_gemm_w4a16_ws (what ops.w4a16_gemm and the benchmark call): small, launch-bound
problems and 17 .. 32 activation rows take the single-launch kernels although a workspace is there, two fp16 activation
rows on many weight rows take the ring GEMV.  Observed through the outputs: the automatic choice must return the bits of
the kernel it is meant to pick (the kernels differ in summation order), and every result is checked against the oracle."""
import pytest
import torch

from helpers import assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference

pytestmark = pytest.mark.gpu


def run_ws(A, Wp, s, z, group, algo, workspace=True):
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, K = A.shape
    N = Wp.shape[0]
    dA, dW, dS, dZ = A.cuda(), Wp.cuda(), s.cuda(), z.cuda()
    need = max(lib.tlq_w4a16_workspace_bytes(M, N, K), N * K * 2, 16) if workspace else 0
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    print(f"kernel choice M={M} N={N} K={K} g={group} algo={algo} workspace={need}", flush=True)
    lib.tlq_debug_launch_log(1)
    rc = lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, 0.0, _abi.F16, _abi.F16, algo,
                               P(ws) if workspace else None, need, torch.cuda.current_stream().cuda_stream)
    run_ws.log = lib.tlq_debug_launch_log_text().decode()
    lib.tlq_debug_launch_log(0)
    _abi.check(rc)
    torch.cuda.synchronize()
    return C.cpu()


def cases():
    from tilelang_ascend_amd import _abi

    return [
        # M, N, K, group, the kernel the automatic choice is meant to take
        (256, 256, 256, 128, _abi.ALGO_MFMA),      # the reference's own CPU-runnable case: one launch of the tile kernel
        (128, 1024, 512, 128, _abi.ALGO_MFMA),
        (64, 1024, 1024, 128, _abi.ALGO_SKINNY),
        (48, 4096, 1024, 64, _abi.ALGO_SKINNY),
        (24, 4096, 4096, 128, _abi.ALGO_DECODE),
        (32, 1024, 2048, 32, _abi.ALGO_DECODE),
        (2, 8192, 2048, 64, _abi.ALGO_GEMV),       # ring kernel, two activation rows
        (2, 4096, 4096, 128, _abi.ALGO_DECODE),    # 4096 rows: one per wavefront, the decode kernel is ahead
        (64, 4096, 4096, 128, _abi.ALGO_STREAM),   # large enough for K slices and a second launch
        (256, 1024, 1024, 128, _abi.ALGO_STREAM),
        (16, 5120, 5120, 128, _abi.ALGO_DECODE),   # rows of 5120 values, 320 tiles of 16 weight rows (more than CUs): decode kernel on K chunks
        (512, 4096, 2048, 128, _abi.ALGO_STREAM),  # 512 rows on 4096 weight rows: the tile kernels would fill half the machine
        (384, 10240, 2048, 128, _abi.ALGO_STREAM),  # three blocks of 128 activation rows: streaming kernel whatever the tile kernels' fill
        (512, 8192, 2048, 128, _abi.ALGO_STREAM),   # four blocks, 32 x 4 x 2 = 256 streaming work-groups: they fit the machine at once
        (512, 8192, 1024, 128, _abi.ALGO_MFMA),     # short rows, one round of 128 x 128 tiles: the tile kernel in one launch (19 against 23 us)
        (48, 8192, 1024, 128, _abi.ALGO_SKINNY),    # short rows, 33 .. 64 activation rows, up to 2^24 weights: the skinny kernel's one launch
        (112, 32768, 4096, 128, _abi.ALGO_PANELM),    # one tile of 128 rows on 2^27 weights or more: the middle-M kernel
        (144, 50304, 4096, 128, _abi.ALGO_PANEL256),  # two streaming blocks of 96 rows in two rounds against one round of 256-row tiles, by estimate
        (448, 5120, 13824, 128, _abi.ALGO_PANEL256),  # 108 groups per row (the middle-M kernel wants multiples of eight): two 256-row tiles against four streaming blocks by estimate
        (768, 16384, 4096, 128, _abi.ALGO_PANEL256),  # above 512 rows where the 256-row panel kernel's work-groups fill the machine (3 x 64 tiles) and 128-row tiles would need a second round
        (768, 8192, 4096, 128, _abi.ALGO_PANELM),  # 6 x 32 tiles of 128 rows in one round against 3 x 32 x 2 K slices of 256 rows and their partial tiles: the middle-M kernel by estimate (65 against 71 us)
        (2048, 4096, 2048, 128, _abi.ALGO_PANELM),  # 8 x 16 tiles of 256 rows and too few steps to cut (half the CUs idle) against 16 x 16 tiles of 128 rows: the middle-M kernel by estimate
        (192, 28672, 8192, 128, _abi.ALGO_STREAM),  # largest matrices at 192 rows: the streaming kernel (122 us against 154 us for the tile kernel over two long K slices)
        (224, 28672, 8192, 128, _abi.ALGO_PANELM),  # 196 .. 256 rows on wide or very large matrices: the middle-M panel kernel (two tiles of 128 rows)
        (256, 6144, 6144, 128, _abi.ALGO_STREAM),   # 256 rows on fewer than 56 million weights and fewer than 10240 outputs: the streaming kernel
        (256, 14336, 4096, 512, _abi.ALGO_STREAM),  # groups of 512 values up to 256 rows: the panel kernels' windows of eight groups leave K uncut, the streaming kernel cuts inside a group
        (80, 81920, 1024, 128, _abi.ALGO_PANEL),    # 65 .. 128 rows on output-layer widths: 160 .. 256 work-groups of the 128-row panel kernel (512 weight rows each) in one round
        (256, 14336, 4096, 128, _abi.ALGO_PANELM),  # 257 .. 512 rows on 2^25 weights or more, 256 rows on 10240 outputs or more: the middle-M panel kernel
    ]


@pytest.mark.parametrize("case", range(28))
def test_automatic_choice_returns_the_bits_of_the_kernel_it_is_meant_to_take(case):
    from tilelang_ascend_amd import _abi

    M, N, K, group, algo = cases()[case]
    A = torch.randn(M, K, generator=gen(90 + case)).to(torch.float16)
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=110 + case)
    auto = run_ws(A, Wp, s, z, group, _abi.ALGO_AUTO)
    auto_log = run_ws.log
    want = run_ws(A, Wp, s, z, group, algo)
    assert_bit_equal(auto, want, f"automatic choice vs algo {algo} for M={M} N={N} K={K}")
    # (the two four-wavefront panel kernels add up in the same order: told apart by the launch log)
    assert auto_log == run_ws.log, (auto_log, run_ws.log)
    check_float_output(auto, w4a16_reference(A, Wp, s, z, group), "automatic choice vs oracle")


@pytest.mark.parametrize("M,N,K,group", [(601, 4096, 2048, 128), (1003, 2048, 4096, 64), (2049, 1024, 1024, 128), (513, 11008, 4096, 128)])
def test_row_counts_that_are_no_multiple_of_four_run_as_head_and_tail(M, N, K, group):
    """Above 512 rows the automatic choice runs M - M % 4 rows through the choice for that count (the panel kernels take
    multiples of four) and the last rows through the small-M kernels: the result's rows are bit for bit those of the two
    calls made separately, and the whole agrees with the oracle."""
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    A = torch.randn(M, K, generator=gen(700 + M)).to(torch.float16)
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=800 + M)
    whole = run_ws(A, Wp, s, z, group, _abi.ALGO_AUTO)
    log = run_ws.log
    head = M - M % 4
    first = run_ws(A[:head].contiguous(), Wp, s, z, group, _abi.ALGO_AUTO)
    assert log.startswith(run_ws.log.strip()), (log, run_ws.log)  # the head's launches come first, then the tail's
    assert len(log.strip().split(" + ")) > len(run_ws.log.strip().split(" + "))
    assert_bit_equal(whole[:head], first, f"rows 0 .. {head - 1}")
    dA, dW, dS, dZ = A[head:].contiguous().cuda(), Wp.cuda(), s.cuda(), z.cuda()
    C = torch.empty(M - head, N, dtype=torch.float16, device="cuda")
    _abi.check(lib.tlq_gemm_w4a16(P(dA), P(dW), P(dS), P(dZ), P(C), M - head, N, K, group, 0.0, _abi.F16, _abi.F16, _abi.ALGO_AUTO,
                                  torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert_bit_equal(whole[head:], C.cpu(), f"rows {head} .. {M - 1}")
    check_float_output(whole, w4a16_reference(A, Wp, s, z, group), "head and tail vs oracle")
