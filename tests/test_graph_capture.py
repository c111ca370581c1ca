"""The entry points under HIP graph capture: every call only enqueues kernels on the stream it is given (no allocation,
no memset node, no synchronisation), so a serving loop may record a chain of them once and replay it.

Each graph is replayed several times with eager work of the same process and synchronisations in between, its
outputs and scratch memory overwritten before every replay, and every replay is compared bit for bit with the eager
result of the same calls.  The reference has no counterpart (its kernels are launched by the TVM runtime, one by one).
"""
import pytest
import torch

from helpers import assert_bit_equal, gen, make_w4

pytestmark = pytest.mark.gpu


def _replay_and_compare(calls, outputs, scratch, what):
    """calls(stream) enqueues the work; outputs are the device tensors it writes; scratch the workspaces it may use."""
    calls(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    want = [o.clone() for o in outputs]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        calls(side.cuda_stream)  # a warm-up on the side stream, as torch asks for before a capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        calls(torch.cuda.current_stream().cuda_stream)
    busy = torch.randn(1 << 20, device="cuda")
    for rep in range(4):
        for o in outputs:
            o.view(torch.uint8).fill_(0xA0 + rep)
        for s in scratch:
            s.fill_(0x50 + rep)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (o, w) in enumerate(zip(outputs, want)):
            assert_bit_equal(o.cpu(), w.cpu(), f"{what}: output {i}, replay {rep}")
        busy = (busy * 1.0001 + 1.0).sort().values  # eager launches (torch's own, several kernels) between replays
        assert torch.isfinite(busy.sum()).item()


def test_w4a16_calls_with_a_workspace_in_one_graph():
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    # the GEMV, the streaming kernel with K slices, the tile kernel with K slices and the two passes
    shapes = [(1, 4096, 4096, 128, torch.float16), (48, 1024, 2048, 64, torch.float16),
              (200, 2048, 4096, 128, torch.bfloat16), (1024, 2048, 2048, 128, torch.bfloat16)]
    work, outs, scratch = [], [], []
    for i, (M, N, K, group, dt) in enumerate(shapes):
        code = _abi.F16 if dt == torch.float16 else _abi.BF16
        A = torch.randn(M, K, generator=gen(40 + i)).to(dt).cuda()
        Wp, s, z = make_w4(N, K, group, dt, "int", 50 + i)
        Wp, s, z = Wp.cuda(), s.cuda(), z.cuda()
        need = max(int(lib.tlq_w4a16_workspace_bytes(M, N, K)), 256)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        C = torch.empty(M, N, dtype=dt, device="cuda")
        work.append((A, Wp, s, z, C, M, N, K, group, code, ws, need))
        outs.append(C)
        scratch.append(ws)

    def calls(st):
        for A, Wp, s, z, C, M, N, K, group, code, ws, need in work:
            _abi.check(lib.tlq_gemm_w4a16_ws(P(A), P(Wp), P(s), P(z), P(C), M, N, K, group, 0.0, code, code,
                                             _abi.ALGO_AUTO, P(ws), need, st))

    _replay_and_compare(calls, outs, scratch, "W4A16 with workspaces")


def test_w4a16_noalloc_in_a_graph():
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    assert lib.tlq_gemm_w4a16_noalloc_init() == 0, _abi.last_error()
    # calls on one stream share the built-in array one after the other: a two-pass problem, then K slices over its start
    shapes = [(1024, 2048, 2048, 128, torch.bfloat16), (48, 1024, 2048, 64, torch.float16)]
    work, outs = [], []
    for i, (M, N, K, group, dt) in enumerate(shapes):
        code = _abi.F16 if dt == torch.float16 else _abi.BF16
        A = torch.randn(M, K, generator=gen(60 + i)).to(dt).cuda()
        Wp, s, _ = make_w4(N, K, group, dt, "scalar8", 70 + i)
        C = torch.empty(M, N, dtype=dt, device="cuda")
        work.append((A, Wp.cuda(), s.cuda(), C, M, N, K, group, code))
        outs.append(C)

    def calls(st):
        for A, Wp, s, C, M, N, K, group, code in work:
            _abi.check(lib.tlq_gemm_w4a16_noalloc(P(A), P(Wp), P(s), None, P(C), M, N, K, group, 8.0, code, code,
                                                  _abi.ALGO_AUTO, st))

    _replay_and_compare(calls, outs, [], "W4A16 without allocation")


def test_quantiser_int8_and_plain_slices_in_one_graph():
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, N, K = 16, 2048, 4096
    X = torch.randn(M, K, generator=gen(80)).bfloat16().cuda()
    Aq = torch.empty(M, K, dtype=torch.int8, device="cuda")
    Sa = torch.empty(M, dtype=torch.float32, device="cuda")
    W8 = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=gen(81)).cuda()
    Sb = (torch.rand(N, generator=gen(82)) * 0.01).cuda()
    C8 = torch.empty(M, N, dtype=torch.float16, device="cuda")
    nb8 = int(lib.tlq_w8a8_workspace_bytes(1, M, N, K))
    assert nb8 > 0, "the case is meant to run K slices"
    ws8 = torch.empty(nb8, dtype=torch.uint8, device="cuda")
    W4 = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=gen(83)).view(torch.int8).cuda()
    C4 = torch.empty(M, N, dtype=torch.int32, device="cuda")
    nb4 = 4 * M * N * 4
    ws4 = torch.empty(nb4, dtype=torch.uint8, device="cuda")
    Ci = torch.empty(M, N, dtype=torch.int32, device="cuda")  # no workspace: slices add into C
    Ah = torch.randn(M, K, generator=gen(84)).half().cuda()
    Wh = torch.randn(K, N, generator=gen(85)).half().cuda()
    Ch = torch.empty(M, N, dtype=torch.float16, device="cuda")
    nbh = int(lib.tlq_f16_workspace_bytes(1, M, N, K))
    assert nbh > 0
    wsh = torch.empty(nbh, dtype=torch.uint8, device="cuda")

    def calls(st):
        _abi.check(lib.tlq_act_quant_i8(P(X), P(Aq), P(Sa), M, K, _abi.BF16, 0, st))
        _abi.check(lib.tlq_gemm_w8a8_ws(P(Aq), P(W8), P(Sa), P(Sb), P(C8), P(ws8), nb8, 1, M, N, K, N, _abi.B_NK,
                                        _abi.F16, st))
        _abi.check(lib.tlq_gemm_w4a8_ws(P(Aq), P(W4), P(ws4), nb4, P(C4), M, N, K, 0, st))
        _abi.check(lib.tlq_gemm_i8(P(Aq), P(W8), P(Ci), 1, M, N, K, _abi.B_NK, st))
        _abi.check(lib.tlq_gemm_f16_ws(P(Ah), P(Wh), P(Ch), P(wsh), nbh, 1, M, N, K, _abi.F16, _abi.F16, _abi.B_KN, st))

    _replay_and_compare(calls, [Aq, Sa, C8, C4, Ci, Ch], [ws8, ws4, wsh], "quantiser, int8 and plain K slices")
