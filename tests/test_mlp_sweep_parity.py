"""The MLP-shaped sweep (M in {16, 64, 256, 1024, 8192} x (N, K) in {(14336, 4096), (4096, 14336)} x group in
{64, 128}; fp16 activations, fp16 per-group scales and zero points) at every one of its 20 shapes, through
tlq_gemm_w4a16_ws with the automatic kernel choice and a workspace of tlq_w4a16_workspace_bytes -- the call the
benchmark's sweep times -- against oracle.ref.ref_program_w4a16, as the reference compares its wrapper with
ref_program_fp16 (examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:315-348).

The kernel always runs on the full M.  From M = 1024 on the oracle evaluates a seeded sample of 256 rows of A (the
CPU side then stays within seconds); every output column of those rows is compared.  The dequantised fp32 weight
matrix of a (N, K, group) combination is computed once and shared by the five values of M.
"""
import functools

import pytest
import torch

from helpers import check_float_output, gen, make_w4
from oracle import ref

pytestmark = pytest.mark.gpu

NK = [(14336, 4096), (4096, 14336)]
MS = [16, 64, 256, 1024, 8192]
SAMPLE_ROWS = 256


@functools.lru_cache(maxsize=1)
def _weights(N, K, group):
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=1000 + group + N)
    W = ref.dequant_w4(Wp, s, z, group, torch.float16).float()  # what ref_program_w4a16 multiplies with
    return Wp, s, z, W, Wp.cuda(), s.cuda(), z.cuda()


@pytest.mark.parametrize("M", MS)
@pytest.mark.parametrize("group", [128, 64])
@pytest.mark.parametrize("N,K", NK)
def test_mlp_sweep_shape_against_the_oracle(N, K, group, M):
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    Wp, s, z, W, dW, dS, dZ = _weights(N, K, group)
    A = torch.randn(M, K, generator=gen(7 * M + group)).to(torch.float16)
    dA = A.cuda()
    C = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    need = lib.tlq_w4a16_workspace_bytes(M, N, K)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    print(f"mlp sweep M={M} N={N} K={K} g={group} workspace={need}", flush=True)
    _abi.check(lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, 0.0, _abi.F16, _abi.F16,
                                     _abi.ALGO_AUTO, P(ws) if need else None, need, st))
    torch.cuda.synchronize()
    got = C.cpu()
    assert torch.isfinite(got.float()).all(), "unwritten or non-finite outputs"
    if M > SAMPLE_ROWS:
        rows = torch.randperm(M, generator=gen(M + N))[:SAMPLE_ROWS].sort().values
        rows[0], rows[-1] = 0, M - 1  # the first and the last row are always among them
    else:
        rows = torch.arange(M)
    want = A[rows].float() @ W.T
    if M <= 16 and group == 128 and N == 14336:  # once: the shared fp32 weights are those of the oracle's own program
        torch.testing.assert_close(want, ref.ref_program_w4a16(A, Wp, s, z, group, "float32"), rtol=1e-6, atol=1e-6)
    check_float_output(got[rows], want, f"mlp sweep M={M} N={N} K={K} g={group}")
