"""Seeded random shapes through the automatic kernel choice (tlq_gemm_w4a16_ws with the workspace its query asks for, and
tlq_gemm_w4a16 without one) against the oracle: ragged M and N, K any multiple of 64, every group size that divides K, all
zero-point kinds, both activation types.  Whatever kernel the choice lands on must accept the shape and agree with
ref_program_fp16 extended by scales / zero points (examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:269-289)."""
import random

import pytest
import torch

from helpers import DT, check_float_output, gen, make_w4, w4a16_reference

pytestmark = pytest.mark.gpu


def random_case(seed):
    rnd = random.Random(seed)
    M = rnd.choice([1, 2, 3, 5, 8, 16, 17, 24, 32, 33, 48, 64, 65, 100, 128, 200, 256, 300, 512, 513, 700, 1024])
    N = rnd.choice([4, 8, 16, 20, 64, 100, 256, 260, 1000, 1024, 2048, 3000, 4096, 5120, 8192, 11008])
    K = 64 * rnd.choice([1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 40, 64, 86, 128])
    while M * N * K > 1 << 31:  # keep the oracle's matmul in seconds
        N = max(4, N // 2 // 4 * 4)
    groups = [g for g in (32, 64, 128, 256, 512) if K % g == 0]
    group = rnd.choice(groups)
    zeros_kind = rnd.choice([None, "scalar8", "int", "frac"])
    in_dtype = rnd.choice(["float16", "bfloat16"])
    return M, N, K, group, zeros_kind, in_dtype


@pytest.mark.parametrize("seed", range(72))
def test_automatic_choice_on_random_shapes(seed):
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, N, K, group, zeros_kind, in_dtype = random_case(seed)
    dt = DT[in_dtype]
    code = _abi.F16 if dt == torch.float16 else _abi.BF16
    A = torch.randn(M, K, generator=gen(1000 + seed)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=2000 + seed)
    zt = z if torch.is_tensor(z) else None
    zs = 0.0 if (torch.is_tensor(z) or z is None) else float(z)
    dA, dW, dS = A.cuda(), Wp.cuda(), s.cuda()
    dZ = zt.cuda() if zt is not None else None
    want = w4a16_reference(A, Wp, s, z, group)
    need = lib.tlq_w4a16_workspace_bytes(M, N, K)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    for with_ws in (True, False):
        C = torch.full((M, N), float("nan"), dtype=dt, device="cuda")
        print(f"random shape seed={seed} M={M} N={N} K={K} g={group} zeros={zeros_kind} {in_dtype} workspace={need if with_ws else 'none'}", flush=True)
        if with_ws:
            rc = lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, code, code, _abi.ALGO_AUTO, P(ws), need, st)
        else:
            rc = lib.tlq_gemm_w4a16(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, code, code, _abi.ALGO_AUTO, st)
        torch.cuda.synchronize()
        if rc != 0:
            # the only shapes no kernel takes: more than 16 activation rows with N not a multiple of 4 (MFMA tile stores)
            assert M > 16 and N % 4 != 0, _abi.last_error()
            continue
        check_float_output(C.cpu(), want, f"seed {seed} {'with' if with_ws else 'without'} workspace")
