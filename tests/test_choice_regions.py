"""Seeded shapes aimed at the regions where the automatic kernel choice of tlq_gemm_w4a16_ws changes hands -- short rows,
196 .. 512 rows on large matrices, rows whose group count is no multiple of eight, very wide matrices, one scale per weight
row, ragged weight-row counts, output-layer widths -- against the oracle (ref_program_fp16 extended by scales / zero points,
examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:269-289): whatever kernel a rule lands on must take the shape
and agree."""
import random

import pytest
import torch

from helpers import DT, check_float_output, gen, make_w4, w4a16_reference

pytestmark = pytest.mark.gpu


def region_case(seed):
    rnd = random.Random(100 + seed)
    region = seed % 5 if seed < 25 else 5 + seed % 2
    if region == 0:    # short rows
        M = rnd.choice([33, 48, 64, 65, 96, 128, 192, 200, 256, 384, 512])
        N = rnd.choice([1000, 2048, 4096, 6144, 8192, 16384])
        K = 128 * rnd.choice([2, 3, 4, 6, 8, 10, 12, 16])
    elif region == 1:  # 196 .. 512 rows on large matrices, group counts that are no multiple of eight among them
        M = rnd.choice([196, 204, 224, 252, 256, 260, 388, 448, 512])
        N = rnd.choice([5120, 8192, 10240, 11008, 14336])
        K = 128 * rnd.choice([28, 32, 43, 54, 64, 108])
    elif region == 2:  # above 512 rows
        M = rnd.choice([516, 640, 768, 1024, 1536])
        N = rnd.choice([2048, 4096, 5120, 11008])
        K = 128 * rnd.choice([8, 16, 28, 32, 43])
    elif region == 3:  # very wide matrices, one or two tiles of rows
        M = rnd.choice([100, 112, 128, 132, 160, 192, 256])
        N = rnd.choice([32000, 32768, 50304])
        K = 128 * rnd.choice([28, 32])
    elif region == 5:  # weight-row counts that are no multiple of four / eight, rows whose length is no power of two with one group per row
        M = rnd.choice([33, 64, 100, 200, 300, 600, 1001])
        N = rnd.choice([7, 31, 1001, 2050, 4100, 5001, 8207])
        K = 64 * rnd.choice([10, 22, 44, 56])
    elif region == 6:  # output-layer widths at 65 .. 128 rows; decode batches on long rows
        N = rnd.choice([81920, 10240, 12288, 17408])
        M = rnd.choice([68, 96, 128] if N == 81920 else [3, 12, 16])
        K = 128 * rnd.choice([4, 8] if N == 81920 else [40, 48, 64])
    else:              # groups longer than a K slice
        M = rnd.choice([48, 64, 128, 200, 256, 512, 768])
        N = rnd.choice([1024, 2048, 4096, 8192])
        K = 128 * rnd.choice([16, 32, 64])
    if region == 5:
        group = rnd.choice([g for g in (32, 64, 128) if K % g == 0] + [K, K])
    elif region == 4:
        group = rnd.choice([g for g in (1024, 2048, 4096, K) if K % g == 0 and g & (g - 1) == 0])
    else:
        group = rnd.choice([g for g in (32, 64, 128, 256) if K % g == 0])
    return M, N, K, group, rnd.choice([None, "scalar8", "int", "frac"]), rnd.choice(["float16", "bfloat16"])


@pytest.mark.parametrize("seed", range(45))
def test_automatic_choice_where_the_rules_change_hands(seed):
    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    M, N, K, group, zeros_kind, in_dtype = region_case(seed)
    dt = DT[in_dtype]
    code = _abi.F16 if dt == torch.float16 else _abi.BF16
    A = torch.randn(M, K, generator=gen(3000 + seed)).to(dt)
    Wp, s, z = make_w4(N, K, group, dt, zeros_kind, seed=4000 + seed)
    zt = z if torch.is_tensor(z) else None
    zs = 0.0 if (torch.is_tensor(z) or z is None) else float(z)
    dA, dW, dS = A.cuda(), Wp.cuda(), s.cuda()
    dZ = zt.cuda() if zt is not None else None
    need = lib.tlq_w4a16_workspace_bytes(M, N, K)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=dt, device="cuda")
    print(f"choice region seed={seed} M={M} N={N} K={K} g={group} zeros={zeros_kind} {in_dtype} workspace={need}", flush=True)
    lib.tlq_debug_launch_log(1)
    rc = lib.tlq_gemm_w4a16_ws(P(dA), P(dW), P(dS), P(dZ), P(C), M, N, K, group, zs, code, code, _abi.ALGO_AUTO, P(ws), need,
                               torch.cuda.current_stream().cuda_stream)
    log = lib.tlq_debug_launch_log_text().decode().strip()
    lib.tlq_debug_launch_log(0)
    torch.cuda.synchronize()
    assert rc == 0, _abi.last_error()  # (with the workspace the size function asks for, every shape here is taken)
    print("  ->", log.replace("\n", " | "), flush=True)
    check_float_output(C.cpu(), w4a16_reference(A, Wp, s, z, group), f"seed {seed}: {log.splitlines()[0] if log else ''}")
