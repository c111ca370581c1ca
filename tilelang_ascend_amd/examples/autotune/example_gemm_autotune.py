#!/usr/bin/env python3
"""Autotuned W4A16 matmul, after the reference's examples/autotune/example_gemm_autotune.py: flags --m --n --k
(1024), a list of configurations, ``@autotune`` stacked on ``@jit``; the call leaves the tunable parameters
out, prints "Best Config: ..." and "Test passed!".  The tunables here are the library's kernel family and
tile instead of block_M / block_N / K_L1."""
import argparse

import torch

import tilelang_ascend_amd as tl
from tilelang_ascend_amd.examples._checks import unpack_nibbles
from tilelang_ascend_amd.ops import w4a16_gemm

GROUP = 128


def get_config(M, N, K, **_):
    configs = [{"algo": "mfma", "tile": t} for t in (16, 32, 64, 128, 256) if t <= max(16, 2 * M)]
    if M <= 64 and K % 128 == 0:
        configs.append({"algo": "skinny", "tile": 0})
    if M <= 16:
        configs.append({"algo": "gemv", "tile": 0})
    return configs


def ref_prog(A, B_packed, scales, zero=8.0):
    """W = (u - zero) * scale with one fp16 rounding per operation, then an fp32-accumulated matmul."""
    u = unpack_nibbles(B_packed).to(torch.float16)
    W = (u - zero) * scales.cpu().repeat_interleave(GROUP, dim=1)
    return (A.cpu().float() @ W.float().T).to(A.dtype)


def main(custom_args=None):
    parser = argparse.ArgumentParser(description="Autotuned W4A16 matmul")
    for flag in ("--m", "--n", "--k"):
        parser.add_argument(flag, type=int, default=1024, help=f"Matrix {flag[2:].upper()} dimension")
    args, _ = parser.parse_known_args(custom_args)
    M, N, K = args.m, args.n, args.k
    tl.cache.clear_cache()

    def supply_prog(params):
        torch.manual_seed(0)
        return [torch.randn(M, K).half().cuda(), torch.randint(0, 256, (N, K // 2), dtype=torch.uint8).cuda(),
                (torch.rand(N, K // GROUP) * 0.015 + 0.005).half().cuda()]

    matmul = tl.autotune(configs=get_config, ref_prog=ref_prog, supply_prog=supply_prog, atol=1e-2, rtol=1e-2,
                         warmup=5, rep=20)(w4a16_gemm)
    # the tunable parameters (algo, tile) are left out, which triggers the search
    func = matmul(M, N, K, group_size=GROUP, zeros=8)
    result = func.get_tuner_result()
    print("Best Config:", result.config)
    print("Best latency (ms):", round(result.latency, 4), "| configurations tried:", len(result.trials))
    A, Bp, S = supply_prog(None)
    torch.testing.assert_close(func(A, Bp, S).cpu(), ref_prog(A, Bp, S), rtol=1e-2, atol=1e-2)
    print("Test passed!")


if __name__ == "__main__":
    main()
