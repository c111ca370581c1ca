#!/usr/bin/env python3
"""Split-K GEMM with the command line of the reference's examples/gemm_splitk/example_tilelang_gemm_splitk.py
(:73-94): --M --N --K --split-k (all four, or none for the two default cases), prints "Test passed: M=..., N=...,
K=..., split_k=..." per case and "Kernel Output Match!" last."""
import argparse

import torch

import tilelang_ascend_amd as tl
from tilelang_ascend_amd.ops import gemm_splitk


def test(M, N, K, split_k):
    block_M, block_N, block_K = 128, 128, 32
    kernel = gemm_splitk(M, N, K, block_M, block_N, block_K, split_k)
    torch.manual_seed(42)
    a = torch.randn(M, K).half()
    b = torch.randn(K, N).half()
    c = torch.zeros(M, N, dtype=torch.float).cuda()
    kernel(a.cuda(), b.cuda(), c)
    ref_c = a.float() @ b.float()
    torch.testing.assert_close(c.cpu(), ref_c.to(c.dtype), rtol=1e-2, atol=1e-2)
    print(f"Test passed: M={M}, N={N}, K={K}, split_k={split_k}")


def main(custom_args=None):
    parser = argparse.ArgumentParser(description="Split-K GEMM")
    parser.add_argument("--M", type=int, default=0)
    parser.add_argument("--N", type=int, default=0)
    parser.add_argument("--K", type=int, default=0)
    parser.add_argument("--split-k", type=int, default=0)
    args = parser.parse_args(custom_args)
    tl.disable_cache()
    try:
        if args.M > 0 and args.N > 0 and args.K > 0 and args.split_k > 0:
            test(args.M, args.N, args.K, args.split_k)
        else:
            test(128, 128, 128, 2)
            test(1024, 1024, 1024, 4)
    finally:
        tl.enable_cache()
    print("Kernel Output Match!")


if __name__ == "__main__":
    main()
