#!/usr/bin/env python3
"""Batched GEMM with the command line of the reference's examples/batch_gemm/batch_gemm.py (:9-14: --b --m --n --k,
defaults 8 x 1024^3), the same factory call (:64, blocks 128 / 256 / 64), the same check (:77,
assert_close(rtol=atol=1e-2) against torch.matmul) and the same closing line "Batch Kernel Output Match!"."""
import argparse

import torch

from tilelang_ascend_amd.ops import batch_matmul


def main(custom_args=None):
    parser = argparse.ArgumentParser(description="Batched GEMM")
    parser.add_argument("--b", type=int, default=8, help="Batch size")
    parser.add_argument("--m", type=int, default=1024, help="Matrix M dimension")
    parser.add_argument("--n", type=int, default=1024, help="Matrix N dimension")
    parser.add_argument("--k", type=int, default=1024, help="Matrix K dimension")
    args = parser.parse_args(custom_args)
    func = batch_matmul(args.b, args.m, args.n, args.k, 128, 256, 64)
    torch.manual_seed(0)
    a = torch.randn(args.b, args.m, args.k).half().cuda()
    b = torch.randn(args.b, args.k, args.n).half().cuda()
    print("init successful!")
    c = func(a, b)
    ref_c = torch.matmul(a.float().cpu(), b.float().cpu()).half()
    torch.testing.assert_close(c.cpu(), ref_c, rtol=1e-2, atol=1e-2)
    print("Batch Kernel Output Match!")


if __name__ == "__main__":
    main()
