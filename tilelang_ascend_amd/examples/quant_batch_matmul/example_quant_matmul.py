#!/usr/bin/env python3
"""2-D W8A8 matmul with rescale, with the command line of the reference's
examples/quant_batch_matmul/example_quant_matmul.py (:118-135): --m --n --k (1024), runs scale_size
"1" with bfloat16 output then "N", last lines "QuantMatmul example passed!" / "Kernel Output Match!"."""
import argparse

import torch

import tilelang_ascend_amd as tl
from tilelang_ascend_amd.examples._checks import DTYPES, exact_int_matmul
from tilelang_ascend_amd.ops import simple_quant_matmul


def ref_program(A, B, scale, out_dtype, accum_dtype):
    return (exact_int_matmul(A, B).to(accum_dtype).to(scale.dtype) * scale).to(out_dtype)


def check_case(M, N, K, scale_size, block_M, block_N, block_K, in_dtype="int8", out_dtype="float16",
               accum_dtype="int32", scale_dtype="float32"):
    A = torch.randint(-128, 127, [M, K], dtype=DTYPES[in_dtype])
    B = torch.randint(-128, 127, [K, N], dtype=DTYPES[in_dtype])
    scale = torch.randn([N if scale_size == "N" else 1], dtype=DTYPES[scale_dtype])
    kernel = simple_quant_matmul(M, N, K, scale_size, block_M, block_N, block_K, in_dtype, out_dtype, accum_dtype,
                                 scale_dtype)
    C = kernel(A.cuda(), B.cuda(), scale.cuda())
    torch.testing.assert_close(C.cpu(), ref_program(A, B, scale, DTYPES[out_dtype], DTYPES[accum_dtype]), rtol=1e-2,
                               atol=1e-2)


def main(custom_args=None):
    parser = argparse.ArgumentParser(description="QuantMatmul Example")
    for flag in ("--m", "--n", "--k"):
        parser.add_argument(flag, type=int, default=1024, help=f"Matrix {flag[2:].upper()} dimension")
    args, remains = parser.parse_known_args(custom_args)
    if remains:
        print(f"[{parser.description}]", "Unknown args:", remains)
    tl.cache.clear_cache()
    torch.manual_seed(0)
    check_case(args.m, args.n, args.k, scale_size="1", block_M=128, block_N=256, block_K=64, out_dtype="bfloat16")
    check_case(args.m, args.n, args.k, scale_size="N", block_M=128, block_N=256, block_K=64)
    print("QuantMatmul example passed!")
    print("Kernel Output Match!")


if __name__ == "__main__":
    main()
