#!/usr/bin/env python3
"""Weight-only int4 GEMM example with the command line and output lines of the reference's
examples/dequantize_gemm/example_dequant_gemm_fine_grained.py (:405-479): --m --n --k (default 256),
--input-dtype {float16,bfloat16,int8}, unknown flags tolerated, `main(custom_args=None)`,
last lines "All tests passed!" / "Kernel Output Match!"."""
import argparse

import torch

import tilelang_ascend_amd as tl
from tilelang_ascend_amd.examples._checks import DTYPES, exact_int_matmul, unpack_nibbles
from tilelang_ascend_amd.ops import (dequant_gemm_fp16_wrapper, dequant_gemm_int8_wrapper, torch_unpack_uint4_to_fp16,
                                     torch_unpack_uint4_to_int8)

tl.cache.clear_cache()


def ref_program_fp16(A, B_packed, output_dtype):
    return (A.float() @ unpack_nibbles(B_packed).float().T).to(DTYPES[output_dtype])


def ref_program_int8(A, B_packed, output_dtype):
    return exact_int_matmul(A, unpack_nibbles(B_packed).T).to(torch.int32).to(DTYPES[output_dtype])


def check_case_fp16(M, N, K, block_M, block_N, block_K, input_dtype="float16", output_dtype="float16"):
    assert K % 2 == 0, "K must be divisible by 2 (INT4 packed format)"
    A = torch.randn(M, K, dtype=DTYPES[input_dtype])
    B_packed = torch.randint(0, 255, [N, K // 2], dtype=torch.uint8)
    C = dequant_gemm_fp16_wrapper(M, N, K, block_M, block_N, block_K, input_dtype, output_dtype)(A, B_packed)
    tol = 1e-2 if output_dtype in ("float16", "bfloat16") else 1e-4
    torch.testing.assert_close(C, ref_program_fp16(A, B_packed, output_dtype), rtol=tol, atol=tol)
    print(f"FP16 Test passed: M={M}, N={N}, K={K}, input={input_dtype}, output={output_dtype}")


def check_case_int8(M, N, K, block_M, block_N, block_K, output_dtype="int32"):
    assert K % 2 == 0, "K must be divisible by 2 (INT4 packed format)"
    A = torch.randint(-128, 127, [M, K], dtype=torch.int8)
    B_packed = torch.randint(0, 255, [N, K // 2], dtype=torch.uint8)
    C = dequant_gemm_int8_wrapper(M, N, K, block_M, block_N, block_K, output_dtype)(A, B_packed)
    tol = 0 if output_dtype == "int32" else 1e-2
    torch.testing.assert_close(C, ref_program_int8(A, B_packed, output_dtype), rtol=tol, atol=tol)
    print(f"INT8 Test passed: M={M}, N={N}, K={K}, output={output_dtype}")


def check_unpack_functions():
    packed = torch.tensor([[0x12, 0x34]], dtype=torch.uint8)
    for fn, dtype, label in ((torch_unpack_uint4_to_fp16, torch.float16, "FP16"), (torch_unpack_uint4_to_int8, torch.int8, "INT8")):
        out = fn(packed)
        assert out.shape == (1, 4), f"{label} shape mismatch: {out.shape}"
        assert out.dtype == dtype, f"{label} dtype mismatch: {out.dtype}"
        assert out.tolist() == [[2, 1, 4, 3]], f"{label} value mismatch: {out.tolist()}"
        print(f"INT4 -> {label} unpack test passed!")


def main(custom_args=None):
    parser = argparse.ArgumentParser(description="Dequantize GEMM Example (INT4 -> FP16/INT8)")
    for flag in ("--m", "--n", "--k"):
        parser.add_argument(flag, type=int, default=256, help=f"Matrix {flag[2:].upper()} dimension")
    parser.add_argument("--input-dtype", type=str, default="float16", choices=["float16", "bfloat16", "int8"],
                        help="Input data type")
    args, remains = parser.parse_known_args(custom_args)
    if remains:
        print(f"[{parser.description}] Unknown args:", remains)
    M, N, K = args.m, args.n, args.k
    tl.cache.clear_cache()
    torch.manual_seed(0)

    bar = "=" * 60
    print(f"{bar}\nDequantize GEMM Tests (Unsigned INT4)\n{bar}")
    print("\n[Unpack Function Tests]")
    check_unpack_functions()
    fp16_tiles, int8_tiles = dict(block_M=128, block_N=256, block_K=64), dict(block_M=128, block_N=128, block_K=64)
    custom_in = args.input_dtype if args.input_dtype != "int8" else "float16"
    plan = [
        ("[FP16 Mode Tests - Level 0: Small Scale]", check_case_fp16, [(256, 256, 256, "float16", "float16")], fp16_tiles),
        ("[FP16 Mode Tests - Level 1: Typical Scale]", check_case_fp16,
         [(512, 512, 512, "float16", "float16"), (1024, 1024, 1024, "float16", "float16")], fp16_tiles),
        ("[FP16 Mode Tests - Level 1: BFloat16 Input]", check_case_fp16, [(512, 512, 512, "bfloat16", "bfloat16")], fp16_tiles),
        ("[FP16 Mode Tests - Custom Dimensions]", check_case_fp16, [(M, N, K, custom_in, "float16")], fp16_tiles),
        ("[INT8 Mode Tests - Level 0: Small Scale]", check_case_int8, [(256, 256, 256, "int32")], int8_tiles),
        ("[INT8 Mode Tests - Level 1: Typical Scale]", check_case_int8, [(512, 512, 512, "int32"), (1024, 1024, 1024, "int32")],
         int8_tiles),
        ("[INT8 Mode Tests - Level 1: Output to Float16]", check_case_int8, [(512, 512, 512, "float16")], int8_tiles),
        ("[INT8 Mode Tests - Custom Dimensions]", check_case_int8, [(M, N, K, "int32")], int8_tiles),
    ]
    for title, fn, cases, tiles in plan:
        print("\n" + title)
        for m, n, k, *dtypes in cases:
            fn(m, n, k, tiles["block_M"], tiles["block_N"], tiles["block_K"], *dtypes)
    print(f"{bar}\nAll tests passed!\nKernel Output Match!\n{bar}")


if __name__ == "__main__":
    main()
