#!/usr/bin/env python3
"""int8 activations x packed two's-complement int4 weights, with the command line of the reference's
examples/dequantize_gemm/example_dequant_gemm_w4a8.py (:185-210): --M --N --K (0 = run the three
built-in sizes), last line "Test Passed!"."""
import argparse

import torch

import tilelang_ascend_amd as tilelang
from tilelang_ascend_amd.examples._checks import exact_int_matmul, sign_extend4, unpack_nibbles
from tilelang_ascend_amd.ops import torch_convert, w4a8_gemm_cv


def generate_quantized_weight(N, K):
    """Random int4 values in [-8, 8) and their packing, two per byte, low nibble first."""
    B_int8 = torch.randint(-8, 8, (N, K), dtype=torch.int8)
    nib = B_int8.to(torch.int16) & 0xF
    return ((nib[:, 1::2] << 4) | nib[:, 0::2]).to(torch.uint8), B_int8


def ref_program(A, qB):
    """[N, M] int32, like the reference's golden (it returns the transpose)."""
    B = sign_extend4(unpack_nibbles(qB))
    return exact_int_matmul(A, B.T).to(torch.int32).transpose(0, 1)


def test(M, N, K):
    kernel = w4a8_gemm_cv(M, N, K)
    A_int8 = torch.randint(-8, 8, (M, K), dtype=torch.int8).cuda()
    qB, B_int8_ref = generate_quantized_weight(N, K)
    workspace = torch.zeros(N, K, dtype=torch.int8).cuda()  # kept for signature compatibility; the unpack is fused
    C_output = torch.zeros(M, N, dtype=torch.int32).cuda()
    result = kernel(A_int8, qB.cuda(), workspace, C_output)
    torch.cuda.synchronize()
    torch.testing.assert_close(result.cpu().transpose(0, 1), ref_program(A_int8.cpu(), qB), rtol=0, atol=0)
    assert torch.equal(torch_convert(qB), B_int8_ref)
    print(f"Test passed: M={M}, N={N}, K={K}")


def main(custom_args=None):
    tilelang.disable_cache()
    torch.manual_seed(42)
    parser = argparse.ArgumentParser()
    for flag in ("--M", "--N", "--K"):
        parser.add_argument(flag, type=int, default=0)
    args = parser.parse_args(custom_args)
    if args.M > 0 and args.N > 0 and args.K > 0:
        test(args.M, args.N, args.K)
    else:
        for shape in ((64, 64, 256), (128, 128, 512), (256, 256, 1024)):
            test(*shape)
    tilelang.enable_cache()
    print("Test Passed!")


if __name__ == "__main__":
    main()
