#!/usr/bin/env python3
"""Per-token x per-channel W8A8 GEMM, the run of the reference's examples/deepseek_v4/int8_gemm.py
(:142-176): M=N=K=1024, bfloat16 activations and weights quantised per row on the host exactly as
there (clamp to [-128, 127], round), kernel(N, K, 64, 64, 64, out_dtype=bfloat16), checked against
the float32 torch golden with rtol=atol=1e-2; logs "init successful!" then "Kernel Output Match!"."""
import logging

import torch

from tilelang_ascend_amd.ops import int8_gemm_kernel_corrected

logging.basicConfig(level=logging.INFO)
BF16 = "bfloat16"


def int8_gemm_torch_optimized(a_int8, a_scales, b_int8, b_scales, out_dtype=torch.float32):
    out = torch.matmul(a_int8.reshape(-1, a_int8.shape[-1]).float(), b_int8.float().T)
    out = out * torch.outer(a_scales.reshape(-1), b_scales.reshape(-1))
    if out_dtype == torch.bfloat16:
        out = out.bfloat16()
    return out.view(*a_int8.shape[:-1], b_int8.shape[0])


def quantize_rows(x_bf16):
    x = x_bf16.float()
    scales = torch.clamp(x.abs().amax(dim=1, keepdim=True), min=1e-4) / 127.0
    return torch.clamp(x / scales, -128, 127).round().to(torch.int8), scales


def test(custom_args=None):
    torch.manual_seed(42)
    M, N, K = 1024, 1024, 1024
    a_int8, a_scales = quantize_rows(torch.randn(M, K, dtype=torch.bfloat16))
    b_int8, b_scales = quantize_rows(torch.randn(N, K, dtype=torch.bfloat16))
    kernel = int8_gemm_kernel_corrected(N, K, block_M=64, block_N=64, block_K=64, out_dtype=BF16)
    logging.info("init successful!")
    result = kernel(a_int8.cuda(), b_int8.cuda(), a_scales.reshape(M).cuda(), b_scales.reshape(N).cuda())
    torch.cuda.synchronize()
    want = int8_gemm_torch_optimized(a_int8, a_scales, b_int8, b_scales, out_dtype=torch.bfloat16)
    torch.testing.assert_close(result.cpu(), want, rtol=1e-2, atol=1e-2)
    logging.info("Kernel Output Match!")


if __name__ == "__main__":
    test()
