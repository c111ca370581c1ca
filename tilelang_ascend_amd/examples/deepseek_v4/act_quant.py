#!/usr/bin/env python3
"""Per-token int8 activation quantiser, the run of the reference's examples/deepseek_v4/act_quant.py
(:151-172): M=128, N=1024 bfloat16, kernel(N, block_M=16, block_N=N), checked against the torch
golden with Y atol=1 and S rtol=atol=1e-2; logs "init successful!" then "Kernel Output Match!"."""
import logging
from typing import Tuple

import torch

from tilelang_ascend_amd.ops import act_quant_kernel_int8_optimized

logging.basicConfig(level=logging.INFO)


def act_quant_torch(x: torch.Tensor, round_scale: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    x2 = x.reshape(-1, x.shape[-1]).float()
    abs_max = torch.clamp(x2.abs().amax(dim=1, keepdim=True), min=1e-4)
    scales = 2 ** torch.ceil(torch.log2(abs_max / 127.0)) if round_scale else abs_max / 127.0
    y = torch.round(torch.clamp(x2 / scales, -127, 127)).to(torch.float16).to(torch.int8)
    return y.view(x.shape), scales.view(*x.shape[:-1], 1)


def test(custom_args=None):
    torch.manual_seed(42)
    M, N = 128, 1024
    x_bf16 = torch.randn(M, N, dtype=torch.bfloat16)
    kernel = act_quant_kernel_int8_optimized(N, block_M=16, block_N=N, round_scale=False)
    logging.info("init successful!")
    Y, S = kernel(x_bf16.cuda())
    torch.cuda.synchronize()
    x_int8_torch, scales_torch = act_quant_torch(x_bf16)
    torch.testing.assert_close(Y.cpu(), x_int8_torch, rtol=1e-2, atol=1)
    torch.testing.assert_close(S.cpu().reshape(M), scales_torch.reshape(M), rtol=1e-2, atol=1e-2)
    logging.info("Kernel Output Match!")


if __name__ == "__main__":
    test()
