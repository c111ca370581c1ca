#!/usr/bin/env python3
"""Writes the committed fixtures of this directory from the CPU oracles.

    python tests/golden/make_golden.py

* kat_unpack_uint4.json -- the known-answer vector held by the reference's own test
  (examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:384-401), typed in as data.
* w4a16_small.npz / int8_small.npz -- seeded inputs and the outputs both oracles (numpy/torch
  and the C restatement) agree on; the generator refuses to write a case on which they differ.

The fixtures let the GPU tests compare against frozen numbers as well as against the live
oracle, and let the CPU tests notice an accidental change of the oracle.
"""
from __future__ import annotations

import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import cref, ref  # noqa: E402

KAT = {"source": "examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:384-401",
       "packed": [[0x12, 0x34]], "shape": [1, 4], "expected": [[2, 1, 4, 3]]}


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def w4a16_cases() -> dict:
    """name -> array.  Per case c: c.A, c.Wp, c.S, c.Z (bit patterns, absent when unused), c.meta
    = [M, N, K, group, dtype(0 f16 / 1 bf16), zero_scalar], c.W (dequantised weights, bits) and
    c.C (fp32 accumulate, fp32 output)."""
    out = {}
    cases = [("f16_g128_tensorz", 3, 48, 256, 128, torch.float16, "tensor"),
             ("f16_g32_scalar8", 17, 40, 192, 32, torch.float16, 8.0),
             ("bf16_g64_tensorz", 1, 64, 128, 64, torch.bfloat16, "tensor"),
             ("bf16_g128_scalar8", 33, 16, 384, 128, torch.bfloat16, 8.0),
             ("f16_plain", 16, 16, 64, 64, torch.float16, None)]
    for i, (name, M, N, K, g, dt, zk) in enumerate(cases):
        gen = torch.Generator().manual_seed(100 + i)
        kind = 0 if dt == torch.float16 else 1
        A = torch.randn(M, K, generator=gen).to(dt)
        Wp = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=gen)
        S = None if zk is None else (torch.rand(N, K // g, generator=gen) * 0.015 + 0.005).to(dt)
        Z = torch.randint(6, 10, (N, K // g), generator=gen).to(dt) if zk == "tensor" else None
        zs = float(zk) if isinstance(zk, float) else 0.0
        W = ref.dequant_w4(Wp, S, Z if Z is not None else (zs if zs else None), g, dt)
        Wc = cref.dequant_w4(Wp.numpy(), None if S is None else _bits(S), None if Z is None else _bits(Z), zs, g, kind)
        if not np.array_equal(Wc, _bits(W)):
            raise SystemExit(f"{name}: the two oracles disagree on the dequantised weights")
        C = ref.ref_program_w4a16(A, Wp, S, Z if Z is not None else (zs if zs else None), g, "float32").numpy()
        Cc = cref.gemm_w4a16(_bits(A), _bits(W), kind, 2)
        if not np.allclose(C, Cc, rtol=2e-6, atol=1e-6):
            raise SystemExit(f"{name}: the two oracles disagree on the GEMM")
        out[f"{name}.meta"] = np.array([M, N, K, g, kind, zs], dtype=np.float64)
        out[f"{name}.A"] = _bits(A)
        out[f"{name}.Wp"] = Wp.numpy().copy()
        if S is not None:
            out[f"{name}.S"] = _bits(S)
        if Z is not None:
            out[f"{name}.Z"] = _bits(Z)
        out[f"{name}.W"] = _bits(W)
        out[f"{name}.C"] = Cc.astype(np.float32)  # double accumulation rounded once to fp32
    return out


def int8_cases() -> dict:
    """Integer cases: i8 x i8 (both weight layouts), uint4 / int4 weights, and the rescaled output."""
    out = {}
    gen = torch.Generator().manual_seed(200)
    B, M, N, K = 2, 19, 48, 160
    A = torch.randint(-128, 128, (B, M, K), dtype=torch.int8, generator=gen)
    W = torch.randint(-128, 128, (B, K, N), dtype=torch.int8, generator=gen)
    acc = ref.int_matmul_exact(A, W).to(torch.int32)
    for b in range(B):
        if not np.array_equal(cref.gemm_i8(A[b].numpy(), W[b].numpy(), 0), acc[b].numpy()):
            raise SystemExit("int8: the two oracles disagree")
    sa = (torch.rand(B, M, generator=gen) * 0.04 + 0.01).float()
    sb = (torch.rand(N, generator=gen) * 0.009 + 0.001).float()
    out["i8.A"], out["i8.W_kn"], out["i8.acc"] = A.numpy().copy(), W.numpy().copy(), acc.numpy().copy()
    out["i8.scale_a"], out["i8.scale_b"] = sa.numpy().copy(), sb.numpy().copy()
    out["i8.C_scale_b_f16"] = _bits(ref.ref_program_quant(A, W, sb, torch.float16))
    out["i8.C_scale_1_bf16"] = _bits(ref.ref_program_quant(A, W, sb[:1], torch.bfloat16))
    seq = ref.ref_int8_gemm_sequential(A, W.transpose(1, 2).contiguous(), sa, sb, torch.float16)
    for b in range(B):
        c = cref.rescale(acc[b].numpy(), sa[b].numpy(), sb.numpy(), 0)
        if not np.array_equal(c, _bits(seq[b])):
            raise SystemExit("rescale: the two oracles disagree")
    out["i8.C_token_channel_f16"] = _bits(seq)
    # packed 4-bit weights against int8 activations
    Wp = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=gen)
    out["w4.Wp"] = Wp.numpy().copy()
    out["w4.unsigned"] = ref.torch_unpack_uint4_to_int8(Wp).numpy().copy()
    out["w4.signed"] = ref.torch_convert(Wp).numpy().copy()
    if not np.array_equal(out["w4.unsigned"], cref.unpack_u4(Wp.numpy())) or \
            not np.array_equal(out["w4.signed"], cref.convert_s4(Wp.numpy())):
        raise SystemExit("unpack: the two oracles disagree")
    out["w4.C_unsigned"] = ref.ref_program_int8(A[0], Wp, "int32").numpy().copy()
    out["w4.C_signed_t"] = ref.ref_program_w4a8(A[0], Wp).contiguous().numpy().copy()  # [N, M]
    return out


def main() -> None:
    with open(os.path.join(HERE, "kat_unpack_uint4.json"), "w") as f:
        json.dump(KAT, f, indent=1)
        f.write("\n")
    np.savez_compressed(os.path.join(HERE, "w4a16_small.npz"), **w4a16_cases())
    np.savez_compressed(os.path.join(HERE, "int8_small.npz"), **int8_cases())
    for n in sorted(os.listdir(HERE)):
        print(n, os.path.getsize(os.path.join(HERE, n)))


if __name__ == "__main__":
    main()
