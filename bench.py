#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload gemv|prefill|w8a8|skinny|actquant|mlp-sweep] [--units U]

Headline workload (default): the W4A16 decode GEMV -- M=1, N=11008, K=4096, fp16 activations,
uint4 weights packed low-nibble-first, group 128, fp16 scales U[0.005,0.02] and fp16 zeros U{6..9},
fp16 output, fp32 accumulation.  One "step" is one launch of the GEMV kernel over `units`
independent weight sets (default 1).  The weight sets rotate through a pool larger than the
256 MB last-level cache, so every step streams its weights from HBM.  Inputs are resident in
HBM before the timed region starts.

Prints ONE JSON line.  `value` is algorithmic bytes / wall time (GB/s); `roofline` describes the
dominant kernel from HIP events recorded on the launch stream around the timed region;
`cpu_baseline` is the CPU oracle (the reference's torch ref_program arithmetic) timed on the
host cores on a bounded sample; `other_workloads` carries the prefill GEMM and W8A8 figures.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
MFMA_I8_PEAK_TOPS = 5000.0
POOL_BYTES = 576 * 1024 * 1024  # weight pool > 2x the 256 MB last-level cache
# HBM bytes per launch from hardware counters (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE in separate
# runs of this script with --calibrate-copy, each scaled by what the counter reads for the 256 MiB
# copy kernel: x2.000 and x1.000); the summaries are the text files under profiles/.
TRAFFIC_GEMV_1SET = 24_110_000
TRAFFIC_PREFILL = 162_900_000
TRAFFIC_W8A8 = 935_200_000
TRAFFIC_SKINNY = 33_130_000
TRAFFIC_ACT_QUANT = 201_554_000


def w4a16_bytes(M, N, K, group, zeros_tensor=True, elem=2):
    """Algorithmic bytes of one W4A16 problem: packed weights + scales (+ zeros) + A + C."""
    return N * K // 2 + (2 if zeros_tensor else 1) * elem * N * K // group + elem * M * K + elem * M * N


def w8a8_bytes(B, M, N, K):
    return B * M * K + B * K * N + 2 * B * M * N + 4 * B * M + 4 * N


def timed(fn, steps, warmup):
    """Returns (wall seconds per step, event-measured seconds per step)."""
    import torch

    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) / steps, e0.elapsed_time(e1) * 1e-3 / steps


def bench_gemv(args, units=None, steps=None, warmup=None, cpu=True):
    import torch

    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    dev = torch.device("cuda:0")
    M, N, K, g = 1, 11008, 4096, 128
    units = units or args.units
    steps = steps or args.steps
    warmup = args.warmup if warmup is None else warmup
    unit_bytes = w4a16_bytes(M, N, K, g)
    sets = max(2 * units, -(-POOL_BYTES // unit_bytes))
    sets = -(-sets // units) * units
    gen = torch.Generator(device="cpu").manual_seed(0)
    Wp = torch.randint(0, 256, (sets, N, K // 2), dtype=torch.uint8, generator=gen).to(dev)
    S = (torch.rand(sets, N, K // g, generator=gen) * 0.015 + 0.005).to(torch.float16).to(dev)
    Z = torch.randint(6, 10, (sets, N, K // g), generator=gen).to(torch.float16).to(dev)
    A = torch.randn(sets, M, K, generator=gen).to(torch.float16).to(dev)
    C = torch.empty(sets, M, N, dtype=torch.float16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    groups = sets // units

    # argument tuples are prepared up front: per-step tensor indexing would cost more host time
    # than the kernel runs for
    if units == 1:
        pre = [(P(A[j]), P(Wp[j]), P(S[j]), P(Z[j]), P(C[j]), M, N, K, g, 0.0, _abi.F16, _abi.F16, _abi.ALGO_GEMV, stream)
               for j in range(sets)]
        entry = lib.tlq_gemm_w4a16
    else:
        pre = [(P(A[j]), P(Wp[j]), P(S[j]), P(Z[j]), P(C[j]), units, M, N, K, g, 0.0, _abi.F16, _abi.F16, stream)
               for j in range(0, sets, units)]
        entry = lib.tlq_gemv_w4a16_batched

    def step(i):
        if entry(*pre[i % groups]):
            raise RuntimeError(_abi.last_error())

    wall, ev = timed(step, steps, warmup)
    step_bytes = unit_bytes * units
    # spot check of the last result against the oracle (outside the timed region)
    from oracle import ref

    j = ((steps - 1) % groups) * units
    want = ref.ref_program_w4a16(A[j].cpu(), Wp[j].cpu(), S[j].cpu(), Z[j].cpu(), g, "float32")
    rel = ((C[j].float().cpu() - want).norm() / want.norm()).item()
    if rel > 1e-3:
        raise RuntimeError(f"GEMV result differs from the oracle: relative L2 {rel}")

    cpu = cpu_baseline_gemv(A[0].cpu(), Wp[0].cpu(), S[0].cpu(), Z[0].cpu(), g, unit_bytes) if cpu else None
    return {
        "metric": "W4A16 GEMV GB/s (%HBM peak) at M=1; W4A16/W8A8 GEMM TFLOP/s (%MFMA peak)",
        "value": round(step_bytes / wall / 1e9, 1),
        "unit": "GB/s",
        "ms_per_step": wall * 1e3,
        "dtype": "f16",
        "config": {"workload": f"W4A16 decode GEMV M=1 N=11008 K=4096 group=128 fp16 scales+zeros, {units} weight set(s) per launch, "
                               f"{sets} sets rotating ({sets * unit_bytes >> 20} MiB)",
                   "M": M, "N": N, "K": K, "group": g, "units_per_launch": units},
        "roofline": {"kernel": "gemv_w4a16_f16_rows_kernel", "bound": "hbm", "achieved": round(step_bytes / ev / 1e9, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(step_bytes / ev / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": TRAFFIC_GEMV_1SET * units, "bytes_per_launch": step_bytes, "avg_launch_us": round(ev * 1e6, 3)},
        "cpu_baseline": cpu,
        "parity_rel_l2": rel,
    }


def cpu_baseline_gemv(A, Wp, S, Z, g, unit_bytes, budget_s=10.0):
    """The reference's CPU path for this workload: vectorised nibble unpack, (u - z) * s in fp16,
    fp32 matmul, cast (oracle.ref.ref_program_w4a16), timed on the host cores."""
    import torch

    from oracle import ref

    ref.ref_program_w4a16(A, Wp, S, Z, g, "float16")  # warm-up
    reps, t0 = 0, time.perf_counter()
    while True:
        ref.ref_program_w4a16(A, Wp, S, Z, g, "float16")
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s and reps >= 3 or reps >= 200:
            break
    per = dt / reps
    return {"value": round(unit_bytes / per / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{reps} evaluations of the same M=1 N=11008 K=4096 GEMV (unpack + dequant + fp32 matmul) in {dt:.1f} s",
            "ms_per_eval": round(per * 1e3, 2), "host_cpus": os.cpu_count()}


def bench_prefill(args, steps=None):
    import torch

    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    dev = torch.device("cuda:0")
    M = N = K = 4096
    g = 128
    gen = torch.Generator(device="cpu").manual_seed(1)
    Wp = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=gen).to(dev)
    S = (torch.rand(N, K // g, generator=gen) * 0.015 + 0.005).to(torch.bfloat16).to(dev)
    A = torch.randn(M, K, generator=gen).to(torch.bfloat16).to(dev)
    C = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    ws_bytes = lib.tlq_w4a16_workspace_bytes(M, N, K)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

    def step(i):  # dequantise into the workspace, then the plain MFMA GEMM (two launches)
        rc = lib.tlq_gemm_w4a16_ws(P(A), P(Wp), P(S), None, P(C), M, N, K, g, 8.0, _abi.BF16, _abi.BF16, _abi.ALGO_AUTO,
                                   P(ws), ws_bytes, stream)
        if rc:
            raise RuntimeError(_abi.last_error())

    def step_fused(i):  # the single fused kernel, for comparison
        rc = lib.tlq_gemm_w4a16(P(A), P(Wp), P(S), None, P(C), M, N, K, g, 8.0, _abi.BF16, _abi.BF16, _abi.ALGO_MFMA, stream)
        if rc:
            raise RuntimeError(_abi.last_error())

    wall, ev = timed(step_fused, steps or args.steps, args.warmup)
    wall2, ev2 = timed(step, steps or args.steps, min(args.warmup, 4))
    flops = 2.0 * M * N * K
    # primary figure: the fused kernel (dequantised weight tiles staged through LDS into MFMA); alongside, the two
    # launches that a caller-owned workspace allows (whole step priced against the MFMA peak)
    return {"workload": "W4A16 prefill GEMM M=N=K=4096 bf16 group=128 zero=8", "dtype": "bf16",
            "value": round(flops / wall / 1e12, 1), "unit": "TFLOP/s", "ms_per_step": wall * 1e3,
            "roofline": {"kernel": "gemm_mfma_kernel<MmaBF16,RowLoaderDirect,W4Loader>", "bound": "mfma", "achieved": round(flops / ev / 1e12, 1),
                         "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(flops / ev / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                         "traffic": TRAFFIC_PREFILL, "flops_per_launch": flops, "avg_launch_us": round(ev * 1e6, 2)},
            "with_workspace": {"path": "tlq_gemm_w4a16_ws: dequant_w4_vec8 into a caller-owned workspace, then "
                                       "gemm_mfma_kernel<MmaBF16,RowLoaderDirect,RowLoaderDirect>",
                               "value": round(flops / wall2 / 1e12, 1), "unit": "TFLOP/s", "us_per_step": round(ev2 * 1e6, 2),
                               "frac_of_mfma_peak": round(flops / ev2 / 1e12 / MFMA_F16_PEAK_TFLOPS, 4)}}


def bench_skinny(args, steps=None):
    """cfg-5 decode batch: M=16 activations against a 14336 x 4096 weight matrix (HBM bound)."""
    import torch

    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    dev = torch.device("cuda:0")
    M, N, K, g = 16, 14336, 4096, 128
    unit_bytes = w4a16_bytes(M, N, K, g)
    sets = -(-POOL_BYTES // unit_bytes)
    gen = torch.Generator(device="cpu").manual_seed(3)
    Wp = torch.randint(0, 256, (sets, N, K // 2), dtype=torch.uint8, generator=gen).to(dev)
    S = (torch.rand(sets, N, K // g, generator=gen) * 0.015 + 0.005).to(torch.float16).to(dev)
    Z = torch.randint(6, 10, (sets, N, K // g), generator=gen).to(torch.float16).to(dev)
    A = torch.randn(M, K, generator=gen).to(torch.float16).to(dev)
    C = torch.empty(M, N, dtype=torch.float16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    pre = [(P(A), P(Wp[j]), P(S[j]), P(Z[j]), P(C), M, N, K, g, 0.0, _abi.F16, _abi.F16, _abi.ALGO_AUTO, stream)
           for j in range(sets)]

    def step(i):
        if lib.tlq_gemm_w4a16(*pre[i % sets]):
            raise RuntimeError(_abi.last_error())

    wall, ev = timed(step, steps or args.steps, args.warmup)
    return {"workload": f"W4A16 decode batch M=16 N=14336 K=4096 group=128 fp16 scales+zeros, {sets} weight sets rotating",
            "dtype": "f16", "value": round(unit_bytes / wall / 1e9, 1), "unit": "GB/s", "ms_per_step": wall * 1e3,
            "roofline": {"kernel": "w4a16_skinny_lds_kernel", "bound": "hbm", "achieved": round(unit_bytes / ev / 1e9, 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(unit_bytes / ev / 1e9 / HBM_PEAK_GBS, 4),
                         "traffic": TRAFFIC_SKINNY, "bytes_per_launch": unit_bytes, "avg_launch_us": round(ev * 1e6, 3)}}


def bench_act_quant(args, steps=None):
    """Per-token int8 quantiser on the activations of the W8A8 workload: 16384 tokens x 4096, bf16 in."""
    import torch

    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    dev = torch.device("cuda:0")
    M, N = 8 * 2048, 4096
    unit_bytes = M * N * 3 + 4 * M
    sets = -(-POOL_BYTES // (2 * M * N))
    gen = torch.Generator(device="cpu").manual_seed(4)
    X = torch.randn(M, N, generator=gen).to(torch.bfloat16).to(dev).repeat(sets, 1, 1)
    X *= torch.linspace(0.5, 2.0, sets, device=dev).view(sets, 1, 1).to(torch.bfloat16)
    Y = torch.empty(M, N, dtype=torch.int8, device=dev)
    S = torch.empty(M, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    pre = [(P(X[j]), P(Y), P(S), M, N, _abi.BF16, 0, stream) for j in range(sets)]

    def step(i):
        if lib.tlq_act_quant_i8(*pre[i % sets]):
            raise RuntimeError(_abi.last_error())

    wall, ev = timed(step, steps or args.steps, args.warmup)
    return {"workload": f"per-token int8 activation quantiser M=16384 N=4096 bf16 in, {sets} inputs rotating",
            "dtype": "f32", "value": round(unit_bytes / wall / 1e9, 1), "unit": "GB/s", "ms_per_step": wall * 1e3,
            "roofline": {"kernel": "act_quant_rows_kernel<bf16,8,1>", "bound": "hbm", "achieved": round(unit_bytes / ev / 1e9, 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(unit_bytes / ev / 1e9 / HBM_PEAK_GBS, 4),
                         "traffic": TRAFFIC_ACT_QUANT, "bytes_per_launch": unit_bytes, "avg_launch_us": round(ev * 1e6, 3)}}


def bench_mlp_sweep(args, steps=None):
    """cfg-5 sweep: M in {16, 64, 256, 1024, 8192} x (N, K) in {(14336, 4096), (4096, 14336)} x group in {128, 64},
    fp16, per-group scales and zeros, automatic kernel choice with a workspace (tlq_gemm_w4a16_ws)."""
    import torch

    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    for (N, K) in ((14336, 4096), (4096, 14336)):
        for g in (128, 64):
            sets = 6  # 6 x 29 MB of packed weights rotate: small-M launches always stream from HBM
            gen = torch.Generator(device="cpu").manual_seed(5)
            Wp = torch.randint(0, 256, (sets, N, K // 2), dtype=torch.uint8, generator=gen).to(dev)
            S = (torch.rand(sets, N, K // g, generator=gen) * 0.015 + 0.005).to(torch.float16).to(dev)
            Z = torch.randint(6, 10, (sets, N, K // g), generator=gen).to(torch.float16).to(dev)
            for M in (16, 64, 256, 1024, 8192):
                A = torch.randn(M, K, generator=gen).to(torch.float16).to(dev)
                C = torch.empty(M, N, dtype=torch.float16, device=dev)
                ws_bytes = lib.tlq_w4a16_workspace_bytes(M, N, K)
                ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
                pre = [(P(A), P(Wp[j]), P(S[j]), P(Z[j]), P(C), M, N, K, g, 0.0, _abi.F16, _abi.F16, _abi.ALGO_AUTO,
                        P(ws) if ws_bytes else None, ws_bytes, stream) for j in range(sets)]

                def step(i):
                    if lib.tlq_gemm_w4a16_ws(*pre[i % sets]):
                        raise RuntimeError(_abi.last_error())

                _, ev = timed(step, steps or (12 if M < 8192 else 4), 3)
                flops, nbytes = 2.0 * M * N * K, w4a16_bytes(M, N, K, g)
                rows.append({"M": M, "N": N, "K": K, "group": g, "us": round(ev * 1e6, 1),
                             "TFLOP/s": round(flops / ev / 1e12, 1), "frac_mfma": round(flops / ev / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                             "GB/s": round(nbytes / ev / 1e9), "frac_hbm": round(nbytes / ev / 1e9 / HBM_PEAK_GBS, 4)})
                del A, C, ws
            del Wp, S, Z
    big = max(rows, key=lambda r: r["TFLOP/s"])
    return {"workload": "W4A16 MLP-shaped sweep, fp16, 20 shapes, automatic kernel choice with workspace", "dtype": "f16",
            "value": big["TFLOP/s"], "unit": "TFLOP/s", "ms_per_step": big["us"] * 1e-3,
            "roofline": {"kernel": "best of the sweep (M=%d N=%d K=%d)" % (big["M"], big["N"], big["K"]), "bound": "mfma",
                         "achieved": big["TFLOP/s"], "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": big["frac_mfma"],
                         "traffic": None},
            "shapes": rows}


def bench_w8a8(args, steps=None):
    import torch

    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    dev = torch.device("cuda:0")
    B, M, N, K = 8, 2048, 4096, 4096
    gen = torch.Generator(device="cpu").manual_seed(2)
    A = torch.randint(-127, 128, (B, M, K), dtype=torch.int8, generator=gen).to(dev)
    W = torch.randint(-127, 128, (B, K, N), dtype=torch.int8, generator=gen).to(dev)
    sa = (torch.rand(B, M, generator=gen) * 0.04 + 0.01).to(dev)
    sb = (torch.rand(N, generator=gen) * 0.009 + 0.001).to(dev)
    C = torch.empty(B, M, N, dtype=torch.float16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def step(i):
        rc = lib.tlq_gemm_w8a8(P(A), P(W), P(sa), P(sb), P(C), B, M, N, K, N, _abi.B_KN, _abi.F16, stream)
        if rc:
            raise RuntimeError(_abi.last_error())

    wall, ev = timed(step, steps or args.steps, args.warmup)
    ops = 2.0 * B * M * N * K
    return {"workload": "W8A8 quant batch matmul B=8 M=2048 N=K=4096, per-token x per-channel rescale, fp16 out",
            "dtype": "i8", "value": round(ops / wall / 1e12, 1), "unit": "TOP/s", "ms_per_step": wall * 1e3,
            "roofline": {"kernel": "gemm_mfma_kernel<MmaI8,RowLoaderDirect,I8KNLoaderDirect,EpiRescale>", "bound": "mfma",
                         "achieved": round(ops / ev / 1e12, 1), "peak": MFMA_I8_PEAK_TOPS, "unit": "TOP/s",
                         "frac": round(ops / ev / 1e12 / MFMA_I8_PEAK_TOPS, 4), "traffic": TRAFFIC_W8A8, "ops_per_launch": ops,
                         "avg_launch_us": round(ev * 1e6, 2)}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=480)
    ap.add_argument("--warmup", type=int, default=48)
    ap.add_argument("--workload", default="gemv", choices=["gemv", "prefill", "w8a8", "skinny", "actquant", "mlp-sweep"])
    ap.add_argument("--units", type=int, default=1, help="independent weight sets per GEMV launch")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-side baseline (profiling runs)")
    ap.add_argument("--tune", action="append", default=[], metavar="HOOK=VALUE",
                    help="call a single-integer tuning hook of the library before measuring, e.g. --tune gemm_slots=1 "
                         "(tlq_tune_gemm_slots(1)); repeatable; recorded in the output line")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain elementwise copy of 256 MiB (int32 x+0 -> y) after the timed region, "
                         "the known-size kernel that hardware traffic counters are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU's share of the path; --gpus {args.gpus} is not supported in this build "
              "(the path shards over the weight rows N: each GPU holds its rows and all activations, no exchange).",
              file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)

    tuned = {}
    if args.tune:
        from tilelang_ascend_amd import _abi

        lib = _abi.load()
        for item in args.tune:
            name, _, value = item.partition("=")
            hook = "tlq_tune_" + name.strip()
            sig = _abi.SIGNATURES.get(hook)
            if sig is None or len(sig[1]) != 1:
                print(f"bench.py: no single-integer tuning hook {hook}", file=sys.stderr)
                sys.exit(2)
            getattr(lib, hook)(int(value))
            tuned[hook] = int(value)

    if args.workload == "gemv":
        line = bench_gemv(args, cpu=not args.no_cpu_baseline)
        if not args.no_extra:
            # secondary workloads: a failure in one of them is reported in its place and never costs the headline figure
            def many_sets():
                many = bench_gemv(args, units=24, steps=20, warmup=4, cpu=False)
                return {"workload": many["config"]["workload"], "dtype": "f16", "value": many["value"], "unit": "GB/s",
                        "ms_per_step": many["ms_per_step"], "roofline": many["roofline"]}

            others = []
            for name, fn in (("gemv, 24 weight sets per launch", many_sets),
                             ("skinny", lambda: bench_skinny(args, steps=60)),
                             ("prefill", lambda: bench_prefill(args, steps=20)),
                             ("w8a8", lambda: bench_w8a8(args, steps=10)),
                             ("actquant", lambda: bench_act_quant(args, steps=40))):
                try:
                    others.append(fn())
                except Exception as e:  # noqa: BLE001
                    others.append({"workload": name, "error": f"{type(e).__name__}: {e}"})
            line["other_workloads"] = others
    else:
        res = {"prefill": bench_prefill, "w8a8": bench_w8a8, "skinny": bench_skinny,
               "actquant": bench_act_quant, "mlp-sweep": bench_mlp_sweep}[args.workload](args)
        line = {"metric": "W4A16 GEMV GB/s (%HBM peak) at M=1; W4A16/W8A8 GEMM TFLOP/s (%MFMA peak)",
                "value": res["value"], "unit": res["unit"], "ms_per_step": res["ms_per_step"], "dtype": res["dtype"],
                "config": {"workload": res["workload"]}, "roofline": res["roofline"], "cpu_baseline": None}
        for extra in ("shapes", "with_workspace"):
            if extra in res:
                line[extra] = res[extra]
    if args.calibrate_copy:
        src = torch.zeros(64 * 1024 * 1024, dtype=torch.int32, device="cuda:0")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        torch.add(src, 0, out=dst)
        torch.cuda.synchronize()
    line.update({"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
                 "vs_baseline": None, "data": "synthetic"})
    if tuned:
        line["tuning_hooks"] = tuned
    order = ["metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
             "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"]
    out = {k: line[k] for k in order if k in line}
    out.update({k: v for k, v in line.items() if k not in out})
    print(json.dumps(out))


if __name__ == "__main__":
    main()
