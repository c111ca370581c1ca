#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload gemv|small|prefill|w8a8|skinny|actquant|mlp-sweep|vendor-gemm] [--units U]

Headline workload (default): the W4A16 decode GEMV -- M=1, N=11008, K=4096, fp16 activations,
uint4 weights packed low-nibble-first, group 128, fp16 scales U[0.005,0.02] and fp16 zeros U{6..9},
fp16 output, fp32 accumulation.  One "step" is one launch of the GEMV kernel over `units`
independent weight sets (default 1).  The weight sets rotate through a pool larger than the
256 MB last-level cache, so every step streams its weights from HBM.  Inputs are resident in
HBM before the timed region starts.

Prints ONE JSON line.
  * A timed REGION is exactly K steps (--steps) between two synchronisations, with a HIP event on the launch stream on
    either side.  The region is repeated (`regions`: up to 25 times, within about a second per workload) and the MEDIAN
    region is reported, so that one slow region -- a clock ramp, a noisy neighbour -- does not decide the line; the
    spread is in `roofline.region_us_min` / `region_us_max`.
  * `value` is algorithmic bytes / WALL-CLOCK time per step of the median region: it includes the host side of every
    launch (the ctypes call into the C ABI, about 2 us, which a microsecond kernel does not hide).
  * `roofline.achieved` is algorithmic bytes (or operations) / the step time between the two HIP events of the median
    region.  After the timed regions the same step runs again with one event pair per step; `roofline.median_us` and
    `roofline.min_us` come from those pairs (each pair adds the event markers' own cost, about a microsecond, so they
    bound the kernel from above and are not comparable with the back-to-back average).
  * `roofline.kernel` is the library's own launch log of one step (tlq_debug_launch_log: entry point [kernel, variant]
    of every launch the call made), not a constant of this script.
  * `roofline.traffic` is NOT measured by this run: it is read from the counter summary under profiles/ for that kernel
    and workload (a line "traffic_bytes_per_launch: N"; `roofline.traffic_source` names the file), null without one.
  * `cpu_baseline` is the CPU oracle (the reference's torch ref_program arithmetic) timed on the host cores on a bounded
    sample; every entry of `other_workloads` (the other configurations) carries its own.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
MFMA_I8_PEAK_TOPS = 5000.0
POOL_BYTES = 576 * 1024 * 1024  # weight pool > 2x the 256 MB last-level cache
METRIC = "W4A16 GEMV GB/s (%HBM peak) at M=1; W4A16/W8A8 GEMM TFLOP/s (%MFMA peak)"
WALL_NOTE = "value = algorithmic bytes / wall-clock per step incl. the host-side launch call; roofline.* from HIP events"


def traffic_from_profile(name):
    """HBM bytes per launch as measured with hardware counters in an earlier profiling run: the line
    'traffic_bytes_per_launch: N' of profiles/<name> (FETCH_SIZE + WRITE_SIZE, each scaled by a copy kernel of known
    size).  Returns the two roofline fields {traffic, traffic_source}; traffic is None without such a line."""
    val = None
    try:
        with open(os.path.join(ROOT, "profiles", name)) as f:
            m = re.search(r"^traffic_bytes_per_launch\s*:\s*(\d+)", f.read(), re.M)
        val = int(m.group(1)) if m else None
    except OSError:
        pass
    return {"traffic": val, "traffic_source": ("profiles/" + name + " (counters of an earlier run, not of this one)") if val is not None else None}


def w4a16_bytes(M, N, K, group, zeros_tensor=True, elem=2):
    """Algorithmic bytes of one W4A16 problem: packed weights + scales (+ zeros) + A + C."""
    return N * K // 2 + (2 if zeros_tensor else 1) * elem * N * K // group + elem * M * K + elem * M * N


def w8a8_bytes(B, M, N, K):
    return B * M * K + B * K * N + 2 * B * M * N + 4 * B * M + 4 * N


class Timing:
    """wall / ev: seconds per step of the median timed region (host clock / HIP events around the region's loop);
    ev_all: the same for every region; median / best: seconds per step from one event pair per step, taken after the
    timed regions; kernel: the library's launch log of one step."""

    def __init__(self, walls, evs, per_step, kernel):
        order = sorted(range(len(evs)), key=lambda i: evs[i])
        mid = order[len(order) // 2]
        self.wall, self.ev = walls[mid], evs[mid]
        self.ev_all = evs
        self.median = statistics.median(per_step) if per_step else None
        self.best = min(per_step) if per_step else None
        self.pairs = len(per_step)
        self.kernel = kernel

    def roofline(self, work, peak, unit, scale):
        """work per step (bytes or operations), peak in `unit`, scale = 1e9 for GB/s, 1e12 for T.../s."""
        ach = work / self.ev / scale
        out = {"kernel": self.kernel, "achieved": round(ach, 1), "peak": peak, "unit": unit, "frac": round(ach / peak, 4),
               "avg_launch_us": round(self.ev * 1e6, 3), "regions": len(self.ev_all),
               "region_us_min": round(min(self.ev_all) * 1e6, 3), "region_us_max": round(max(self.ev_all) * 1e6, 3)}
        if self.pairs:
            out.update({"median_us": round(self.median * 1e6, 3), "min_us": round(self.best * 1e6, 3),
                        "per_step_event_pairs": self.pairs})
        return out


def launch_log_of(fn):
    """What one step launches, by the library's own record."""
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    lib.tlq_debug_launch_log(1)
    try:
        fn(0)
        text = lib.tlq_debug_launch_log_text()
    finally:
        lib.tlq_debug_launch_log(0)
    return text.decode() if isinstance(text, bytes) else str(text)


def timed(fn, steps, warmup, pairs=None, regions=None):
    """warmup untimed steps, then regions of exactly `steps` timed ones between two synchronisations each (up to 25
    regions, fewer when a region is long: about a second in all); then `pairs` more steps (default min(steps, 200)) with
    one event pair each."""
    import torch

    kernel = launch_log_of(fn)
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    walls, evs = [], []
    budget_s, t_begin = 1.0, time.perf_counter()
    want = 25 if regions is None else regions
    base = 0
    while len(evs) < want:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for i in range(steps):
            fn(base + i)
        e1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        walls.append((t1 - t0) / steps)
        evs.append(e0.elapsed_time(e1) * 1e-3 / steps)
        base += steps
        if len(evs) >= 5 and time.perf_counter() - t_begin > budget_s:
            break
    n = min(steps, 200) if pairs is None else pairs
    pair_evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for i, (a, b) in enumerate(pair_evs):
        a.record()
        fn(base + i)
        b.record()
    torch.cuda.synchronize()
    per_step = [a.elapsed_time(b) * 1e-3 for a, b in pair_evs]
    return Timing(walls, evs, per_step, kernel)


def cpu_time(fn, budget_s, max_reps=200):
    """Seconds per evaluation of fn on the host: one warm-up, then repeats until budget_s has passed."""
    fn()
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or reps >= max_reps:
            return dt / reps, reps, dt


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

    tm = timed(step, steps, warmup)
    wall = tm.wall
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
        "metric": METRIC,
        "value": round(step_bytes / wall / 1e9, 1),
        "unit": "GB/s",
        "ms_per_step": wall * 1e3,
        "dtype": "f16",
        "config": {"workload": f"W4A16 decode GEMV M=1 N=11008 K=4096 group=128 fp16 scales+zeros, {units} weight set(s) per launch, "
                               f"{sets} sets rotating ({sets * unit_bytes >> 20} MiB); " + WALL_NOTE,
                   "M": M, "N": N, "K": K, "group": g, "units_per_launch": units},
        "roofline": dict({"bound": "hbm"}, **tm.roofline(step_bytes, HBM_PEAK_GBS, "GB/s", 1e9),
                         **(traffic_from_profile("gemv_w4a16_f16_M1_N11008_K4096_g128.txt") if units == 1 else {"traffic": None}),
                         bytes_per_launch=step_bytes),
        "cpu_baseline": cpu,
        "parity_rel_l2": rel,
    }


def cpu_baseline_gemv(A, Wp, S, Z, g, unit_bytes, budget_s=10.0):
    """The reference's CPU path for this workload: vectorised nibble unpack, (u - z) * s in fp16,
    fp32 matmul, cast (oracle.ref.ref_program_w4a16), timed on the host cores."""
    import torch

    from oracle import ref

    per, reps, dt = cpu_time(lambda: ref.ref_program_w4a16(A, Wp, S, Z, g, "float16"), budget_s)
    return {"value": round(unit_bytes / per / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{reps} evaluations of the same M=1 N=11008 K=4096 GEMV (unpack + dequant + fp32 matmul) in {dt:.1f} s",
            "ms_per_eval": round(per * 1e3, 2), "host_cpus": os.cpu_count()}


def bench_small(args, steps=None, cpu=True):
    """The reference's own CPU-runnable case: W4A16 dequant-GEMM M=N=K=256, fp16, group 128, zero point 8."""
    import torch

    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    dev = torch.device("cuda:0")
    M = N = K = 256
    g = 128
    gen = torch.Generator(device="cpu").manual_seed(6)
    Wp_c = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=gen)
    S_c = (torch.rand(N, K // g, generator=gen) * 0.015 + 0.005).to(torch.float16)
    A_c = torch.randn(M, K, generator=gen).to(torch.float16)
    Wp, S, A = Wp_c.to(dev), S_c.to(dev), A_c.to(dev)
    C = torch.empty(M, N, dtype=torch.float16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    ws_bytes = lib.tlq_w4a16_workspace_bytes(M, N, K)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    pre = (P(A), P(Wp), P(S), None, P(C), M, N, K, g, 8.0, _abi.F16, _abi.F16, _abi.ALGO_AUTO, P(ws), ws_bytes, stream)

    def step(i):
        if lib.tlq_gemm_w4a16_ws(*pre):
            raise RuntimeError(_abi.last_error())

    tm = timed(step, steps or args.steps, args.warmup)
    flops, nbytes = 2.0 * M * N * K, w4a16_bytes(M, N, K, g, zeros_tensor=False)
    out = {"workload": "W4A16 dequant-GEMM M=N=K=256 fp16 group=128 zero=8 (launch bound: 0.03 GFLOP, 0.3 MB)", "dtype": "f16",
           "value": round(flops / tm.wall / 1e12, 3), "unit": "TFLOP/s", "ms_per_step": tm.wall * 1e3,
           "roofline": dict({"bound": "hbm"}, **tm.roofline(nbytes, HBM_PEAK_GBS, "GB/s", 1e9), traffic=None, bytes_per_launch=nbytes)}
    if cpu:
        from oracle import ref

        def literal():  # the reference's own per-element unpack loop, then (u - 8) * s in fp16 and the fp32 matmul
            U = ref.unpack_uint4_loop(Wp_c, torch.float16)
            W = (U - 8) * S_c.repeat_interleave(g, dim=1)
            return (A_c.float() @ W.float().T).to(torch.float16)

        want = ref.ref_program_w4a16(A_c, Wp_c, S_c, 8, g, "float32")
        rel = ((C.float().cpu() - want).norm() / want.norm()).item()
        if rel > 1e-3:
            raise RuntimeError(f"M=N=K=256 result differs from the oracle: relative L2 {rel}")
        per, reps, dt = cpu_time(literal, 3.0, 20)
        out["cpu_baseline"] = {"value": round(flops / per / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
                               "sample": f"{reps} evaluations with the literal per-element unpack loop "
                                         f"(example_dequant_gemm_fine_grained.py:10-32) in {dt:.1f} s",
                               "ms_per_eval": round(per * 1e3, 2)}
    return out


def bench_prefill(args, steps=None, cpu=True):
    import torch

    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    dev = torch.device("cuda:0")
    M = N = K = 4096
    g = 128
    gen = torch.Generator(device="cpu").manual_seed(1)
    Wp_c = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=gen)
    S_c = (torch.rand(N, K // g, generator=gen) * 0.015 + 0.005).to(torch.bfloat16)
    A_c = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    Wp, S, A = Wp_c.to(dev), S_c.to(dev), A_c.to(dev)
    C = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    ws_bytes = lib.tlq_w4a16_workspace_bytes(M, N, K)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

    def step(i):  # what the library chooses with a workspace (the launch log of a step is in roofline.kernel)
        rc = lib.tlq_gemm_w4a16_ws(P(A), P(Wp), P(S), None, P(C), M, N, K, g, 8.0, _abi.BF16, _abi.BF16, _abi.ALGO_AUTO,
                                   P(ws), ws_bytes, stream)
        if rc:
            raise RuntimeError(_abi.last_error())

    def step_two(i):  # the reference's own structure, for comparison: dequantise into the workspace, then the plain GEMM
        rc = lib.tlq_gemm_w4a16_ws(P(A), P(Wp), P(S), None, P(C), M, N, K, g, 8.0, _abi.BF16, _abi.BF16, _abi.ALGO_TWO_PASS,
                                   P(ws), ws_bytes, stream)
        if rc:
            raise RuntimeError(_abi.last_error())

    def step_fused(i):  # the tile kernel that dequantises into LDS through registers, for comparison
        rc = lib.tlq_gemm_w4a16(P(A), P(Wp), P(S), None, P(C), M, N, K, g, 8.0, _abi.BF16, _abi.BF16, _abi.ALGO_MFMA, stream)
        if rc:
            raise RuntimeError(_abi.last_error())

    tm = timed(step, steps or args.steps, args.warmup)
    two = timed(step_two, steps or args.steps, min(args.warmup, 4), pairs=0, regions=9)
    fused = timed(step_fused, steps or args.steps, min(args.warmup, 4), pairs=0, regions=9)
    flops = 2.0 * M * N * K
    out = {"workload": "W4A16 prefill GEMM M=N=K=4096 bf16 group=128 zero=8, automatic choice with a caller-owned workspace "
                       "(the whole step is priced against the MFMA peak)", "dtype": "bf16",
           "value": round(flops / tm.wall / 1e12, 1), "unit": "TFLOP/s", "ms_per_step": tm.wall * 1e3,
           "roofline": dict({"bound": "mfma"}, **tm.roofline(flops, MFMA_F16_PEAK_TFLOPS, "TFLOP/s", 1e12),
                            **traffic_from_profile("panel_w4a16_bf16_M4096_N4096_K4096_g128.txt"), flops_per_launch=flops),
           "two_passes": {"path": two.kernel, "value": round(flops / two.wall / 1e12, 1), "unit": "TFLOP/s",
                          "us_per_step": round(two.ev * 1e6, 2), "frac_of_mfma_peak": round(flops / two.ev / 1e12 / MFMA_F16_PEAK_TFLOPS, 4)},
           "fused_kernel": {"path": fused.kernel, "value": round(flops / fused.wall / 1e12, 1), "unit": "TFLOP/s",
                            "us_per_step": round(fused.ev * 1e6, 2),
                            "frac_of_mfma_peak": round(flops / fused.ev / 1e12 / MFMA_F16_PEAK_TFLOPS, 4)}}
    if cpu:
        from oracle import ref

        per, reps, dt = cpu_time(lambda: ref.ref_program_w4a16(A_c, Wp_c, S_c, 8, g, "bfloat16"), 5.0, 20)
        out["cpu_baseline"] = {"value": round(flops / per / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"{reps} evaluations of the same 4096^3 problem (unpack + dequant in bf16 + fp32 matmul) in {dt:.1f} s",
                               "ms_per_eval": round(per * 1e3, 1)}
    return out


def bench_skinny(args, steps=None, cpu=True):
    """Decode batch of the MLP-shaped sweep: M=16 activations against a 14336 x 4096 weight matrix (HBM bound)."""
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

    tm = timed(step, steps or args.steps, args.warmup)
    out = {"workload": f"W4A16 decode batch M=16 N=14336 K=4096 group=128 fp16 scales+zeros, {sets} weight sets rotating",
           "dtype": "f16", "value": round(unit_bytes / tm.wall / 1e9, 1), "unit": "GB/s", "ms_per_step": tm.wall * 1e3,
           "roofline": dict({"bound": "hbm"}, **tm.roofline(unit_bytes, HBM_PEAK_GBS, "GB/s", 1e9),
                            **traffic_from_profile("decode_w4a16_f16_M16_N14336_K4096_g128.txt"), bytes_per_launch=unit_bytes)}
    if cpu:
        from oracle import ref

        a, w, sc, z = A.cpu(), Wp[0].cpu(), S[0].cpu(), Z[0].cpu()
        per, reps, dt = cpu_time(lambda: ref.ref_program_w4a16(a, w, sc, z, g, "float16"), 4.0, 50)
        out["cpu_baseline"] = {"value": round(unit_bytes / per / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"{reps} evaluations of the same M=16 problem (unpack + dequant + fp32 matmul) in {dt:.1f} s",
                               "ms_per_eval": round(per * 1e3, 1)}
    return out


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

    tm = timed(step, steps or args.steps, args.warmup)
    return {"workload": f"per-token int8 activation quantiser M=16384 N=4096 bf16 in, {sets} inputs rotating",
            "dtype": "f32", "value": round(unit_bytes / tm.wall / 1e9, 1), "unit": "GB/s", "ms_per_step": tm.wall * 1e3,
            "roofline": dict({"bound": "hbm"}, **tm.roofline(unit_bytes, HBM_PEAK_GBS, "GB/s", 1e9),
                             **traffic_from_profile("act_quant_bf16_M16384_N4096.txt"), bytes_per_launch=unit_bytes)}


def bench_vendor_gemm(args, steps=None):
    """The vendor library's GEMMs (torch.matmul / torch._int_mm, hipBLASLt underneath) beside this library's kernels on
    the same dense problems, alternating in one process (boxes and thermal states differ by several percent, so only
    figures from one process compare): the plain 16-bit GEMM core, the W4A16 path on the same shape (which reads a
    quarter of the weight bytes and dequantises on the way), and the int8 core.  Random operands.  A kernel trace of
    this command holds the vendor kernels' names and launch records (work-group size, LDS, registers)."""
    import torch

    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device=dev).manual_seed(11)
    steps = steps or min(args.steps, 10)
    rows = []

    def med(fns, rounds=5):  # alternating rounds; median us per launch for each callable
        acc = [[] for _ in fns]
        for r in range(rounds):
            for k, fn in enumerate(fns):
                fn(); fn()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(steps):
                    fn()
                e1.record()
                torch.cuda.synchronize()
                acc[k].append(e0.elapsed_time(e1) * 1e3 / steps)
        return [statistics.median(a) for a in acc]

    def check(rc):
        if rc:
            raise RuntimeError(_abi.last_error())

    g = 128
    for dt, code, peak in ((torch.bfloat16, _abi.BF16, MFMA_F16_PEAK_TFLOPS), (torch.float16, _abi.F16, MFMA_F16_PEAK_TFLOPS)):
        for (M, N, K) in ((4096, 4096, 4096), (8192, 8192, 8192), (8192, 14336, 4096)):
            A = torch.randn(M, K, dtype=dt, device=dev, generator=gen)
            W = (torch.randn(N, K, dtype=dt, device=dev, generator=gen) * 0.05)
            C = torch.empty(M, N, dtype=dt, device=dev)
            Wp = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, device=dev, generator=gen)
            S = (torch.rand(N, K // g, device=dev, generator=gen) * 0.015 + 0.005).to(dt)
            ws_bytes = lib.tlq_w4a16_workspace_bytes(M, N, K)
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
            fns = [lambda: torch.matmul(A, W.t(), out=C),
                   lambda: check(lib.tlq_gemm_f16(P(A), P(W), P(C), M, N, K, code, code, _abi.B_NK, stream)),
                   lambda: check(lib.tlq_gemm_w4a16_ws(P(A), P(Wp), P(S), None, P(C), M, N, K, g, 8.0, code, code, _abi.ALGO_AUTO, P(ws), ws_bytes, stream))]
            v, own, w4 = med(fns)
            flops = 2.0 * M * N * K
            rows.append({"problem": f"{str(dt)[6:]} M={M} N={N} K={K}, weights [N,K]", "vendor_us": round(v, 1), "gemm_f16_us": round(own, 1),
                         "w4a16_us": round(w4, 1), "vendor_frac_of_peak": round(flops / v / 1e6 / peak, 4),
                         "gemm_f16_frac_of_peak": round(flops / own / 1e6 / peak, 4), "w4a16_frac_of_peak": round(flops / w4 / 1e6 / peak, 4)})
            del A, W, C, Wp, S, ws
    for (M, N, K) in ((16384, 4096, 4096), (8192, 8192, 8192)):
        A = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=dev, generator=gen)
        B = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=dev, generator=gen)
        C = torch.empty(M, N, dtype=torch.int32, device=dev)
        fns = [lambda: torch._int_mm(A, B, out=C), lambda: check(lib.tlq_gemm_i8(P(A), P(B), P(C), 1, M, N, K, _abi.B_KN, stream))]
        v, own = med(fns)
        ops = 2.0 * M * N * K
        rows.append({"problem": f"int8 M={M} N={N} K={K}, weights [K,N]", "vendor_us": round(v, 1), "gemm_i8_us": round(own, 1),
                     "vendor_frac_of_peak": round(ops / v / 1e6 / MFMA_I8_PEAK_TOPS, 4), "gemm_i8_frac_of_peak": round(ops / own / 1e6 / MFMA_I8_PEAK_TOPS, 4)})
        del A, B, C
    first = rows[0]
    flops = 2.0 * 4096 ** 3
    return {"workload": "vendor library (hipBLASLt through torch.matmul / torch._int_mm) beside this library's GEMMs, alternating in one "
                        "process, random operands; value: this library's W4A16 path on bf16 4096^3",
            "dtype": "bf16", "value": round(flops / first["w4a16_us"] / 1e6, 1), "unit": "TFLOP/s", "ms_per_step": first["w4a16_us"] * 1e-3,
            "roofline": {"bound": "mfma", "achieved": round(flops / first["w4a16_us"] / 1e6, 1), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": first["w4a16_frac_of_peak"], "traffic": None},
            "shapes": rows}


def bench_mlp_sweep(args, steps=None):
    """MLP-shaped sweep: M in {16, 64, 256, 1024, 8192} x (N, K) in {(14336, 4096), (4096, 14336)} x group in {128, 64},
    fp16, per-group scales and zeros, automatic kernel choice with a workspace (tlq_gemm_w4a16_ws).  Inputs are drawn
    on the device (timing only; every shape is checked against the oracle by the GPU tests)."""
    import torch

    from tilelang_ascend_amd import _abi

    lib, P = _abi.load(), _abi.ptr
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    gen = torch.Generator(device=dev).manual_seed(5)
    for (N, K) in ((14336, 4096), (4096, 14336)):
        for g in (128, 64):
            sets = 6  # 6 x 29 MB of packed weights rotate: small-M launches always stream from HBM
            Wp = torch.randint(0, 256, (sets, N, K // 2), dtype=torch.uint8, generator=gen, device=dev)
            S = (torch.rand(sets, N, K // g, generator=gen, device=dev) * 0.015 + 0.005).to(torch.float16)
            Z = torch.randint(6, 10, (sets, N, K // g), generator=gen, device=dev).to(torch.float16)
            for M in (16, 64, 256, 1024, 8192):
                A = torch.randn(M, K, generator=gen, device=dev).to(torch.float16)
                C = torch.empty(M, N, dtype=torch.float16, device=dev)
                ws_bytes = lib.tlq_w4a16_workspace_bytes(M, N, K)
                ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
                pre = [(P(A), P(Wp[j]), P(S[j]), P(Z[j]), P(C), M, N, K, g, 0.0, _abi.F16, _abi.F16, _abi.ALGO_AUTO,
                        P(ws) if ws_bytes else None, ws_bytes, stream) for j in range(sets)]

                def step(i):
                    if lib.tlq_gemm_w4a16_ws(*pre[i % sets]):
                        raise RuntimeError(_abi.last_error())

                n = steps or (12 if M < 8192 else 4)
                tm = timed(step, n, 3, pairs=n, regions=7)
                ev = tm.ev
                flops, nbytes = 2.0 * M * N * K, w4a16_bytes(M, N, K, g)
                rows.append({"M": M, "N": N, "K": K, "group": g, "kernel": tm.kernel, "us": round(ev * 1e6, 1), "median_us": round(tm.median * 1e6, 1),
                             "min_us": round(tm.best * 1e6, 1),
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


def bench_w8a8(args, steps=None, cpu=True):
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

    tm = timed(step, steps or args.steps, args.warmup)
    ops = 2.0 * B * M * N * K
    out = {"workload": "W8A8 quant batch matmul B=8 M=2048 N=K=4096, per-token x per-channel rescale, fp16 out",
           "dtype": "i8", "value": round(ops / tm.wall / 1e12, 1), "unit": "TOP/s", "ms_per_step": tm.wall * 1e3,
           "roofline": dict({"bound": "mfma"}, **tm.roofline(ops, MFMA_I8_PEAK_TOPS, "TOP/s", 1e12),
                            **traffic_from_profile("gemm_w8a8_B8_M2048_N4096_K4096.txt"), ops_per_launch=ops)}
    if cpu:
        from oracle import ref

        a, w, s_a, s_b = A[0].cpu(), W[0].cpu().T.contiguous(), sa[0].cpu(), sb.cpu()
        per, reps, dt = cpu_time(lambda: ref.ref_int8_gemm_sequential(a, w, s_a, s_b, torch.float16), 4.0, 10)
        out["cpu_baseline"] = {"value": round(ops / B / per / 1e12, 4), "unit": "TOP/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"{reps} evaluations of ONE of the 8 batch elements (exact integer matmul through float64, "
                                         f"two fp32 rescales) in {dt:.1f} s; the whole batch takes 8 x ms_per_eval",
                               "ms_per_eval": round(per * 1e3, 1)}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=480)
    ap.add_argument("--warmup", type=int, default=48)
    ap.add_argument("--workload", default="gemv", choices=["gemv", "small", "prefill", "w8a8", "skinny", "actquant", "mlp-sweep", "vendor-gemm"])
    ap.add_argument("--units", type=int, default=1, help="independent weight sets per GEMV launch")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-side baseline (profiling runs)")
    ap.add_argument("--tune", action="append", default=[], metavar="HOOK=VALUE",
                    help="call a single-integer tuning hook of the library before measuring, e.g. --tune gemm_slots=0 "
                         "(tlq_tune_gemm_slots(0): the two-stage main loop instead of the five-slot one); repeatable; "
                         "recorded in the output line")
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
            cpu = not args.no_cpu_baseline
            for name, fn in (("gemv, 24 weight sets per launch", many_sets),
                             ("small", lambda: bench_small(args, steps=100, cpu=cpu)),
                             ("skinny", lambda: bench_skinny(args, steps=60, cpu=cpu)),
                             ("prefill", lambda: bench_prefill(args, steps=20, cpu=cpu)),
                             ("w8a8", lambda: bench_w8a8(args, steps=10, cpu=cpu)),
                             ("actquant", lambda: bench_act_quant(args, steps=40)),
                             ("mlp-sweep", lambda: bench_mlp_sweep(args))):
                try:
                    others.append(fn())
                except Exception as e:  # noqa: BLE001
                    others.append({"workload": name, "error": f"{type(e).__name__}: {e}"})
            line["other_workloads"] = others
    else:
        cpu = not args.no_cpu_baseline
        res = {"prefill": lambda a: bench_prefill(a, cpu=cpu), "w8a8": lambda a: bench_w8a8(a, cpu=cpu),
               "skinny": lambda a: bench_skinny(a, cpu=cpu), "small": lambda a: bench_small(a, cpu=cpu),
               "actquant": bench_act_quant, "mlp-sweep": bench_mlp_sweep, "vendor-gemm": bench_vendor_gemm}[args.workload](args)
        line = {"metric": METRIC, "value": res["value"], "unit": res["unit"], "ms_per_step": res["ms_per_step"], "dtype": res["dtype"],
                "config": {"workload": res["workload"] + ("; every figure from HIP events" if args.workload in ("mlp-sweep", "vendor-gemm") else "; " + WALL_NOTE)}, "roofline": res["roofline"],
                "cpu_baseline": res.get("cpu_baseline")}
        for extra in ("shapes", "fused_kernel", "two_passes"):
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
