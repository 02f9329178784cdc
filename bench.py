#!/usr/bin/env python3
"""Benchmark of the operator hot path on one MI355X.

``python bench.py [--gpus 1] [--steps K] [--warmup W]`` prints ONE JSON line.

Workload (BASELINE.json configs): the bf16 GEMM (M=N=K=2048), the decode GEMV
sweep and the Llama-3.2-1B-shape decode step.  A "step" is one pass over the
workload's timed unit.  Inputs are synthetic (seeded numpy draws, bf16) and
resident in HBM before the timed region.  Kernels are timed with HIP events on
the stream they are launched on, as replays of a HIP graph holding many launches
over rotating buffers (more than the 256 MB last-level cache), so the figures are
HBM figures and launch overhead from Python is not in them.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published

GEMV_SWEEP = [(2048, 2048), (2048, 512), (2048, 8192), (8192, 2048), (2048, 128256)]  # K -> N


def graph_time_us(torch, launches, replays):
    """Average microseconds per launch: `launches` (callables) captured once in a HIP graph."""
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        for fn in launches[: min(3, len(launches))]:
            fn()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for fn in launches:
                fn()
        graph.replay()
        stream.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(replays):
            graph.replay()
        stop.record(stream)
        stop.synchronize()
    return start.elapsed_time(stop) * 1e3 / (replays * len(launches))


def bench_gemv(torch, K, dev, Kdim, N, steps, rng):
    """One decode GEMV shape over a pool of distinct weights larger than the last-level cache."""
    from iron_amd.bf16 import round_bf16, to_torch

    bytes_w = N * Kdim * 2
    copies = max(2, min(64, int(np.ceil(640e6 / bytes_w))))
    base = to_torch(round_bf16(rng.standard_normal((N, Kdim), dtype=np.float32) * np.float32(0.02))).to(dev)
    pool = [base] + [base.clone() for _ in range(copies - 1)]
    x = to_torch(round_bf16(rng.standard_normal(Kdim, dtype=np.float32))).to(dev)
    y = torch.empty(N, dtype=torch.bfloat16, device=dev)
    launches = [(lambda W=W: K.gemv(W, x, y, M=N, K=Kdim)) for W in pool]
    reps = max(1, steps // len(launches))
    us = graph_time_us(torch, launches, reps)
    algo = 2 * (N * Kdim + Kdim + N)
    return {"K": Kdim, "N": N, "us": round(us, 3), "GBps": round(algo / us / 1e3, 1),
            "frac_hbm": round(algo / us / 1e3 / HBM_PEAK_GBS, 4), "bytes": algo, "copies": copies}


def bench_gemm(torch, K, dev, steps, rng, b_col_maj):
    from iron_amd.bf16 import round_bf16, to_torch

    M = N = Kd = 2048
    A = to_torch(round_bf16(rng.standard_normal((M, Kd), dtype=np.float32) * np.float32(0.02))).to(dev)
    B = to_torch(round_bf16(rng.standard_normal((Kd, N), dtype=np.float32) * np.float32(0.02))).to(dev)
    C = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    launches = [lambda: K.gemm(A, B, C, M=M, N=N, K=Kd, b_col_maj=b_col_maj)] * 20
    us = graph_time_us(torch, launches, max(1, steps // 20))
    flops = 2.0 * M * N * Kd
    return {"M": M, "N": N, "K": Kd, "b_col_maj": b_col_maj, "us": round(us, 3),
            "TFLOPs": round(flops / us / 1e6, 1), "frac_mfma": round(flops / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}


def cpu_gemv_baseline(rng, budget_s=12.0):
    """The oracle's GEMV (the reference's CPU path: the weight up-cast to f32 on every call,
    gemv.py:413) timed on the host cores on a bounded sample of the sweep."""
    import torch as _t

    from iron_amd.bf16 import from_bits, round_bf16, to_bits
    from oracle import ops

    sample = [(2048, 2048), (2048, 8192), (8192, 2048)]
    total_bytes, total_s, calls = 0, 0.0, 0
    for Kdim, N in sample:
        # The weight is held as bf16 storage and widened on every call, as the reference's
        # `A.astype(np.float32)` does.
        W = to_bits(rng.standard_normal((N, Kdim), dtype=np.float32) * np.float32(0.02))
        x = round_bf16(rng.standard_normal(Kdim, dtype=np.float32))
        ops.gemv(from_bits(W), x)
        t0 = time.perf_counter()
        n = 0
        while time.perf_counter() - t0 < budget_s / len(sample):
            ops.gemv(from_bits(W), x)
            n += 1
        dt = time.perf_counter() - t0
        total_bytes += n * 2 * (N * Kdim + Kdim + N)
        total_s += dt
        calls += n
    return {"value": round(total_bytes / total_s / 1e9, 2), "unit": "GB/s", "cores": _t.get_num_threads(),
            "kind": "port", "sample": f"{calls} oracle GEMV calls over K->N {sample}, {total_s:.1f} s wall"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build is a one-GPU hot path; --gpus must be 1 "
              "(sharding is described in DESIGN.md, not built)", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    from iron_amd import kernels as K
    from iron_amd._lib import lib

    lib()  # raises if the HIP library is missing: nothing here runs without it
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    rng = np.random.default_rng(2025)

    # Warm-up: every kernel once, untimed.
    for _ in range(max(1, args.warmup // 10)):
        w = torch.zeros((512, 2048), dtype=torch.bfloat16, device=dev)
        xx = torch.zeros(2048, dtype=torch.bfloat16, device=dev)
        yy = torch.empty(512, dtype=torch.bfloat16, device=dev)
        K.gemv(w, xx, yy, M=512, K=2048)
    torch.cuda.synchronize()

    t_wall = time.perf_counter()
    gemv = [bench_gemv(torch, K, dev, Kd, N, args.steps, rng) for Kd, N in GEMV_SWEEP]
    gemm = [bench_gemm(torch, K, dev, args.steps, rng, b) for b in (False, True)]
    torch.cuda.synchronize()
    wall = time.perf_counter() - t_wall

    sweep_bytes = sum(g["bytes"] for g in gemv)
    sweep_us = sum(g["us"] for g in gemv)
    head = gemv[-1]
    out = {
        "metric": "bf16 GEMM TFLOP/s, GEMV GB/s (% roofline); Llama-3.2-1B-shape decode tok/s",
        "value": round(sweep_bytes / sweep_us / 1e3, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(sweep_us / 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "decode GEMV sweep K->N 2048->2048, 2048->512, 2048->8192, 8192->2048, "
                               "2048->128256 (batch 1, bf16, f32 accumulation); one step = the five GEMVs"},
        "roofline": {"bound": "hbm", "kernel": "gemv_kernel (2048->128256 LM head)",
                     "achieved": head["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": head["frac_hbm"], "traffic": None},
        "gemv": gemv,
        "gemm": gemm,
        "bench_wall_s": round(wall, 1),
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_gemv_baseline(np.random.default_rng(7))
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
