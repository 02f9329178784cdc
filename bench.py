#!/usr/bin/env python3
"""Benchmark of the operator hot path on one MI355X.

``python bench.py [--gpus 1] [--steps K] [--warmup W]`` prints ONE JSON line.

Workload: the reference's benchmark configurations -- the bf16 GEMM (M=N=K=2048), the decode GEMV
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


def verified(torch, what, got, want, rtol=1e-2, atol=1e-2):
    """The timed kernel's own output against a float32 evaluation of the same product on the same
    operands (torch on the GPU, over the rows sampled): the bar of the parity tests, |diff| <= atol +
    rtol |want|.  Raises if it fails, so a number in the line is a number of a checked result."""
    got, want = got.float(), want.float()
    excess = ((got - want).abs() - (atol + rtol * want.abs())).max().item()
    if not excess <= 0.0:
        raise AssertionError(f"bench self-check failed: {what}: |diff| exceeds {atol} + {rtol}|want| by {excess:.4g}")
    return int(got.numel())


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
    rows = torch.from_numpy(rng.choice(N, size=min(N, 4096), replace=False)).to(dev)
    checked = verified(torch, f"gemv {Kdim}->{N}", y[rows], pool[-1][rows].float() @ x.float())
    algo = 2 * (N * Kdim + Kdim + N)
    return {"K": Kdim, "N": N, "us": round(us, 3), "GBps": round(algo / us / 1e3, 1),
            "frac_hbm": round(algo / us / 1e3 / HBM_PEAK_GBS, 4), "bytes": algo, "copies": copies,
            "checked_outputs": checked}


def bench_gemm(torch, K, dev, steps, rng, b_col_maj, M=2048, N=2048, Kd=2048):
    from iron_amd.bf16 import round_bf16, to_torch

    A = to_torch(round_bf16(rng.standard_normal((M, Kd), dtype=np.float32) * np.float32(0.02))).to(dev)
    B = to_torch(round_bf16(rng.standard_normal((N, Kd) if b_col_maj else (Kd, N), dtype=np.float32)
                            * np.float32(0.02))).to(dev)
    C = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    launches = [lambda: K.gemm(A, B, C, M=M, N=N, K=Kd, b_col_maj=b_col_maj)] * 20
    us = graph_time_us(torch, launches, max(1, steps // 20))
    rows = torch.from_numpy(np.sort(rng.choice(M, size=64, replace=False))).to(dev)
    Bf = B.float()
    checked = verified(torch, f"gemm {M}x{N}x{Kd}", C[rows], A[rows].float() @ (Bf.t() if b_col_maj else Bf))
    flops = 2.0 * M * N * Kd
    return {"M": M, "N": N, "K": Kd, "b_col_maj": b_col_maj, "us": round(us, 3),
            "TFLOPs": round(flops / us / 1e6, 1), "frac_mfma": round(flops / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
            "checked_outputs": checked}


def bench_library_reference(torch, dev, n, rng):
    """The vendor libraries on the same shapes and data, for scale (not this build's path, and
    nothing here is compared for parity): ``torch.matmul`` (hipBLASLt / rocBLAS) on the GEMM shapes
    with B as (N, K), and ``scaled_dot_product_attention`` on the prefill shapes."""
    import torch.nn.functional as F

    out = {"what": "torch.matmul and torch SDPA (vendor libraries), same shapes and data; for scale only",
           "gemm_b_col_maj": [], "attention_prefill": []}
    for M, N, Kd in ((2048, 2048, 2048), (2048, 8192, 2048), (4096, 4096, 4096), (8192, 8192, 8192)):
        A = (torch.randn(M, Kd, device=dev) * 0.02).bfloat16()
        B = (torch.randn(N, Kd, device=dev) * 0.02).bfloat16()
        C = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
        us = graph_time_us(torch, [lambda: torch.matmul(A, B.t(), out=C)] * 10, max(1, n // 40))
        out["gemm_b_col_maj"].append({"M": M, "N": N, "K": Kd, "us": round(us, 2),
                                      "TFLOPs": round(2.0 * M * N * Kd / us / 1e6, 1)})
    for S in (512, 2048, 8192):
        q = torch.randn(1, 32, S, 64, device=dev).bfloat16()
        k, v = (torch.randn(1, 8, S, 64, device=dev).bfloat16() for _ in range(2))
        try:
            us = graph_time_us(torch, [lambda: F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)] * 5,
                               max(1, n // 40))
            out["attention_prefill"].append({"S": S, "us": round(us, 2),
                                             "TFLOPs": round(4.0 * 32 * 64 * S * (S + 1) / 2 / us / 1e6, 1)})
        except Exception as e:  # a library without this shape is no failure of the bench
            out["attention_prefill"].append({"S": S, "error": str(e)[:80]})
    return out


def bench_decode_kernels(torch, K, dev, n, rng):
    """Each kernel the captured decode step of the Llama-3.2-1B shape launches, alone at its own shape:
    a replayed HIP graph of back-to-back launches over distinct weights (more than the last-level
    cache holds), timed with HIP events on the graph's stream.  ``per_step`` is how often a decode
    step launches it; ``bytes`` the algorithmic bytes of one launch (its weights, vectors and cache
    rows), ``frac_hbm`` those over the duration against the published HBM peak."""
    E, F, H, G, D, V, L, pos = 2048, 8192, 32, 8, 64, 128256, 2048, 576

    def drawn(*shape, scale=0.02):
        return (torch.randn(*shape, device=dev) * scale).to(torch.bfloat16)

    def pool(bytes_each, make):
        return [make() for _ in range(max(2, min(96, int(np.ceil(640e6 / bytes_each)))))]

    x, gain = drawn(E, scale=1.0), (torch.rand(E, device=dev) * 0.2 + 0.9).to(torch.bfloat16)
    position = torch.tensor([pos], dtype=torch.int32, device=dev)
    kv_valid = torch.tensor([pos + 1], dtype=torch.int32, device=dev)
    angles = drawn(D, scale=1.0)
    q, y, m = torch.empty(H * D, dtype=torch.bfloat16, device=dev), torch.empty(E, dtype=torch.bfloat16, device=dev), \
        drawn(F, scale=1.0)
    rows = []

    def add(name, kernel, per_step, nbytes, launches):
        us = graph_time_us(torch, launches, max(1, n // len(launches)))
        rows.append({"name": name, "kernel": kernel, "per_step": per_step, "bytes": int(nbytes), "us": round(us, 3),
                     "GBps": round(nbytes / us / 1e3, 1), "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)})

    # attention's first half: norm, q/k/v projections, RoPE, the cache rows
    qkv_bytes = 2 * ((H + 2 * G) * D * E + 2 * E + (H + 2 * G) * D)
    caches = pool(2 * L * G * D * 2, lambda: (drawn(L, G, D, scale=1.0), drawn(L, G, D, scale=1.0)))
    ws = pool(qkv_bytes, lambda: (drawn(H * D, E), drawn(G * D, E), drawn(G * D, E)))
    add("norm + q/k/v + RoPE + cache write", "decode_qkv_kernel<64,1,false,2>", 16, qkv_bytes,
        [(lambda w=w, c=caches[i % len(caches)]: K.decode_qkv(x, gain, w[0], w[1], w[2], angles, q, c[0], c[1], eps=1e-5,
                                                               hidden=E, heads=H, kv_heads=G, d=D, cache_rows=L,
                                                               position=position)) for i, w in enumerate(ws)])
    del ws
    # attention over the cache (one query, pos + 1 keys)
    att_bytes = 2 * (pos + 1) * G * D * 2 + 2 * H * D * 2
    wsp = K.mha_decode_workspace(H, D, dev)
    o = torch.empty(1, H, D, dtype=torch.bfloat16, device=dev)
    add(f"attention, one query over {pos + 1} keys", "mha_decode_single_kernel<64>", 16, att_bytes,
        [(lambda c=c: K.mha_decode(q.reshape(1, H, D), c[0], c[1], o, heads=H, kv_heads=G, d=D, kv_len=L, scale=0.125,
                                   kv_interleaved=True, kv_valid=kv_valid, workspace=wsp)) for c in caches])
    del caches
    # o projection + residual
    ws = pool(2 * E * H * D, lambda: drawn(E, H * D))
    add("o projection + residual", "gemv_fused_kernel<1,1,false,1>", 16, 2 * (E * H * D + H * D + 2 * E),
        [(lambda w=w: K.gemv_fused(w, q, y, M=E, K=H * D, residual=x, epilogue=1)) for w in ws])
    del ws
    # norm + gate/up + SiLU * mul
    ws = pool(4 * F * E, lambda: (drawn(F, E), drawn(F, E)))
    mm = torch.empty(F, dtype=torch.bfloat16, device=dev)
    add("norm + gate/up + SiLU*mul", "gemv_fused_kernel<2,1,true,2>", 16, 2 * (2 * F * E + 2 * E + F),
        [(lambda w=w: K.gemv_fused(w[0], x, mm, M=F, K=E, W2=w[1], norm_w=gain, eps=1e-5, epilogue=2)) for w in ws])
    del ws
    # down projection + residual
    ws = pool(2 * E * F, lambda: drawn(E, F))
    add("down projection + residual", "gemv_fused_kernel<2,4,false,1>", 16, 2 * (E * F + F + 2 * E),
        [(lambda w=w: K.gemv_fused(w, m, y, M=E, K=F, residual=x, epilogue=1)) for w in ws])
    del ws
    # final norm + head
    ws = pool(2 * V * E, lambda: drawn(V, E))
    logits = torch.empty(V, dtype=torch.bfloat16, device=dev)
    add("final norm + LM head", "gemv_fused_kernel<4,1,true,0>", 1, 2 * (V * E + 2 * E + V),
        [(lambda w=w: K.gemv_fused(w, x, logits, M=V, K=E, norm_w=gain, eps=1e-5, epilogue=0)) for w in ws])
    del ws
    torch.cuda.empty_cache()
    total = sum(r["per_step"] * r["us"] for r in rows)
    for r in rows:
        r["share_of_listed_us"] = round(r["per_step"] * r["us"] / total, 4)
    return rows


def bench_attention(torch, K, dev, n, rng):
    """GQA causal attention, 32 q / 8 kv heads, d 64, scale 1/8: prefill at S = 512, 2048, 8192 (MFMA bound)
    and one query over caches of 1024, 4096, 16384 keys (HBM bound); beside them prefill at S = 2048 with
    256- and 512-wide heads."""
    H, G, D = 32, 8, 64
    out = {"prefill": [], "decode": []}

    def rand(*shape):
        return torch.randn(shape, device=dev, dtype=torch.float32).to(torch.bfloat16)

    def attend(q, keys, values):
        """One query row of every head over `keys` / `values` (rows, G, D) in float32: (H, D)."""
        qf = q.float().reshape(G, H // G, D)
        scores = torch.einsum("ghd,lgd->ghl", qf, keys.float()) * 0.125
        return torch.einsum("ghl,lgd->ghd", torch.softmax(scores, dim=-1), values.float()).reshape(H, D)

    for S in (512, 2048, 8192):
        Q, Kc, Vc = rand(S, H, D), rand(S, G, D), rand(S, G, D)
        O = torch.empty_like(Q)
        launches = [lambda: K.mha_prefill(Q, Kc, Vc, O, heads=H, kv_heads=G, d=D, seq=S, kv_len=S, scale=0.125,
                                          q_interleaved=True, kv_interleaved=True)] * 10
        us = graph_time_us(torch, launches, max(1, n // (10 * max(1, S // 512))))
        checked = 0
        for i in sorted({0, 63, 64, S // 2 - 1, S - 129, S - 1}):   # query rows, every head: keys 0..i
            checked += verified(torch, f"prefill attention S={S} row {i}", O[i], attend(Q[i], Kc[: i + 1], Vc[: i + 1]))
        flops = 4.0 * H * D * S * (S + 1) / 2
        out["prefill"].append({"S": S, "us": round(us, 2), "TFLOPs": round(flops / us / 1e6, 1),
                               "frac_mfma": round(flops / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
                               "checked_outputs": checked})
    # Wider heads (not a BASELINE configuration; Gemma's 256- and 512-wide ones), unscaled, S = 2048.
    out["prefill_wide_heads"] = []
    for Dw in (256, 512):
        S = 2048
        Q, Kc, Vc = rand(S, H, Dw) * 0.25, rand(S, G, Dw) * 0.25, rand(S, G, Dw)
        O = torch.empty_like(Q)
        launches = [lambda: K.mha_prefill(Q, Kc, Vc, O, heads=H, kv_heads=G, d=Dw, seq=S, kv_len=S, scale=1.0,
                                          q_interleaved=True, kv_interleaved=True)] * 4
        us = graph_time_us(torch, launches, max(1, n // 40))
        checked = 0
        for i in sorted({0, 15, 16, 127, 128, S // 2 - 1, S - 1}):
            qf = Q[i].float().reshape(G, H // G, Dw)
            scores = torch.einsum("ghd,lgd->ghl", qf, Kc[: i + 1].float())
            want = torch.einsum("ghl,lgd->ghd", torch.softmax(scores, dim=-1), Vc[: i + 1].float()).reshape(H, Dw)
            checked += verified(torch, f"prefill attention d={Dw} row {i}", O[i], want)
        flops = 4.0 * H * Dw * S * (S + 1) / 2
        out["prefill_wide_heads"].append({"d": Dw, "S": S, "us": round(us, 2), "TFLOPs": round(flops / us / 1e6, 1),
                                          "frac_mfma": round(flops / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
                                          "checked_outputs": checked})
    for L in (1024, 4096, 16384):
        copies = max(2, min(64, int(np.ceil(400e6 / (L * G * D * 4)))))
        Q = rand(1, H, D)
        Ks, Vs = [rand(L, G, D) for _ in range(copies)], [rand(L, G, D) for _ in range(copies)]
        O = torch.empty_like(Q)
        ws = K.mha_decode_workspace(H, D, dev)
        launches = [(lambda a=a, b=b: K.mha_decode(Q, a, b, O, heads=H, kv_heads=G, d=D, kv_len=L, scale=0.125,
                                                   kv_interleaved=True, workspace=ws)) for a, b in zip(Ks, Vs)]
        us = graph_time_us(torch, launches, max(1, n // len(launches)))
        checked = verified(torch, f"decode attention L={L}", O[0], attend(Q[0], Ks[-1], Vs[-1]))
        algo = 2 * L * G * D * 2 + 2 * H * D * 2
        out["decode"].append({"L": L, "us": round(us, 2), "GBps": round(algo / us / 1e3, 1),
                              "frac_hbm": round(algo / us / 1e3 / HBM_PEAK_GBS, 4), "bytes": algo,
                              "checked_outputs": checked})
    return out


def bench_sample(torch, K, dev, n, rng):
    """The draw over 128256 logits N(0, 3): greedy (an all-zero draw row) and at temperature 0.7 over the
    top 50; a latency, launched back to back in a replayed graph."""
    from iron_amd.bf16 import round_bf16, to_torch
    from iron_amd.operators.sample import draw_row

    vocab = 128256
    logits = to_torch(round_bf16(rng.normal(0, 3, vocab).astype(np.float32))).to(dev)
    token = torch.zeros(1, dtype=torch.int32, device=dev)
    ws = K.sample_workspace(vocab, dev)
    out = {"vocab": vocab}
    for name, (t, k) in (("greedy_us", (0.0, 1)), ("top50_t0.7_us", (0.7, 50))):
        row = torch.from_numpy(np.ascontiguousarray(draw_row(t, k, 1234567890123))).to(dev)
        launches = [lambda row=row: K.sample(logits, row, token, workspace=ws)] * 20
        out[name] = round(graph_time_us(torch, launches, max(1, n // 20)), 2)
        drawn = int(token.item())
        if k == 1 and drawn != int(torch.argmax(logits.float()).item()):
            raise AssertionError(f"bench self-check failed: the greedy draw {drawn} is not the largest logit's index")
        if not 0 <= drawn < vocab or logits[drawn].float() < torch.topk(logits.float(), k).values[-1]:
            raise AssertionError(f"bench self-check failed: the draw {drawn} is not among the top {k}")
    out["checked"] = "greedy = argmax; the sampled token among the top k"
    return out


def bench_pre_attention(torch, K, dev, n):
    """The pre-attention block at sequence 2048, hidden 2048: RMSNorm, the Q/K/V projections (32 q / 8 kv heads,
    d 64) and RoPE on q and k, as the prompt chunk runs them (five operator steps)."""
    S, E, H, G, D = 2048, 2048, 32, 8, 64

    def rand(*shape, scale=1.0):
        return (torch.randn(shape, device=dev, dtype=torch.float32) * scale).to(torch.bfloat16)

    x, gain = rand(S, E), (torch.rand(E, device=dev) * 0.2 + 0.9).to(torch.bfloat16)
    Wq, Wk, Wv = rand(H * D, E, scale=0.02), rand(G * D, E, scale=0.02), rand(G * D, E, scale=0.02)
    theta = torch.rand(S, D // 2, device=dev) * 6.28
    ang = torch.stack([torch.cos(theta), torch.sin(theta)], dim=-1).reshape(S, D).to(torch.bfloat16)
    n_, q, k, v = torch.empty_like(x), rand(S, H * D), rand(S, G * D), rand(S, G * D)
    qr, kr = torch.empty_like(q), torch.empty_like(k)

    def block():
        K.rmsnorm(x, gain, n_, rows=S, cols=E, eps=1e-5)
        K.gemm(n_, Wq, q, M=S, N=H * D, K=E, b_col_maj=True)
        K.gemm(n_, Wk, k, M=S, N=G * D, K=E, b_col_maj=True)
        K.gemm(n_, Wv, v, M=S, N=G * D, K=E, b_col_maj=True)
        K.rope(q, ang, qr, rows=S * H, cols=D, angle_rows=S)
        K.rope(k, ang, kr, rows=S * G, cols=D, angle_rows=S)

    def fused():
        K.rmsnorm(x, gain, n_, rows=S, cols=E, eps=1e-5)
        K.prefill_qkv(n_, Wq, Wk, Wv, ang, qr, kr, v, rows=S, hidden=E, heads=H, kv_heads=G, d=D)

    us = graph_time_us(torch, [block] * 4, max(1, n // 8))
    stepwise = [t.clone() for t in (qr, kr, v)]
    us_fused = graph_time_us(torch, [fused] * 4, max(1, n // 8))
    checked = sum(verified(torch, f"fused projections, output {i}", got, want)
                  for i, (got, want) in enumerate(zip((qr, kr, v), stepwise)))
    flops = 2.0 * S * E * (H + 2 * G) * D
    return {"us": round(us_fused, 2), "TFLOPs": round(flops / us_fused / 1e6, 1), "kernels": 2,
            "note": "RMSNorm, then one launch for the three projections with RoPE in its epilogue "
                    "(what the compiled prompt chunk runs)",
            "unfused": {"us": round(us, 2), "TFLOPs": round(flops / us / 1e6, 1), "kernels": 6},
            "checked_outputs": checked,
            "bytes_unfused": 71_600_000, "bytes_fused_min": 33_600_000}


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


def llama_weights(torch, config, dev, seed=0):
    """Random-init weights of ``config``'s shape on the GPU: matrices N(0, 0.02), norm gains 1, bf16."""
    from iron_amd.applications.llama import shapes

    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    out = {}
    for name, shape in shapes(config).items():
        if len(shape) >= 2:
            w = torch.randn(shape, generator=g, device=dev, dtype=torch.float32).mul_(0.02)
            out[name] = w.to(torch.bfloat16)
            del w
        else:
            out[name] = torch.ones(shape, device=dev, dtype=torch.bfloat16)
    return out


def prompt_probe(torch, dev, repeats=20):
    """Only the decoder's 512-token prompt chunk, ``repeats`` times: what a kernel trace of the time
    to the first token needs (the bench's own run buries its one chunk under the micro-benchmarks)."""
    import dataclasses

    from iron_amd.applications.llama import LLAMA_3_2_1B, Llama

    config = dataclasses.replace(LLAMA_3_2_1B, max_seq_len=2048, prefill_chunk=2048)
    model = Llama(config, llama_weights(torch, config, dev))
    model.load_versions()
    prompt = np.random.default_rng(512).integers(0, config.vocab_size, 512)
    times = []
    for _ in range(repeats):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for inputs, values in model.session.chunk_calls(prompt, 0):
            model(*inputs, **values)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    print(json.dumps({"probe": "prompt", "prefill_tokens": 512, "repeats": repeats,
                      "launches_per_chunk": model.prompt_chunk.launches_per_call,
                      "ttft_ms_median": round(1e3 * float(np.median(times)), 3)}))


def bench_decoder_contexts(torch, dev, steps, warmup, weights, contexts=(8192, 131072)):
    """The same 512-token prompt + ``steps`` decode steps with the caches compiled for longer contexts
    (131072 is Llama-3.2-1B's own max_seq_len): what a token costs is to follow the context, not the
    cache (the reference's "one compile, any context", AGENTS.md:246-255)."""
    import dataclasses

    from iron_amd.applications.llama import LLAMA_3_2_1B, Llama

    out = []
    prompt = np.random.default_rng(512).integers(0, LLAMA_3_2_1B.vocab_size, 512)
    for rows in contexts:
        config = dataclasses.replace(LLAMA_3_2_1B, max_seq_len=rows, prefill_chunk=2048)
        model = Llama(config, weights)
        model.load_versions()
        decode = model.decode_step

        def prefill():
            carry = None
            for inputs, values in model.session.chunk_calls(prompt, 0):
                _, carry = model(*inputs, **values)
            return carry

        decode.start(**prefill())
        decode.replay(max(warmup, 1))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        carry = prefill()
        torch.cuda.synchronize()
        ttft = time.perf_counter() - t0
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        decode.start(**carry)
        decode.replay(steps - 1)
        stop.record()
        stop.synchronize()
        ms = start.elapsed_time(stop)
        tokens = decode.read(model.drawn)[512 : 512 + steps]
        out.append({"max_seq_len": rows, "tok_s": round(steps / (ms / 1e3), 1), "ms_per_token": round(ms / steps, 4),
                    "ttft_ms": round(ttft * 1e3, 2), "launches_per_step": decode.launches_per_replay,
                    "first_tokens": [int(t) for t in tokens[:4]]})
        model.release()
        del model
        torch.cuda.empty_cache()
    return out


def bench_decoder(torch, dev, steps, warmup, with_cpu, probe_steps=0):
    """Llama-3.2-1B shape: a 512-token prompt prefill, then ``steps`` greedy decode steps as
    replays of the captured decode step (each starts from the token and position the last one
    carried on the device)."""
    import dataclasses

    from iron_amd.applications.llama import LLAMA_3_2_1B, Llama

    config = dataclasses.replace(LLAMA_3_2_1B, max_seq_len=2048, prefill_chunk=2048)
    weights = llama_weights(torch, config, dev)
    model = Llama(config, weights)
    model.load_versions()
    prompt = np.random.default_rng(512).integers(0, config.vocab_size, 512)
    session, decode = model.session, model.decode_step

    def prefill():
        carry = None
        for inputs, values in session.chunk_calls(prompt, 0):
            logits, carry = model(*inputs, **values)
        prefill.last = logits
        return carry

    carry = prefill()
    # A copy now: the decode steps write their logits where the prompt's were.
    prompt_logits = np.array(prefill.last.numpy()).reshape(-1)[: config.vocab_size]
    decode.start(**carry)
    decode.replay(max(warmup, 1))
    torch.cuda.synchronize()
    if probe_steps:   # a decode-only run for a kernel trace or a counter run: nothing else is launched after this
        carry = prefill()
        decode.start(**carry)
        decode.replay(probe_steps - 1)
        torch.cuda.synchronize()
        # ... and a plain copy of known size, which turns a counter run's FETCH_SIZE / WRITE_SIZE into bytes
        from iron_amd import kernels as K

        rows = PROBE_COPY_BYTES // 4096
        src = torch.zeros(PROBE_COPY_BYTES // 4, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(2):
            K.copy_rows(src, dst, rows=rows, row_elems=1024, src_rows=rows, dst_rows=rows)
        torch.cuda.synchronize()
        print(json.dumps({"probe": "decode", "prefill_tokens": 512, "decode_steps": probe_steps,
                          "launches_per_step": decode.launches_per_replay,
                          "copy": {"launches": 2, "bytes_read": PROBE_COPY_BYTES, "bytes_written": PROBE_COPY_BYTES}}))
        model.release()
        return None, None

    # The time to the first token: the median of five prefills of the same prompt (host clock around a
    # call and its synchronization; one sample moves by a tenth with the host's scheduling).
    ttfts = []
    for _ in range(5):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        carry = prefill()
        torch.cuda.synchronize()
        ttfts.append(time.perf_counter() - t0)
    ttft = float(np.median(ttfts))

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    decode.start(**carry)
    decode.replay(steps - 1)
    stop.record()
    stop.synchronize()
    wall = time.perf_counter() - t0
    ms = start.elapsed_time(stop)
    tokens = decode.read(model.drawn)[512 : 512 + steps]
    weight_bytes = 2 * (sum(int(np.prod(s)) for n, s in __import__("iron_amd.applications.llama", fromlist=["shapes"]).shapes(config).items()
                            if "embed" not in n) + config.vocab_size * config.hidden_size)
    kv_bytes = sum((512 + 1 + i) * 2 * config.num_key_value_heads * config.head_dim * 2 * config.num_hidden_layers
                   for i in range(steps)) / steps
    per_token = weight_bytes + kv_bytes
    tok_s = steps / (ms / 1e3)
    out = {"tok_s": round(tok_s, 1), "ms_per_token": round(ms / steps, 4), "ttft_ms": round(ttft * 1e3, 2),
           "ttft_runs_ms": [round(t * 1e3, 2) for t in ttfts], "prefill_tokens": 512, "decode_steps": steps, "wall_s": round(wall, 4),
           "bytes_per_token": int(per_token), "GBps": round(per_token * tok_s / 1e9, 1),
           "frac_hbm": round(per_token * tok_s / 1e9 / HBM_PEAK_GBS, 4),
           "steps_recorded": len(decode.recording.steps),
           "launches_per_step": decode.launches_per_replay,
           "launches_per_prompt_chunk": model.prompt_chunk.launches_per_call, "first_tokens": [int(t) for t in tokens[:4]]}
    cpu = None
    if with_cpu:
        drawn = decode.read(model.drawn)[511 : 512 + steps]   # the prompt's draw, then each decode step's
        cpu, out["checked"] = cpu_decoder_baseline(torch, config, weights, prompt, prompt_logits, [int(t) for t in drawn])
    model.release()
    del model
    torch.cuda.empty_cache()
    out["max_seq_len"] = config.max_seq_len
    out["by_max_seq_len"] = [{"max_seq_len": config.max_seq_len, "tok_s": out["tok_s"], "ms_per_token": out["ms_per_token"],
                              "ttft_ms": out["ttft_ms"], "launches_per_step": out["launches_per_step"],
                              "first_tokens": out["first_tokens"]}] + bench_decoder_contexts(torch, dev, steps, warmup, weights)
    return out, cpu


def cpu_decoder_baseline(torch, config, weights, prompt, gpu_prompt_logits, gpu_tokens, budget_s=12.0):
    """The oracle's graph reference (the reference's CPU path: the graph run step by step through
    each operator's numpy reference) on the same 16-layer model and the same 512-token prompt.

    First the check that makes the timed model a checked one: the host's logits after the prompt
    against the GPU's by the reference's rule (within 5 % of the largest logit, the same argmax
    where the top two are further apart than that: iron/lm/testing.py:182-206), and the GPU's first
    drawn token against the host's logits.  Then decode steps from the GPU's own tokens are timed on
    the host cores for about ``budget_s`` seconds, each compared with the GPU's next token the same way."""
    import dataclasses

    import oracle
    from iron_amd.applications.llama import Llama
    from iron_amd.bf16 import from_torch
    from iron_amd.lm.causal import OnHost

    oracle.install()

    class HostLlama(OnHost, Llama):
        pass

    def judge(host_logits, got_logits, got_token, what):
        scale = float(np.abs(host_logits).max())
        second, best = np.sort(host_logits)[-2:]
        if got_logits is not None:
            err = float(np.abs(got_logits - host_logits).max())
            assert err <= 0.05 * scale, f"{what}: max |diff| {err:.4f} against |logits| {scale:.3f}"
            if best - second > 0.05 * scale:
                assert int(got_logits.argmax()) == int(host_logits.argmax()), f"{what}: argmax differs"
        # the token the device drew is the host's best, or within the logits' tolerance of it
        assert host_logits[got_token] >= best - 0.05 * scale, f"{what}: the drawn token {got_token} is not a best one"
        return round(float(np.abs(got_logits - host_logits).max()) / scale, 5) if got_logits is not None else None

    host_weights = {n: from_torch(t) for n, t in weights.items()}
    # The host's chunk is as long as the prompt: the rows past a bound are nobody's.
    model = HostLlama(dataclasses.replace(config, prefill_chunk=len(prompt)), host_weights)
    model.load_versions()
    t0 = time.perf_counter()
    host_logits = model.logits(prompt)
    prefill_s = time.perf_counter() - t0
    share = judge(host_logits, gpu_prompt_logits, gpu_tokens[0], "the prompt's logits")
    # Two timed legs over the same steps' worth of budget.  First as the reference's CPU path runs a
    # GEMV: the weight is held as bf16 storage and widened to float32 on every call (gemv.py:413) --
    # the oracle's GEMV is handed the weight's bits and widens them; then with the weights held as
    # float32 (no widening), which is the faster host program and is reported beside it.
    from iron_amd.bf16 import from_bits, to_bits
    from iron_amd.common.declare import REFERENCES

    from iron_amd.common.graph import Param, Weight, walk

    # The host reference keeps each weight as one float32 array (``Resident.host``) and hands the GEMV
    # a view of it: the view's address names the weight whose bits to widen.
    bits = {x.host.ctypes.data: to_bits(x.host.reshape(x.shape)) for _, x, _, _ in walk(model)
            if isinstance(x, (Param, Weight)) and len(x.shape) == 2 and getattr(x, "host", None) is not None}
    plain_gemv = REFERENCES["GEMV"]
    widened = [0]

    def widening_gemv(op, A, B):
        held = bits.get(np.asarray(A).ctypes.data)
        if held is None:
            return plain_gemv(op, A, B)
        widened[0] += 1
        return plain_gemv(op, from_bits(held), B)

    history, checked, legs = list(map(int, prompt)), 1, {}
    at = 0
    for leg, gemv in (("widened", widening_gemv), ("float32", plain_gemv)):
        REFERENCES["GEMV"] = gemv
        steps = 0
        t0 = time.perf_counter()
        try:
            while time.perf_counter() - t0 < budget_s / 2 and at + 1 < len(gpu_tokens):
                history.append(gpu_tokens[at])
                row = model.logits(history)
                at += 1
                steps += 1
                judge(row, None, gpu_tokens[at], f"decode step {at}")
                checked += 1
        finally:
            REFERENCES["GEMV"] = plain_gemv
        legs[leg] = (steps, time.perf_counter() - t0)
    steps, dt = legs["widened"]
    plain_steps, plain_dt = legs["float32"]
    assert steps == 0 or widened[0] >= steps * (7 * config.num_hidden_layers + 1), "the widening leg widened nothing"
    cpu = {"value": round(steps / dt, 3) if steps else None, "unit": "tok/s", "cores": torch.get_num_threads(), "kind": "port",
           "value_float32_weights": round(plain_steps / plain_dt, 3) if plain_steps else None,
           "sample": f"{steps} decode steps after the same 512-token prompt (prefilled on the host in {prefill_s:.1f} s) "
                     f"of the same 16-layer model through the oracle's graph reference, teacher-forced on the GPU's "
                     f"tokens, {dt:.1f} s wall, every weight widened from bf16 storage on every call as the reference's "
                     f"GEMV does (gemv.py:413); value_float32_weights: the next {plain_steps} steps with the weights held "
                     f"as float32, {plain_dt:.1f} s wall"}
    return cpu, {"rule": "within 5 % of the largest logit; same argmax where the top two are apart; each GPU token a best "
                         "one of the host's logits", "prompt_logits_max_diff_share": share, "tokens_checked": checked}


PROBE_COPY_BYTES = 512 << 20
# HBM bytes one launch moves, by kernel, from hardware counters (FETCH_SIZE and WRITE_SIZE per
# dispatch, each scaled by what the same counter reads for a plain copy of PROBE_COPY_BYTES): filled
# from counter runs of `--decode-probe` / `--counter-probe`; a kernel without a reading reports null.
DOMINANT_TRAFFIC_SOURCE = ("profiles/llama1b_decode_step_hbm_counters.txt (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, over "
                           "`bench.py --decode-probe 8`; the kernels' template arguments as of that run: a kernel whose "
                           "arguments have changed since finds no entry and reports null)")
DOMINANT_TRAFFIC_BYTES: dict[str, int] = {
    "gemv_fused_kernel<2,1,true,2>": 67_353_000,     # norm + gate/up + SiLU*mul: 67.222 MB fetched + 0.131 written
    "gemv_fused_kernel<2,4,false,1>": 33_783_000,    # down projection + residual: 33.750 + 0.033
    "gemv_fused_kernel<4,1,true,0>": 526_446_000,    # final norm + LM head: 525.42 + 1.03
    "decode_qkv_kernel<64,1,false,2>": 12_753_000,   # norm + q/k/v + RoPE + cache rows: 12.708 + 0.045
    "gemv_fused_kernel<1,1,false,1>": 8_513_000,     # o projection + residual: 8.48 + 0.03
}


def counter_probe(torch, K, dev, rng):
    """The dominant kernel (the 2048 -> 128256 head GEMV over two distinct weights, 4 launches) and a
    plain copy that reads and writes PROBE_COPY_BYTES (2 launches): what a hardware-counter run needs
    to turn FETCH_SIZE / WRITE_SIZE readings of the GEMV into bytes."""
    from iron_amd.bf16 import round_bf16, to_torch

    Kdim, N = GEMV_SWEEP[-1]
    base = to_torch(round_bf16(rng.standard_normal((N, Kdim), dtype=np.float32) * np.float32(0.02))).to(dev)
    pool = [base, base.clone()]
    x = to_torch(round_bf16(rng.standard_normal(Kdim, dtype=np.float32))).to(dev)
    y = torch.empty(N, dtype=torch.bfloat16, device=dev)
    rows, row_bytes = PROBE_COPY_BYTES // 4096, 4096
    src = torch.zeros(PROBE_COPY_BYTES // 4, dtype=torch.int32, device=dev)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    for i in range(4):
        K.gemv(pool[i % 2], x, y, M=N, K=Kdim)
    for _ in range(2):
        K.copy_rows(src, dst, rows=rows, row_elems=row_bytes // 4, src_rows=rows, dst_rows=rows)
    # The MFMA kernels, for a run that reads the matrix pipe's counters: the headline GEMM (weights as
    # stored, (N,K)), the 256 x 256-tile kernel at 8192^3, and prompt attention at S = 2048 and 8192.
    def drawn(*shape, scale=0.02):
        return (torch.randn(*shape, device=dev) * scale).to(torch.bfloat16)

    for n_, launches in ((2048, 3), (8192, 2)):
        A, B, C = drawn(n_, n_), drawn(n_, n_), torch.empty((n_, n_), dtype=torch.bfloat16, device=dev)
        for _ in range(launches):
            K.gemm(A, B, C, M=n_, N=n_, K=n_, b_col_maj=True)
        del A, B, C
    H, G, D = 32, 8, 64
    for S in (2048, 8192):
        Q, Kc, Vc = drawn(S, H, D, scale=1.0), drawn(S, G, D, scale=1.0), drawn(S, G, D, scale=1.0)
        O = torch.empty_like(Q)
        for _ in range(2):
            K.mha_prefill(Q, Kc, Vc, O, heads=H, kv_heads=G, d=D, seq=S, seq_len=S, kv_len=S, scale=D**-0.5, causal=True,
                          q_interleaved=True, kv_interleaved=True)
    torch.cuda.synchronize()
    print(json.dumps({"probe": "counter", "gemv": {"K": Kdim, "N": N, "launches": 4,
                                                     "algorithmic_bytes": 2 * (N * Kdim + Kdim + N)},
                      "copy": {"launches": 2, "bytes_read": PROBE_COPY_BYTES, "bytes_written": PROBE_COPY_BYTES},
                      "gemm": [{"n": 2048, "launches": 3}, {"n": 8192, "launches": 2}],
                      "attention_prefill": [{"S": 2048, "launches": 2}, {"S": 8192, "launches": 2}]}))


def attention_probe(torch, K, dev):
    """One query over caches of 1024, 4096 and 16384 keys (32 q / 8 kv heads, d 64), 4 launches each over
    distinct caches, then a plain copy of known size: what a counter or kernel-trace run of decode
    attention alone needs."""
    H, G, D = 32, 8, 64
    ws = K.mha_decode_workspace(H, D, dev)
    shapes = []
    for L in (1024, 4096, 16384):
        Q = torch.randn((1, H, D), device=dev).to(torch.bfloat16)
        O = torch.empty_like(Q)
        for _ in range(4):
            Kc, Vc = (torch.randn((L, G, D), device=dev).to(torch.bfloat16) for _ in range(2))
            K.mha_decode(Q, Kc, Vc, O, heads=H, kv_heads=G, d=D, kv_len=L, scale=0.125, kv_interleaved=True, workspace=ws)
        shapes.append({"L": L, "launches": 4, "algorithmic_bytes": 2 * L * G * D * 2 + 2 * H * D * 2})
    rows = PROBE_COPY_BYTES // 4096
    src = torch.zeros(PROBE_COPY_BYTES // 4, dtype=torch.int32, device=dev)
    dst = torch.empty_like(src)
    for _ in range(2):
        K.copy_rows(src, dst, rows=rows, row_elems=1024, src_rows=rows, dst_rows=rows)
    torch.cuda.synchronize()
    print(json.dumps({"probe": "attention", "decode": shapes,
                      "copy": {"launches": 2, "bytes_read": PROBE_COPY_BYTES, "bytes_written": PROBE_COPY_BYTES}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128, help="timed decode steps (tokens)")
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--kernel-launches", type=int, default=400, help="timed launches per kernel micro-benchmark")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--counter-probe", action="store_true",
                    help="launch only the LM-head GEMV, a plain copy of known size and the MFMA kernels (for a rocprofv3 --pmc run) and exit")
    ap.add_argument("--no-library", action="store_true",
                    help="skip the vendor-library leg (torch.matmul / SDPA for scale): a kernel trace then lists this build's kernels only")
    ap.add_argument("--decode-probe", type=int, default=0, metavar="N",
                    help="prefill the 512-token prompt once, replay N decode steps and exit (for a rocprofv3 --kernel-trace or --pmc run)")
    ap.add_argument("--prompt-probe", action="store_true",
                    help="run only the decoder's 512-token prompt chunk, 20 times (for a rocprofv3 --kernel-trace run) and exit")
    ap.add_argument("--attention-probe", action="store_true",
                    help="launch only decode attention at 1024 / 4096 / 16384 keys and a plain copy of known size "
                         "(for a rocprofv3 --pmc or --kernel-trace run) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build is a one-GPU hot path; --gpus must be 1 "
              "(how the path would shard is described, not built)", file=sys.stderr)
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

    if args.counter_probe:
        counter_probe(torch, K, dev, rng)
        return 0
    if args.prompt_probe:
        prompt_probe(torch, dev)
        return 0
    if args.attention_probe:
        attention_probe(torch, K, dev)
        return 0
    if args.decode_probe:
        bench_decoder(torch, dev, args.steps, args.warmup, False, probe_steps=args.decode_probe)
        return 0

    t_wall = time.perf_counter()
    n = args.kernel_launches
    gemv = [bench_gemv(torch, K, dev, Kd, N, n, rng) for Kd, N in GEMV_SWEEP]
    gemm = [bench_gemm(torch, K, dev, n, rng, b) for b in (False, True)]
    # The prefill projections of the decoder (2048 tokens; weights (N,K)) and two larger squares.
    gemm += [bench_gemm(torch, K, dev, max(20, n // 4), rng, True, M=m, N=nn, Kd=k)
             for m, nn, k in ((2048, 8192, 2048), (2048, 2048, 8192), (4096, 4096, 4096), (8192, 8192, 8192))]
    gemm.append(bench_gemm(torch, K, dev, max(20, n // 4), rng, False, M=4096, N=4096, Kd=4096))   # B (K,N) on the large tiles
    attention = bench_attention(torch, K, dev, n, rng)
    pre_attention = bench_pre_attention(torch, K, dev, n)
    sample = bench_sample(torch, K, dev, n, rng)
    library = None if args.no_library else bench_library_reference(torch, dev, n, rng)
    decode_kernels = bench_decode_kernels(torch, K, dev, n, rng)
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    decoder, cpu = bench_decoder(torch, dev, args.steps, args.warmup, not args.no_cpu)
    wall = time.perf_counter() - t_wall

    dominant = max(decode_kernels, key=lambda r: r["per_step"] * r["us"])
    sweep_bytes = sum(g["bytes"] for g in gemv)
    sweep_us = sum(g["us"] for g in gemv)
    head = gemv[-1]
    out = {
        "metric": "bf16 GEMM TFLOP/s, GEMV GB/s (% roofline); Llama-3.2-1B-shape decode tok/s",
        "value": decoder["tok_s"],
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": decoder["ms_per_token"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "Llama-3.2-1B-shape decoder (16 layers, hidden 2048, 32 q / 8 kv heads, head_dim 64, "
                               "SwiGLU 8192, vocab 128256, tied embeddings), random-init bf16 N(0,0.02), batch 1: "
                               "512-token prompt prefill, then greedy decode steps replayed as a HIP graph; "
                               "one step = one decoded token",
                   "prefill_tokens": 512, "decode_steps": args.steps},
        "roofline": {"bound": "hbm", "kernel": dominant["kernel"], "what": dominant["name"],
                     "why": f"the decode step's dominant kernel by time ({dominant['per_step']} launches a step, "
                            f"{dominant['share_of_listed_us']:.0%} of the step's kernel time); timed alone at its shape "
                            "over distinct weights with HIP events in this run",
                     "achieved": dominant["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dominant["frac_hbm"],
                     "us": dominant["us"], "algorithmic_bytes": dominant["bytes"],
                     "traffic": DOMINANT_TRAFFIC_BYTES.get(dominant["kernel"]),
                     "traffic_source": DOMINANT_TRAFFIC_SOURCE + "; not measured in this run"},
        "decode_step_kernels": decode_kernels,
        "decoder": decoder,
        "gemv_sweep": {"GBps": round(sweep_bytes / sweep_us / 1e3, 1), "shapes": gemv},
        "gemm": gemm,
        "attention": attention,
        "pre_attention_block": pre_attention,
        "sample": sample,
        **({} if library is None else {"library_reference": library}),
        "bench_wall_s": round(wall, 1),
    }
    if cpu is not None:
        out["cpu_baseline"] = cpu
        out["cpu_baseline_gemv"] = cpu_gemv_baseline(np.random.default_rng(7), budget_s=6.0)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
