#!/usr/bin/env python3
"""Benchmark of the raw-block quantized matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--eager] [--no-extra] [--no-cpu-baseline]

A step is one pass of the decode matvec over the Q4_K / Q5_K weights of the Qwen3-27B-like shapes
(N x K = 5120 x 5120 and 17408 x 5120, one bf16 activation row): four operator calls, each on the
next copy in a ring of weight copies that together exceed the 256 MB last-level cache several
times, so the bytes come from HBM.  Inputs are synthetic (seeded N(0, 0.02) weights quantized by
this package's encoders, N(0, 1) activations) and resident in HBM before the timed region.  Steps
are replayed from one HIP graph that holds a step for every ring slot, so that the Python wrapper is
not what is timed; --eager times the plain operator calls instead.  --pmc-pass runs only a few
launches of the dominant kernel and of a plain copy of the same size: the short program the
rocprofv3 counter passes under profiles/ are taken from.

The one JSON line printed at the end carries whole-step throughput (weight bytes / time), the
roofline figures of the dominant kernel measured with HIP events on the launch stream, the CPU
dequantize-then-matmul baseline, and a table of the other formats of the path (`cases`).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np
import torch

HBM_PEAK_GBS = 8000.0
RING = 12                     # weight copies per case

CASES = [  # (type name, type id, N, K)
    ("q4_k", 3, 5120, 5120),
    ("q4_k", 3, 17408, 5120),
    ("q5_k", 4, 5120, 5120),
    ("q5_k", 4, 17408, 5120),
]
DOMINANT = 3   # index into CASES: the launch the roofline object describes

# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by
# what the same counters read for a plain copy of known size (profiles/q5k_matvec_17408x5120_counters.md)
TRAFFIC_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "traffic.json")


def _encoders():
    from pocketllm_amd import block_codec as C
    return {"q4_k": C.quantize_q4_k, "q5_k": C.quantize_q5_k, "q2_k": C.quantize_q2_k}


def ring_of(blocks: np.ndarray, device, copies: int = RING):
    first = torch.from_numpy(blocks).to(device)
    return [first] + [first.clone() for _ in range(copies - 1)]


MIN_TIMED_LAUNCHES = 200      # per repeat
REPEATS = 5                   # the median of this many repeats is reported
RING_BYTES = 512 << 20        # a case's weight copies in rotation: twice the 256 MB last-level cache


def ring_copies(nbytes: int, least: int = 2) -> int:
    return max(least, -(-RING_BYTES // max(1, nbytes)))


def event_time_us(fn, slots, iters, warm=5):
    """Median over REPEATS of the average duration of fn(slot) over `iters` back-to-back calls, HIP events on the current stream."""
    for i in range(warm):
        fn(i % slots)
    torch.cuda.synchronize()
    samples = []
    for _ in range(REPEATS):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(iters):
            fn(i % slots)
        e1.record()
        torch.cuda.synchronize()
        samples.append(e0.elapsed_time(e1) * 1e3 / iters)
    return float(np.median(samples))


def capture(fn, slots):
    """One HIP graph holding fn(0) .. fn(slots - 1); returns (replay, True), or (None, False) if capture fails."""
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for s in range(slots):
                fn(s)                                   # warm allocator and kernels on a side stream first
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for s in range(slots):
                fn(s)
        torch.cuda.synchronize()
        return g.replay, True
    except Exception as exc:                             # pragma: no cover - depends on the runtime
        print(f"bench.py: graph capture failed ({exc!r}); timing eager calls", file=sys.stderr)
        torch.cuda.synchronize()
        return None, False


def time_calls_us(fn, slots, iters=MIN_TIMED_LAUNCHES, eager=False):
    """Duration of one fn(slot) call: a graph of `slots` calls replayed until at least `iters` calls have run, or eager calls;
    the median of REPEATS such measurements."""
    replay, graphed = (None, False) if eager else capture(fn, slots)
    if graphed:
        reps = max(1, -(-iters // slots))
        return event_time_us(lambda _s: replay(), 1, reps, warm=2) / slots, True
    return event_time_us(fn, slots, max(iters, slots)), False


def _median_time(fn, budget_s: float, most: int = 10):
    """Median wall time of fn() over up to `most` calls within the budget (at least two; the first call only warms up)."""
    times = []
    t_begin = time.perf_counter()
    while len(times) < most + 1 and (time.perf_counter() - t_begin < budget_s or len(times) < 2):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    times = times[1:]
    return float(np.median(times)), len(times)


def cpu_baseline(blocks: np.ndarray, type_name: str, k: int, x: np.ndarray, budget_s: float = 8.0):
    """The reference's CPU path restated: numpy block decode to float32, then torch matmul."""
    from oracle import gguf_oracle as O
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    xt = torch.from_numpy(x.astype(np.float32))
    parts = []

    def call():
        t0 = time.perf_counter()
        w = O.dequant_rows(blocks, type_name, k)
        t1 = time.perf_counter()
        torch.nn.functional.linear(xt, torch.from_numpy(w))
        parts.append((t1 - t0, time.perf_counter() - t1))

    total, calls = _median_time(call, budget_s, most=5)
    parts = parts[1:]
    return {
        "value": round(blocks.size / total / 1e9, 4),
        "unit": "GB/s",
        "cores": int(torch.get_num_threads()),
        "kind": "port",
        "sample": (f"{type_name} {blocks.shape[0]}x{k} matvec, numpy block decode ({np.median([t[0] for t in parts]) * 1e3:.0f} ms, "
                   f"one thread) + torch F.linear fp32 ({np.median([t[1] for t in parts]) * 1e3:.1f} ms, {torch.get_num_threads()} threads), "
                   f"median of {calls} calls"),
        "ms_per_call": round(total * 1e3, 3),
    }


def cpu_baselines_more(q4k_blocks: np.ndarray, x5120: np.ndarray):
    """Further CPU lines, each a few seconds of host work:
      * BASELINE config 1 as the reference runs it on the CPU (src/kernels/ops.py:766-792): Q8_0 4096x4096 dequantized to a
        float32 matrix, then F.linear, restated with the oracle's decoder;
      * this repository's plain-C raw-block matvec (oracle/rawblock_cpu.c, OpenMP over rows, no float copy of the matrix) on
        the same Q8_0 matrix and on Q4_K 5120x5120;
      * the reference's own compiled CPU kernel gguf_quantized_matmul (src/csrc/deepseek_cpu_moe_ext.cpp:2759-2803, AVX2 +
        OpenMP; it serves IQ2_XXS and Q2_K) where oracle/_ref holds it: Q2_K 5120x5120, kind "reference"."""
    from oracle import gguf_oracle as O
    from pocketllm_amd import block_codec as C
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    rng = np.random.default_rng(1001)
    out = []
    w = rng.standard_normal((4096, 4096), dtype=np.float32) * np.float32(0.02)
    q8 = C.pack_q8_0(w)
    x1 = rng.standard_normal((1, 4096), dtype=np.float32)
    xt = torch.from_numpy(x1)
    total, calls = _median_time(lambda: torch.nn.functional.linear(xt, torch.from_numpy(O.dequant_rows(q8, "q8_0", 4096))), 4.0, most=8)
    out.append({"case": "q8_0 4096x4096 T=1 (BASELINE config 1): dequantize to float32 + F.linear", "kind": "port", "cores": threads,
                "ms_per_call": round(total * 1e3, 3), "value": round(q8.size / total / 1e9, 4), "unit": "GB/s", "calls": calls})
    try:
        from oracle import rawblock_cpu as R
        if R.available():
            for label, blocks, name, xx in (("q8_0 4096x4096 T=1", q8, "q8_0", x1), ("q4_k 5120x5120 T=1", q4k_blocks, "q4_k", x5120)):
                total, calls = _median_time(lambda: R.matvec(blocks, name, xx), 2.0, most=20)
                out.append({"case": f"{label}: raw-block matvec in plain C, OpenMP over rows (oracle/rawblock_cpu.c)", "kind": "port",
                            "cores": threads, "ms_per_call": round(total * 1e3, 3), "value": round(blocks.size / total / 1e9, 4),
                            "unit": "GB/s", "calls": calls})
    except OSError as exc:                                # pragma: no cover - a library built for another host
        print(f"bench.py: oracle/_build not usable here ({exc})", file=sys.stderr)
    try:
        from oracle import ref_ext
        if ref_ext.available():
            q2 = C.quantize_q2_k(rng.standard_normal((5120, 5120), dtype=np.float32) * np.float32(0.02))
            grid = O.iq2xxs_signed_grid()
            total, calls = _median_time(lambda: ref_ext.quantized_matmul(x5120, q2, 1, grid), 2.0, most=20)
            out.append({"case": "q2_k 5120x5120 T=1: the reference's compiled CPU kernel gguf_quantized_matmul (oracle/_ref)", "kind": "reference",
                        "cores": threads, "ms_per_call": round(total * 1e3, 3), "value": round(q2.size / total / 1e9, 4), "unit": "GB/s",
                        "calls": calls})
    except (OSError, ImportError) as exc:                 # pragma: no cover
        print(f"bench.py: oracle/_ref not usable here ({exc})", file=sys.stderr)
    return out


def extra_cases(mod, dev):
    """Other formats of the path, one line each (event-timed eager launches are launch-bound for the
    small ones, so these replay graphs as well)."""
    from pocketllm_amd import block_codec as C, codebooks
    rng = np.random.default_rng(3003)
    out = []
    empty = torch.empty(0, dtype=torch.int8, device=dev)

    def run(label, nbytes, fn, slots, extra=None):
        us, graphed = time_calls_us(fn, slots)
        rec = {"case": label, "weight_bytes": int(nbytes), "us_per_call": round(us, 3), "gbs": round(nbytes / us / 1e3, 1),
               "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "graph": graphed}
        if extra:
            rec.update(extra)
        out.append(rec)

    # Q8_0, BASELINE config 1 and the large shape
    for n, k in ((4096, 4096), (17408, 5120)):
        blocks = C.pack_q8_0((rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)))
        ring = ring_of(blocks, dev, ring_copies(blocks.size))
        x = torch.randn(1, k, device=dev)
        run(f"q8_0 matvec {n}x{k} T=1", blocks.size, lambda s, ring=ring, x=x, k=k: mod.q8_0_gemm_forward(x, ring[s], k), len(ring))
        del ring
    # Q2_K and the other five formats at the large shape (random valid blocks for those: the kernels' work does not depend on the values)
    x = torch.randn(1, 5120, device=dev, dtype=torch.bfloat16)
    for name, tid, blocks in (("q2_k", 1, C.quantize_q2_k((rng.standard_normal((17408, 5120), dtype=np.float32) * np.float32(0.02)))),
                              ("q6_k", 8, C.random_blocks(rng, "q6_k", 17408, 20)), ("iq4_xs", 7, C.random_blocks(rng, "iq4_xs", 17408, 20)),
                              ("iq3_xxs", 6, C.random_blocks(rng, "iq3_xxs", 17408, 20)), ("iq2_xs", 5, C.random_blocks(rng, "iq2_xs", 17408, 20))):
        ring = ring_of(blocks, dev, ring_copies(blocks.size))
        grid = codebooks.grid_tensor_for_type(tid).to(dev)
        run(f"{name} matvec 17408x5120 T=1", blocks.size,
            lambda s, ring=ring, x=x, tid=tid, grid=grid: mod.gguf_quant_gemm_forward(x, ring[s], 5120, tid, grid), len(ring))
        del ring
    # paired projection (gate and up of a dense MLP): two Q4_K matrices 17408x5120 against one activation row
    blocks = C.quantize_q4_k((rng.standard_normal((17408, 5120), dtype=np.float32) * np.float32(0.02)))
    ring = ring_of(blocks, dev, 12)
    run("q4_k paired projection 2 x 17408x5120 T=1", 2 * blocks.size,
        lambda s, ring=ring: mod.gguf_quant_gemm_pair_forward(x, ring[s], 5120, 3, ring[(s + 6) % 12], 5120, 3, empty), len(ring))
    # a few activation rows (speculative decoding, small batches): up to sixteen rows share one pass over the weights
    for t in (2, 4, 8, 16):
        xt = torch.randn(t, 5120, device=dev, dtype=torch.bfloat16)
        run(f"q4_k matvec 17408x5120 T={t}", blocks.size, lambda s, ring=ring, xt=xt: mod.gguf_quant_gemm_forward(xt, ring[s], 5120, 3, empty), len(ring))
    del ring
    # normalisation + projection as one decode operator against the two operators one after the other (Q4_K 5120x5120)
    blocks = C.quantize_q4_k((rng.standard_normal((5120, 5120), dtype=np.float32) * np.float32(0.02)))
    ring = ring_of(blocks, dev, ring_copies(blocks.size))
    gamma = torch.ones(5120, device=dev)
    run("rmsnorm + q4_k matvec 5120x5120 T=1, one operator", blocks.size,
        lambda s, ring=ring: mod.gguf_quant_gemm_rmsnorm_forward(x, gamma, 1e-6, ring[s], 5120, 3, empty), len(ring))
    run("rmsnorm + q4_k matvec 5120x5120 T=1, two operators", blocks.size,
        lambda s, ring=ring: mod.gguf_quant_gemm_forward(mod.fused_rms_norm_forward(x, gamma, 1e-6), ring[s], 5120, 3, empty), len(ring))
    del ring
    # FP8 E4M3 + 128x128 scales, BASELINE config 4 at T=1
    codes, scale = C.quantize_fp8_block((rng.standard_normal((17408, 5120), dtype=np.float32) * np.float32(0.02)))
    ring = ring_of(codes, dev, 8)
    sc = torch.from_numpy(scale).to(dev)
    run("fp8_e4m3 matvec 17408x5120 T=1", codes.size + scale.size * 4,
        lambda s, ring=ring, x=x, sc=sc: mod.fp8_block_gemm_forward(x, ring[s], sc), len(ring))
    # a few rows of bf16 activations: one pass over the weights for up to 16 rows on the matrix cores
    for t in (2, 4, 16):
        xt = torch.randn(t, 5120, device=dev, dtype=torch.bfloat16)
        run(f"fp8_e4m3 matvec 17408x5120 T={t}", codes.size + scale.size * 4,
            lambda s, ring=ring, xt=xt, sc=sc: mod.fp8_block_gemm_forward(xt, ring[s], sc), len(ring))
    del ring
    # the same weights with fp16 scales behind the C++ engine's operator forms: matvec and fused gate/up SwiGLU (float32 activations)
    from pocketllm_amd import qwen_fp8_ops as Q
    sc16 = torch.from_numpy(scale.astype(np.float16).view(np.int16)).to(dev)
    ring = ring_of(codes, dev, 8)
    xf = torch.randn(1, 5120, device=dev)
    yf = torch.empty(1, 17408, device=dev)
    run("fp8_e4m3 fp16-scale matvec 17408x5120 T=1", codes.size + scale.size * 2,
        lambda s, ring=ring: Q.qwen_fp8_e4m3_fp16scale_matvec(xf, ring[s], sc16, yf, 17408, 5120, 5120, 40), len(ring))
    run("fp8_e4m3 fp16-scale fused gate/up SwiGLU 2 x 17408x5120 T=1", 2 * (codes.size + scale.size * 2),
        lambda s, ring=ring: Q.qwen_fp8_e4m3_fp16scale_swiglu_matvec(xf, ring[s], sc16, ring[(s + 4) % 8], sc16, yf, 17408, 5120, 5120, 40), len(ring))
    del ring
    # IQ2_XXS / IQ1_M dense matvec at the expert shapes stacked 64 experts high
    for name, tid, n, k, gen, grid in (("iq2_xxs", 0, 64 * 1536, 3072, C.random_iq2_xxs, codebooks.get_iq2xxs_signed_grid_tensor().to(dev)),
                                       ("iq1_m", 2, 64 * 3072, 1536, C.random_iq1_m, codebooks.get_iq1_grid_tensor().to(dev))):
        blocks = gen(rng, n, k // 256)
        ring = ring_of(blocks, dev, ring_copies(blocks.size))
        xx = torch.randn(1, k, device=dev, dtype=torch.bfloat16)
        run(f"{name} matvec {n}x{k} T=1", blocks.size,
            lambda s, ring=ring, xx=xx, k=k, tid=tid, grid=grid: mod.gguf_quant_gemm_forward(xx, ring[s], k, tid, grid), len(ring))
        del ring
    # fused routed experts, BASELINE config 5 at T=1: 256 experts, top-8
    e, d, inter = 256, 3072, 1536
    w1 = torch.from_numpy(C.random_iq2_xxs(rng, e, inter, d // 256, d_range=(0.002, 0.006))).to(dev)
    w3 = torch.from_numpy(C.random_iq2_xxs(rng, e, inter, d // 256, d_range=(0.002, 0.006))).to(dev)
    w2 = torch.from_numpy(C.random_iq1_m(rng, e, d, inter // 256, d_range=(0.002, 0.006))).to(dev)
    logits = torch.from_numpy(rng.standard_normal((RING, e)).astype(np.float32))
    probs = torch.softmax(logits, dim=-1)
    topw, topi = probs.topk(8, dim=-1)
    topw = (topw / topw.sum(dim=-1, keepdim=True)).to(dev)
    topi = topi.to(dev)
    xm = torch.randn(1, d, device=dev, dtype=torch.bfloat16)
    per_call = 8 * (2 * inter * (d // 256) * 66 + d * (inter // 256) * 56)
    run("fused experts iq2_xxs gate/up + iq1_m down, 256 experts top-8, T=1", per_call,
        lambda s: mod.gguf_moe_single_token_forward(xm, topi[s], topw[s], w1, w3, w2, 0.0), RING,
        {"note": "each slot routes to a different random top-8 of the 256 resident experts (887 MB)"})
    # routing ahead of the experts: gate logits + sigmoid + top-8 + renormalisation (256 experts x 3072, float32 gate)
    gate = torch.randn(e, d, device=dev) * (d ** -0.5)
    gbias = torch.zeros(e, device=dev)
    for tt in (1, 256):
        xr = torch.randn(tt, d, device=dev, dtype=torch.bfloat16)
        us, graphed = time_calls_us(lambda s, xr=xr: mod.moe_route(xr, gate, gbias, 8), 4)
        out.append({"case": f"expert routing (gate 256x3072 f32, sigmoid + bias, top-8) T={tt}", "us_per_call": round(us, 3), "graph": graphed,
                    "weight_bytes": e * d * 4, "gbs": round(e * d * 4 / us / 1e3, 1)})
    # the same experts at T=256 (BASELINE config 5): 2048 routes grouped by expert
    t = 256
    logits = torch.from_numpy(rng.standard_normal((t, e)).astype(np.float32))
    tw, ti = torch.softmax(logits, dim=-1).topk(8, dim=-1)
    tw = (tw / tw.sum(dim=-1, keepdim=True)).to(dev)
    _, toks, rws, seg = mod.moe_group_routes(ti.to(dev), tw, 0, e)
    xt = torch.randn(t, d, device=dev, dtype=torch.bfloat16)
    grids = (codebooks.get_iq2xxs_signed_grid_tensor().to(dev), codebooks.get_iq1_grid_tensor().to(dev))
    touched = int((seg[1:] > seg[:-1]).sum().item())
    flops = 2.0 * t * 8 * 3 * inter * d
    us, graphed = time_calls_us(lambda s: mod.gguf_moe_prefill_grouped_forward(xt, toks, rws, seg, w1, w3, w2, d, 0, d, 0, inter, 2, grids, 0.0),
                                4)
    nbytes = touched * (2 * inter * (d // 256) * 66 + d * (inter // 256) * 56)
    out.append({"case": "fused experts iq2_xxs gate/up + iq1_m down, 256 experts top-8, T=256", "weight_bytes": nbytes,
                "us_per_call": round(us, 3), "gbs": round(nbytes / us / 1e3, 1), "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                "tflops": round(flops / us / 1e6, 2), "graph": graphed, "note": f"{touched} of 256 experts touched by the 2048 routes"})
    # routed experts of a type without fused expert kernels (the common Q4_K checkpoints): 128 experts of 2048 -> 768, top-8, route by
    # route through the dense decode kernels (random valid blocks: the work does not depend on the values)
    ek, dk, ik = 128, 2048, 768

    def q4k_random(*lead):
        b = rng.integers(0, 256, size=tuple(lead) + (144,), dtype=np.uint8)
        b[..., 0:2] = np.frombuffer(np.float16(0.01).tobytes(), dtype=np.uint8)
        b[..., 2:4] = np.frombuffer(np.float16(0.005).tobytes(), dtype=np.uint8)
        return torch.from_numpy(b).to(dev)
    kw1, kw3, kw2 = q4k_random(ek, ik, dk // 256), q4k_random(ek, ik, dk // 256), q4k_random(ek, dk, ik // 256)
    kbytes = 8 * (2 * ik * (dk // 256) + dk * (ik // 256)) * 144
    ksets = [torch.from_numpy(rng.choice(ek, size=8, replace=False).astype(np.int64)).to(dev) for _ in range(8)]
    kwts = torch.full((8,), 0.125, device=dev)
    xk = torch.randn(1, dk, device=dev, dtype=torch.bfloat16)
    run("routed experts q4_k, 128 experts top-8, 2048 -> 768, T=1 (two launches)", kbytes,
        lambda s: mod.gguf_moe_single_token_forward(xk, ksets[s], kwts, kw1, kw3, kw2, 0.0), 8)
    idx16 = np.stack([rng.choice(ek, size=8, replace=False) for _ in range(16)]).astype(np.int64)
    _, ktoks, krws, kseg = mod.moe_group_routes(torch.from_numpy(idx16).to(dev), torch.full((16, 8), 0.125, device=dev), 0, ek)
    xk16 = torch.randn(16, dk, device=dev, dtype=torch.bfloat16)
    us, graphed = time_calls_us(lambda s: mod.gguf_moe_prefill_grouped_forward(xk16, ktoks, krws, kseg, kw1, kw3, kw2, dk, 3, dk, 3, ik, 3, empty, 0.0), 4)
    out.append({"case": "routed experts q4_k, 128 experts top-8, 2048 -> 768, T=16 (128 routes, route by route)", "us_per_call": round(us, 3), "graph": graphed})
    del kw1, kw3, kw2
    # one decoder layer's quantized-matmul path at T=1, MiniMax-M2 shapes (hidden 3072, 48 query / 8 key-value heads of 128, 256 experts
    # of 1536, top-8): norm + Q5_K q/k/v projections, Q5_K output projection, norm + routing, fused experts.  Attention itself
    # (rotary embedding, cache, softmax) is not on this path: the projection output feeds the next step directly.
    def q5(n, k):
        return torch.from_numpy(C.quantize_q5_k((rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)))).to(dev)
    wq, wk, wv, wo = q5(6144, d), q5(1024, d), q5(1024, d), q5(d, 6144)
    g1, g2 = torch.ones(d, device=dev), torch.ones(d, device=dev)
    hx = torch.randn(1, d, device=dev, dtype=torch.bfloat16)
    hres = torch.zeros(1, d, device=dev, dtype=torch.float32)

    def layer(_s):
        q, _k, _v = mod.gguf_quant_gemm_multi_forward(hx, (wq, wk, wv), d, 4, empty, norm_weight=g1, eps=1e-6)   # one launch
        o = mod.gguf_quant_gemm_accumulate_forward(q, wo, 6144, 4, empty, hres)     # residual connection folded into the projection
        h2 = mod.fused_rms_norm_forward(o, g2, 1e-6)
        ridx, rw = mod.moe_route(h2, gate, gbias, 8)
        return mod.gguf_moe_single_token_forward(h2, ridx[0], rw[0], w1, w3, w2, 0.0)

    layer_bytes = (wq.numel() + wk.numel() + wv.numel() + wo.numel()) + per_call + e * d * 4
    us, graphed = time_calls_us(layer, 4)
    out.append({"case": "decoder layer matmul path only, MiniMax-M2 shapes, T=1, cache-resident (norm + q/k/v projections in one launch, output projection + residual, norm, routing, experts)",
                "us_per_call": round(us, 3), "graph": graphed,
                "note": "7 launches of one layer replayed on the same input: projections, gate and the 8 routed experts stay in cache, no attention core; "
                        "the launch-chain cost of the matmul path, not an HBM figure (the block module itself is timed in the cases that follow)"})
    del wq, wk, wv, wo
    out += block_stack_cases(mod, dev, rng, w1, w3, w2)
    del w1, w3, w2
    # one dense feed-forward block at T=1, hidden 5120, intermediate 17408, Q4_K: y += W_down (SiLU(W_gate n(x)) * W_up n(x)), as three
    # launches (norm + gate/up in one, SiLU * up into the activation image, down projection with the residual in its store) and as the
    # chain of separate operators a runtime would otherwise issue
    dff, iff = 5120, 17408
    def q4(n, k):
        return torch.from_numpy(C.quantize_q4_k((rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)))).to(dev)
    base = (q4(iff, dff), q4(iff, dff), q4(dff, iff))
    rings = [base] + [tuple(t.clone() for t in base) for _ in range(2)]        # 450 MB in rotation: the weights come from HBM
    gff = torch.ones(dff, device=dev)
    xff = torch.randn(1, dff, device=dev, dtype=torch.bfloat16)
    yres = torch.zeros(1, dff, device=dev, dtype=torch.float32)

    def ffn_fused(sl):
        wg, wu, wd = rings[sl]
        g, u = mod.gguf_quant_gemm_multi_forward(xff, (wg, wu), dff, 3, empty, norm_weight=gff, eps=1e-6, out_dtype=torch.float32)
        image = mod.swiglu_quantize_activations(g, u, iff // 256, round_dtype=torch.bfloat16)
        return mod.gguf_quant_gemm_prequantized(image, wd, 3, accumulate_into=yres)

    def ffn_chain(sl):
        wg, wu, wd = rings[sl]
        hn = mod.fused_rms_norm_forward(xff, gff, 1e-6)
        gu = mod.gguf_quant_gemm_pair_forward(hn, wg, dff, 3, wu, dff, 3, empty)
        h = torch.nn.functional.silu(gu[0]) * gu[1]
        yres.add_(mod.gguf_quant_gemm_forward(h, wd, iff, 3, empty, out_dtype=torch.float32))
        return yres

    ffn_bytes = sum(t.numel() for t in rings[0])
    for label, fn in (("three launches (norm + gate/up, SiLU * up image, down + residual)", ffn_fused), ("separate operators", ffn_chain)):
        us, graphed = time_calls_us(fn, 3)
        out.append({"case": f"dense feed-forward block q4_k 5120 -> 17408 -> 5120, T=1, {label}", "weight_bytes": int(ffn_bytes),
                    "us_per_call": round(us, 3), "gbs": round(ffn_bytes / us / 1e3, 1),
                    "frac_hbm_peak": round(ffn_bytes / us / 1e3 / HBM_PEAK_GBS, 4), "graph": graphed})
    del rings, base
    return out + prefill_cases(mod, dev)


def block_stack_cases(mod, dev, rng, w1, w3, w2):
    """The decoder block MODULE (pocketllm_amd.minimax_block.MiniMaxBlock.__call__: norm, q / k / v, rotary phases, key/value store,
    attention over a 2048-token cache, output projection + residual, norm, routing, routed experts, residual) and a
    MiniMaxTransformer-shaped stack of eight such blocks between a raw-block embedding and the vocabulary projection, at MiniMax-M2
    shapes (hidden 3072, 48 / 8 heads of 128, 256 experts of 1536, top-8, vocabulary 200064).  Every layer has its own projection
    and expert tensors (7.3 GB in all) and every replayed step has its own token, so routes differ from step to step and the
    weights come from HBM.  Reported in the form of src/runtime/generation.py:262-268."""
    from pocketllm_amd import block_codec as C
    from pocketllm_amd.minimax_block import ExpertLayer, MiniMaxAttention, MiniMaxBlock, MiniMaxM2Args, MiniMaxMoE, MiniMaxTransformer, RMSNorm
    from pocketllm_amd.quantized_ops import QuantizedGGUFEmbedding, QuantizedGGUFLinear
    from pocketllm_amd.quantized_tensor import QuantizedGGUFTensor
    out = []
    d, inter, e, vocab, n_layers, cache_len = 3072, 1536, 256, 200064, 8, 2048
    a = MiniMaxM2Args(dim=d, n_heads=48, n_kv_heads=8, head_dim=128, rope_dim=64, rope_base=5.0e6, n_routed_experts=e, top_k=8,
                      moe_inter_dim=inter, norm_eps=1e-6)

    def q5_linear(n, k, name):
        blocks = torch.from_numpy(C.quantize_q5_k((rng.standard_normal((n, k), dtype=np.float32) * np.float32(k ** -0.5)))).to(dev)
        return QuantizedGGUFLinear(QuantizedGGUFTensor.from_blocks(blocks, "q5_k", k, source_name=name))

    base = {"q": q5_linear(a.n_heads * a.head_dim, d, "q"), "k": q5_linear(a.n_kv_heads * a.head_dim, d, "k"),
            "v": q5_linear(a.n_kv_heads * a.head_dim, d, "v"), "o": q5_linear(d, a.n_heads * a.head_dim, "o")}
    layers = []
    for i in range(n_layers):
        def own(lin, i=i):                   # this layer's own copy of the tensor, rows rotated so that no two layers hold the same bytes
            t = lin.tensor
            return QuantizedGGUFLinear(QuantizedGGUFTensor.from_blocks(t.blocks.roll(17 * i + 1, 0), "q5_k", int(t.row_elems), source_name=f"blk.{i}"))
        experts = ExpertLayer(*(QuantizedGGUFTensor.from_blocks(t.roll(29 * i + 1, 0), name, k)
                                for t, name, k in ((w1, "iq2_xxs", d), (w3, "iq2_xxs", d), (w2, "iq1_m", inter))))
        gate = torch.randn(e, d, device=dev) * (d ** -0.5)
        moe = MiniMaxMoE(a, gate, torch.zeros(e, device=dev), experts)
        attn = MiniMaxAttention(a, own(base["q"]), own(base["k"]), own(base["v"]), own(base["o"]),
                                RMSNorm(torch.ones(a.n_heads * a.head_dim, device=dev), a.norm_eps), RMSNorm(torch.ones(a.n_kv_heads * a.head_dim, device=dev), a.norm_eps))
        layers.append(MiniMaxBlock(a, torch.ones(d, device=dev), torch.ones(d, device=dev), attn, moe))
    part = vocab // 8
    emb_blocks = torch.from_numpy(C.random_blocks(rng, "q6_k", part, d // 256)).to(dev).repeat(8, 1, 1)
    head_blocks = torch.from_numpy(C.random_blocks(rng, "q6_k", part, d // 256)).to(dev).repeat(8, 1, 1)
    model = MiniMaxTransformer(a, QuantizedGGUFEmbedding(QuantizedGGUFTensor.from_blocks(emb_blocks, "q6_k", d, source_name="token_embd")), layers,
                               torch.ones(d, device=dev), QuantizedGGUFLinear(QuantizedGGUFTensor.from_blocks(head_blocks, "q6_k", d, source_name="output")),
                               device=dev)
    model.reset_cache(1, cache_len)
    for layer in layers:                     # a cache as 2047 earlier tokens would have left it
        layer.attention.store.keys.normal_()
        layer.attention.store.values.normal_()
    layer_bytes = sum(p.tensor.blocks.numel() for p in (layers[0].attention.q_proj, layers[0].attention.k_proj, layers[0].attention.v_proj, layers[0].attention.o_proj)) \
        + 8 * (2 * inter * (d // 256) * 66 + d * (inter // 256) * 56) + e * d * 4 + 2 * cache_len * a.n_kv_heads * a.head_dim * 2
    # (a) one block, decode step at position 2047: sixteen different residual rows over the eight layers
    xs = [torch.randn(1, 1, d, device=dev, dtype=torch.float16) for _ in range(16)]
    with torch.inference_mode():
        us, graphed = time_calls_us(lambda s: layers[s % n_layers](xs[s], cache_len - 1), 16)
    out.append({"case": "MiniMaxBlock.__call__ decode step, MiniMax-M2 shapes, 2048-token cache, fresh routes and weights from HBM every call",
                "weight_bytes": int(layer_bytes), "us_per_call": round(us, 3), "gbs": round(layer_bytes / us / 1e3, 1),
                "frac_hbm_peak": round(layer_bytes / us / 1e3 / HBM_PEAK_GBS, 4), "graph": graphed,
                "note": "bytes = the layer's four projections, gate, 8 routed experts and the key/value cache read once",
                "decode_tps_62_layers_blocks_only": round(1e6 / (62 * us), 2)})
    # (b) the stack: embedding -> 8 blocks -> final norm -> vocabulary projection; decode steps and a 512-token prefill
    tokens = [torch.randint(0, vocab, (1, 1), device=dev) for _ in range(16)]
    with torch.inference_mode():
        dec_us, graphed = time_calls_us(lambda s: model(tokens[s], cache_len - 1), 16, iters=64)
        prompt = torch.randint(0, vocab, (1, 512), device=dev)
        pre_us = event_time_us(lambda _s: model(prompt, 0), 1, 3, warm=1)
    head_bytes = head_blocks.numel()
    out.append({"case": "MiniMaxTransformer stack (embedding, 8 of the 62 blocks, final norm, vocabulary projection 200064 x 3072 q6_k), MiniMax-M2 shapes",
                "decode_us_per_token": round(dec_us, 2), "decode_tps": round(1e6 / dec_us, 2), "prefill_tokens": 512, "prefill_us": round(pre_us, 1),
                "prefill_tps": round(512e6 / pre_us, 1), "graph": graphed, "weight_bytes_per_token": int(n_layers * layer_bytes + head_bytes),
                "gbs": round((n_layers * layer_bytes + head_bytes) / dec_us / 1e3, 1),
                "decode_tps_62_layers_extrapolated": round(1e6 / (dec_us + (62 - n_layers) * us), 2),
                "note": "decode: one token at position 2047 against a filled cache; the 62-layer figure adds 54 more block steps at the block's measured time"})
    # the reference reports generation speed in this form (src/runtime/generation.py:262-268); the measured 8-block stack
    print(f"RESULT prefill_seconds={pre_us * 1e-6:.6f} prefill_tokens=512 prefill_tps={512e6 / pre_us:.2f} decode_seconds={dec_us * 1e-6:.6f} decode_tokens=1 "
          f"decode_tps={1e6 / dec_us:.2f}", file=sys.stderr)
    return out


F16_MFMA_PEAK_TFLOPS = 2500.0


def prefill_cases(mod, dev):
    """BASELINE configs 3 and 4 at T > 1: the MFMA tile kernel, TFLOPS = 2 T K N / t against the dense fp16 peak
    (the tiles are decoded to fp16, see the kernel's header for why)."""
    from pocketllm_amd import block_codec as C, codebooks
    rng = np.random.default_rng(4004)
    out = []
    empty = torch.empty(0, dtype=torch.int8, device=dev)
    k = 5120

    def run(label, t, n, fn):
        us, graphed = time_calls_us(fn, 4)
        tf = 2.0 * t * k * n / us / 1e6
        out.append({"case": label, "us_per_call": round(us, 3), "tflops": round(tf, 1), "frac_mfma_peak": round(tf / F16_MFMA_PEAK_TFLOPS, 4),
                    "peak": "fp16 dense 2.5 PFLOP/s", "graph": graphed})

    for name, tid, enc in (("q4_k", 3, C.quantize_q4_k), ("q5_k", 4, C.quantize_q5_k)):
        for n in (5120, 17408):
            blocks = torch.from_numpy(enc(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))).to(dev)
            for t in (32, 64, 512, 2048):
                x = torch.randn(t, k, device=dev, dtype=torch.bfloat16)
                run(f"{name} prefill {n}x{k} T={t}", t, n,
                    lambda s, x=x, blocks=blocks, tid=tid: mod.gguf_quant_gemm_prefill_forward(x, blocks, k, tid, empty))
            if n == 17408:
                # BASELINE config 3 as it is worded: activations quantized to 32-value int8 blocks, integer dots on the int8 matrix cores
                for t in (512, 2048):
                    x = torch.randn(t, k, device=dev, dtype=torch.bfloat16)
                    us, graphed = time_calls_us(lambda s, x=x, blocks=blocks, tid=tid: mod.gguf_quant_gemm_q8_forward(x, blocks, k, tid, empty), 4, iters=40)
                    tops = 2.0 * t * k * n / us / 1e6
                    out.append({"case": f"{name} int8-MFMA prefill (int8 activations) {n}x{k} T={t}", "us_per_call": round(us, 3), "tflops": round(tops, 1),
                                "frac_mfma_peak": round(tops / 5000.0, 4), "peak": "int8 dense 5.0 POP/s", "graph": graphed})
            del blocks
    n = 17408
    for name, tid in (("q6_k", 8), ("iq4_xs", 7), ("iq3_xxs", 6), ("iq2_xs", 5)):   # random valid blocks: the work does not depend on the values
        blocks = torch.from_numpy(C.random_blocks(rng, name, n, k // 256)).to(dev)
        grid = codebooks.grid_tensor_for_type(tid).to(dev)
        for t in (512, 2048):
            x = torch.randn(t, k, device=dev, dtype=torch.bfloat16)
            run(f"{name} prefill {n}x{k} T={t}", t, n,
                lambda s, x=x, blocks=blocks, tid=tid, grid=grid: mod.gguf_quant_gemm_prefill_forward(x, blocks, k, tid, grid))
        del blocks
    codes, scale = C.quantize_fp8_block(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))
    codes = torch.from_numpy(codes).to(dev)
    scale = torch.from_numpy(scale).to(dev)
    x = torch.randn(512, k, device=dev, dtype=torch.bfloat16)
    run(f"fp8_e4m3 prefill {n}x{k} T=512", 512, n, lambda s: mod.fp8_block_gemm_forward(x, codes, scale))
    # the reference's FP8 linear: act_quant (E4M3 activations, 128-wide scales) + fp8_gemm on the native FP8 matrix path
    a, a_s = mod.fp8_act_quant_forward(x)
    us, graphed = time_calls_us(lambda s: mod.fp8_gemm_forward(a, a_s, codes, scale), 4)
    usq, _ = time_calls_us(lambda s: mod.fp8_act_quant_forward(x), 4)
    tf = 2.0 * 512 * k * n / us / 1e6
    out.append({"case": f"fp8_e4m3 x fp8_e4m3 native MFMA prefill {n}x{k} T=512", "us_per_call": round(us, 3), "tflops": round(tf, 1),
                "frac_mfma_peak": round(tf / 5000.0, 4), "peak": "fp8 dense 5.0 PFLOP/s", "act_quant_us": round(usq, 3), "graph": graphed})
    return out


def pmc_pass(mod, dev) -> None:
    name, tid, n, k = CASES[DOMINANT]
    rng = np.random.default_rng(1002 + DOMINANT)
    blocks = _encoders()[name]((rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)))
    ring = ring_of(blocks, dev, 6)
    x = torch.randn(1, k, device=dev, dtype=torch.bfloat16)
    grid = torch.empty(0, dtype=torch.int8, device=dev)
    nbytes = blocks.size & ~15
    dst = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    for i in range(6):
        mod.gguf_quant_gemm_forward(x, ring[i], k, tid, grid)
    for i in range(6):
        dst.copy_(ring[i].view(-1)[:nbytes])            # the plain copy of known size the counters are scaled by (torch's copy kernel)
    torch.cuda.synchronize()
    print(json.dumps({"pmc_pass": f"{name} matvec {n}x{k}", "weight_bytes": int(blocks.size), "copy_bytes": int(nbytes)}))


def decode_pass(mod, dev) -> None:
    """A few launches of the other dense decode kernels for the profiler: Q8_0 4096x4096 and 17408x5120, FP8 17408x5120,
    Q2_K, Q6_K and IQ4_XS 17408x5120 (rings of weight copies, so that no launch finds its matrix in cache)."""
    from pocketllm_amd import block_codec as C, codebooks
    rng = np.random.default_rng(6006)
    for n, k in ((4096, 4096), (17408, 5120)):
        ring = ring_of(C.pack_q8_0((rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))), dev, 8)
        x = torch.randn(1, k, device=dev)
        for i in range(24):
            mod.q8_0_gemm_forward(x, ring[i % len(ring)], k)
        del ring
    codes, scale = C.quantize_fp8_block((rng.standard_normal((17408, 5120), dtype=np.float32) * np.float32(0.02)))
    ring = ring_of(codes, dev, 8)
    sc = torch.from_numpy(scale).to(dev)
    x = torch.randn(1, 5120, device=dev, dtype=torch.bfloat16)
    for i in range(24):
        mod.fp8_block_gemm_forward(x, ring[i % len(ring)], sc)
    del ring
    for name, tid, blocks in (("q2_k", 1, C.quantize_q2_k((rng.standard_normal((17408, 5120), dtype=np.float32) * np.float32(0.02)))),
                              ("q6_k", 8, C.random_blocks(rng, "q6_k", 17408, 20)), ("iq4_xs", 7, C.random_blocks(rng, "iq4_xs", 17408, 20))):
        ring = ring_of(blocks, dev, 8)
        grid = codebooks.grid_tensor_for_type(tid).to(dev)
        for i in range(24):
            mod.gguf_quant_gemm_forward(x, ring[i % len(ring)], 5120, tid, grid)
        del ring
    # Q4_K 17408x5120 at two rows (the two-row form of the single-launch kernel) and one token through 8 of 128 Q4_K experts of
    # 2048 -> 768 (gate / up launch, then the down projection with the routes as its waves); random valid blocks
    def q4k_random(*lead):
        b = rng.integers(0, 256, size=tuple(lead) + (144,), dtype=np.uint8)
        b[..., 0:2] = np.frombuffer(np.float16(0.01).tobytes(), dtype=np.uint8)
        b[..., 2:4] = np.frombuffer(np.float16(0.005).tobytes(), dtype=np.uint8)
        return b
    ring = ring_of(q4k_random(17408, 20), dev, 8)
    x2 = torch.randn(2, 5120, device=dev, dtype=torch.bfloat16)
    empty = torch.empty(0, dtype=torch.int8, device=dev)
    for i in range(24):
        mod.gguf_quant_gemm_forward(x2, ring[i % len(ring)], 5120, 3, empty)
    del ring
    ek, dk, ik = 128, 2048, 768
    kw1, kw3, kw2 = (torch.from_numpy(q4k_random(*shape)).to(dev) for shape in ((ek, ik, dk // 256), (ek, ik, dk // 256), (ek, dk, ik // 256)))
    xk = torch.randn(1, dk, device=dev, dtype=torch.bfloat16)
    kwts = torch.full((8,), 0.125, device=dev)
    for i in range(24):
        ids = torch.from_numpy(rng.choice(ek, size=8, replace=False).astype(np.int64)).to(dev)
        mod.gguf_moe_single_token_forward(xk, ids, kwts, kw1, kw3, kw2, 0.0)
    torch.cuda.synchronize()
    print(json.dumps({"decode_pass": "q8_0 4096x4096 + 17408x5120, fp8 17408x5120, q2_k / q6_k / iq4_xs 17408x5120, q4_k 17408x5120 at two rows, "
                                     "q4_k experts 128 x (2048 -> 768) top-8 one token; 24 launches each"}))


def few_rows_pass(mod, dev) -> None:
    """Dense calls of two to eight activation rows for the profiler, every one a single pass over its weights: Q4_K 17408x5120 at
    2, 4 and 8 float32 rows, Q6_K 17408x5120 at 4 rows and 5120x5120 at 8 rows, IQ2_XXS, IQ1_M, IQ3_XXS and IQ2_XS 17408x5120
    at 2 rows (rings of weight copies; 24 launches each)."""
    from pocketllm_amd import block_codec as C, codebooks
    rng = np.random.default_rng(8008)
    q4 = rng.integers(0, 256, size=(17408, 20, 144), dtype=np.uint8)
    q4[..., 0:2] = np.frombuffer(np.float16(0.01).tobytes(), dtype=np.uint8)
    q4[..., 2:4] = np.frombuffer(np.float16(0.005).tobytes(), dtype=np.uint8)
    cases = ((3, q4, 5120, (2, 4, 8)), (8, C.random_blocks(rng, "q6_k", 17408, 20), 5120, (4,)), (8, C.random_blocks(rng, "q6_k", 5120, 20), 5120, (8,)),
             (0, C.random_iq2_xxs(rng, 17408, 20), 5120, (2,)), (2, C.random_iq1_m(rng, 17408, 20), 5120, (2,)),
             (6, C.random_blocks(rng, "iq3_xxs", 17408, 20), 5120, (2,)), (5, C.random_blocks(rng, "iq2_xs", 17408, 20), 5120, (2,)))
    for tid, blocks, k, row_counts in cases:
        ring = ring_of(blocks, dev, 8)
        grid = codebooks.grid_tensor_for_type(tid).to(dev)
        for rows in row_counts:
            x = torch.randn(rows, k, device=dev)
            for i in range(24):
                mod.gguf_quant_gemm_forward(x, ring[i % len(ring)], k, tid, grid)
        del ring
    torch.cuda.synchronize()
    print(json.dumps({"few_rows_pass": "q4_k 17408x5120 at 2 / 4 / 8 rows, q6_k 17408x5120 at 4 and 5120x5120 at 8 rows, iq2_xxs, iq1_m, iq3_xxs and iq2_xs "
                                       "17408x5120 at 2 rows; float32 rows, 24 launches each"}))


def iq_pass(mod, dev) -> None:
    """A few launches of the codebook formats for the profiler: IQ2_XXS 98304x3072 and IQ1_M 196608x1536 matvec, then the
    single-token routed experts of the 256-expert top-8 configuration."""
    from pocketllm_amd import block_codec as C, codebooks
    rng = np.random.default_rng(5005)
    for tid, n, k, gen, grid in ((0, 64 * 1536, 3072, C.random_iq2_xxs, codebooks.get_iq2xxs_signed_grid_tensor()),
                                 (2, 64 * 3072, 1536, C.random_iq1_m, codebooks.get_iq1_grid_tensor())):
        ring = ring_of(gen(rng, n, k // 256), dev, 4)
        x = torch.randn(1, k, device=dev, dtype=torch.bfloat16)
        for i in range(8):
            mod.gguf_quant_gemm_forward(x, ring[i % len(ring)], k, tid, grid.to(dev))
        del ring
    e, d, inter = 256, 3072, 1536
    w1 = torch.from_numpy(C.random_iq2_xxs(rng, e, inter, d // 256, d_range=(0.002, 0.006))).to(dev)
    w3 = torch.from_numpy(C.random_iq2_xxs(rng, e, inter, d // 256, d_range=(0.002, 0.006))).to(dev)
    w2 = torch.from_numpy(C.random_iq1_m(rng, e, d, inter // 256, d_range=(0.002, 0.006))).to(dev)
    x = torch.randn(1, d, device=dev, dtype=torch.bfloat16)
    for _ in range(8):
        topi = torch.from_numpy(rng.choice(e, size=8, replace=False).astype(np.int64)).to(dev)
        mod.gguf_moe_single_token_forward(x, topi, torch.full((8,), 0.125, device=dev), w1, w3, w2, 0.0)
    torch.cuda.synchronize()
    print(json.dumps({"iq_pass": "iq2_xxs 98304x3072, iq1_m 196608x1536, single-token experts 256 x top-8"}))


def prefill_pass(mod, dev) -> None:
    """A few launches of the MFMA tile kernel for the profiler: Q4_K 17408x5120 at T=2048 and FP8 at T=512."""
    from pocketllm_amd import block_codec as C, codebooks
    rng = np.random.default_rng(4004)
    k, n = 5120, 17408
    empty = torch.empty(0, dtype=torch.int8, device=dev)
    blocks = torch.from_numpy(C.quantize_q4_k(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))).to(dev)
    x = torch.randn(2048, k, device=dev, dtype=torch.bfloat16)
    for _ in range(6):
        mod.gguf_quant_gemm_prefill_forward(x, blocks, k, 3, empty)
    codes, scale = C.quantize_fp8_block(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))
    codes, scale = torch.from_numpy(codes).to(dev), torch.from_numpy(scale).to(dev)
    x512 = x[:512].contiguous()
    for _ in range(6):
        mod.fp8_block_gemm_forward(x512, codes, scale)
    torch.cuda.synchronize()
    print(json.dumps({"prefill_pass": "q4_k 17408x5120 T=2048 x6, fp8 17408x5120 T=512 x6", "flops_q4k": 2.0 * 2048 * k * n, "flops_fp8": 2.0 * 512 * k * n}))


def fp8_gemm_pass(mod, dev) -> None:
    """A few launches of the native FP8 x FP8 matmul for the profiler: 17408x5120 at T=512, then at T=2048."""
    from pocketllm_amd import block_codec as C
    rng = np.random.default_rng(6006)
    k, n = 5120, 17408
    codes, scale = C.quantize_fp8_block(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))
    codes, scale = torch.from_numpy(codes).to(dev), torch.from_numpy(scale).to(dev)
    for t in (512, 2048):
        a, a_s = mod.fp8_act_quant_forward(torch.randn(t, k, device=dev, dtype=torch.bfloat16))
        for _ in range(8):
            mod.fp8_gemm_forward(a, a_s, codes, scale)
    torch.cuda.synchronize()
    print(json.dumps({"fp8_gemm_pass": "fp8 x fp8 17408x5120, T=512 x8 then T=2048 x8", "flops_512": 2.0 * 512 * k * n, "flops_2048": 2.0 * 2048 * k * n}))


def block_pass(mod, dev) -> None:
    """A few decode steps of one MiniMaxBlock for the profiler: MiniMax-M2 shapes (3072 wide, 48 / 8 heads of 128, 64 resident
    experts of the 256, top-8, Q6_K projections, IQ2_XXS / IQ1_M experts), position 2047 of a 2048-token store."""
    from pocketllm_amd import block_codec as C
    from pocketllm_amd.minimax_block import ExpertLayer, MiniMaxAttention, MiniMaxBlock, MiniMaxM2Args, MiniMaxMoE, RMSNorm
    from pocketllm_amd.quantized_ops import QuantizedGGUFLinear
    from pocketllm_amd.quantized_tensor import QuantizedGGUFTensor
    rng = np.random.default_rng(9009)
    e, d, inter = 64, 3072, 1536
    a = MiniMaxM2Args(dim=d, n_heads=48, n_kv_heads=8, head_dim=128, rope_dim=64, rope_base=5.0e6, n_routed_experts=e, top_k=8,
                      moe_inter_dim=inter, norm_eps=1e-6)

    def lin(n, k):
        return QuantizedGGUFLinear(QuantizedGGUFTensor.from_blocks(torch.from_numpy(C.random_blocks(rng, "q6_k", n, k // 256)).to(dev), "q6_k", k))

    w1 = torch.from_numpy(C.random_iq2_xxs(rng, e, inter, d // 256, d_range=(0.002, 0.006))).to(dev)
    w3 = torch.from_numpy(C.random_iq2_xxs(rng, e, inter, d // 256, d_range=(0.002, 0.006))).to(dev)
    w2 = torch.from_numpy(C.random_iq1_m(rng, e, d, inter // 256, d_range=(0.002, 0.006))).to(dev)
    experts = ExpertLayer(*(QuantizedGGUFTensor.from_blocks(t, n, k) for t, n, k in ((w1, "iq2_xxs", d), (w3, "iq2_xxs", d), (w2, "iq1_m", inter))))
    moe = MiniMaxMoE(a, torch.randn(e, d, device=dev) * d ** -0.5, torch.zeros(e, device=dev), experts)
    attn = MiniMaxAttention(a, lin(6144, d), lin(1024, d), lin(1024, d), lin(d, 6144), RMSNorm(torch.ones(6144, device=dev), 1e-6),
                            RMSNorm(torch.ones(1024, device=dev), 1e-6))
    blk = MiniMaxBlock(a, torch.ones(d, device=dev), torch.ones(d, device=dev), attn, moe)
    blk.reset_cache(1, 2048)
    blk.attention.store.keys.normal_()
    blk.attention.store.values.normal_()
    x = torch.randn(1, 1, d, device=dev, dtype=torch.float16)
    with torch.inference_mode():
        for _ in range(12):
            blk(x, 2047)
    torch.cuda.synchronize()
    print(json.dumps({"block_pass": "MiniMaxBlock decode step at position 2047, 12 steps, one token"}))


def experts_rows_pass(mod, dev) -> None:
    """A few launches of the grouped routed experts for the profiler: 256 tokens, 256 resident experts, top-8 (2048 routes),
    IQ2_XXS gate/up 1536x3072 and IQ1_M down 3072x1536."""
    from pocketllm_amd import block_codec as C, codebooks
    rng = np.random.default_rng(7007)
    e, d, inter, t = 256, 3072, 1536, 256
    w1 = torch.from_numpy(C.random_iq2_xxs(rng, e, inter, d // 256, d_range=(0.002, 0.006))).to(dev)
    w3 = torch.from_numpy(C.random_iq2_xxs(rng, e, inter, d // 256, d_range=(0.002, 0.006))).to(dev)
    w2 = torch.from_numpy(C.random_iq1_m(rng, e, d, inter // 256, d_range=(0.002, 0.006))).to(dev)
    logits = torch.from_numpy(rng.standard_normal((t, e)).astype(np.float32))
    tw, ti = torch.softmax(logits, dim=-1).topk(8, dim=-1)
    tw = (tw / tw.sum(dim=-1, keepdim=True)).to(dev)
    _, toks, rws, seg = mod.moe_group_routes(ti.to(dev), tw, 0, e)
    touched = int((seg[1:] > seg[:-1]).sum().item())
    xt = torch.randn(t, d, device=dev, dtype=torch.bfloat16)
    grids = (codebooks.get_iq2xxs_signed_grid_tensor().to(dev), codebooks.get_iq1_grid_tensor().to(dev))
    for _ in range(6):
        mod.gguf_moe_prefill_grouped_forward(xt, toks, rws, seg, w1, w3, w2, d, 0, d, 0, inter, 2, grids, 0.0)
    torch.cuda.synchronize()
    print(json.dumps({"experts_rows_pass": "iq2_xxs gate/up + iq1_m down, 256 experts top-8, T=256, 6 calls", "experts_touched": touched,
                      "weight_bytes": touched * (2 * inter * (d // 256) * 66 + d * (inter // 256) * 56), "flops": 2.0 * t * 8 * 3 * inter * d}))


def q8_gemm_pass(mod, dev) -> None:
    """A few launches for the profiler of the two prefill forms that the streamed decode and tile kernels do not cover: the
    int8-MFMA matmul on int8-quantized activations (Q4_K 17408x5120 at T=512 and T=2048) and the 17 - 48 row kernel (Q4_K and
    Q5_K 5120x5120 and 17408x5120 at T=32)."""
    from pocketllm_amd import block_codec as C
    rng = np.random.default_rng(8008)
    k = 5120
    empty = torch.empty(0, dtype=torch.int8, device=dev)
    for n in (5120, 17408):
        w = rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)
        for tid, enc in ((3, C.quantize_q4_k), (4, C.quantize_q5_k)):
            blocks = torch.from_numpy(enc(w)).to(dev)
            x = torch.randn(32, k, device=dev, dtype=torch.bfloat16)
            for _ in range(8):
                mod.gguf_quant_gemm_prefill_forward(x, blocks, k, tid, empty)
            if n == 17408 and tid == 3:
                for t in (512, 2048):
                    xt = torch.randn(t, k, device=dev, dtype=torch.bfloat16)
                    for _ in range(6):
                        mod.gguf_quant_gemm_q8_forward(xt, blocks, k, tid, empty)
            del blocks
    torch.cuda.synchronize()
    print(json.dumps({"q8_gemm_pass": "q4_k / q5_k 5120x5120 and 17408x5120 at T=32 x8; q4_k 17408x5120 int8 activations T=512 x6, T=2048 x6",
                      "ops_512": 2.0 * 512 * k * 17408, "ops_2048": 2.0 * 2048 * k * 17408}))


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240, help="timed steps (run exactly, five times over; the median is reported)")
    ap.add_argument("--warmup", type=int, default=24)
    ap.add_argument("--eager", action="store_true", help="time plain operator calls instead of graph replays")
    ap.add_argument("--no-extra", action="store_true", help="skip the table of other formats")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-pass", action="store_true", help="short run for rocprofv3 --pmc: dominant kernel + a copy of the same size")
    ap.add_argument("--prefill-pass", action="store_true", help="short run for rocprofv3: a few launches of the MFMA tile kernel")
    ap.add_argument("--decode-pass", action="store_true", help="short run for rocprofv3: Q8_0, FP8, Q2_K, Q6_K and IQ4_XS decode matvec")
    ap.add_argument("--fp8-gemm-pass", action="store_true", help="short run for rocprofv3: native FP8 x FP8 matmul at T=512 and T=2048")
    ap.add_argument("--few-rows-pass", action="store_true", help="short run for rocprofv3: dense calls of two to eight rows in one pass over the weights")
    ap.add_argument("--iq-pass", action="store_true", help="short run for rocprofv3: IQ2_XXS / IQ1_M matvec and the single-token experts")
    ap.add_argument("--experts-rows-pass", action="store_true", help="short run for rocprofv3: grouped routed experts at T=256")
    ap.add_argument("--block-pass", action="store_true", help="short run for rocprofv3: decode steps of one MiniMaxBlock")
    ap.add_argument("--q8-gemm-pass", action="store_true", help="short run for rocprofv3: int8-activation matmul at T=512 / 2048 and the 17 - 48 row kernel at T=32")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU (no sharding, no collectives); run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")

    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from pocketllm_amd.cuda_loader import load_cuda_kernel
    mod = load_cuda_kernel()
    if mod is None:
        sys.exit("bench.py: libpllm_hip.so is not built (python -c 'import __graft_entry__ as g; g.build()')")

    dev = torch.device("cuda:0")
    grid = torch.empty(0, dtype=torch.int8, device=dev)
    if args.pmc_pass:
        pmc_pass(mod, dev)
        return
    if args.prefill_pass:
        prefill_pass(mod, dev)
        return
    if args.decode_pass:
        decode_pass(mod, dev)
        return
    if args.few_rows_pass:
        few_rows_pass(mod, dev)
        return
    if args.iq_pass:
        iq_pass(mod, dev)
        return
    if args.fp8_gemm_pass:
        fp8_gemm_pass(mod, dev)
        return
    if args.experts_rows_pass:
        experts_rows_pass(mod, dev)
        return
    if args.block_pass:
        block_pass(mod, dev)
        return
    if args.q8_gemm_pass:
        q8_gemm_pass(mod, dev)
        return
    x_np = np.random.default_rng(2002).standard_normal((1, 5120), dtype=np.float32)
    x = torch.from_numpy(x_np).to(dev).to(torch.bfloat16)

    rings, host_blocks, fns = [], [], []
    for idx, (name, tid, n, k) in enumerate(CASES):
        rng = np.random.default_rng(1002 + idx)
        blocks = _encoders()[name]((rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)))
        host_blocks.append(blocks)
        rings.append(ring_of(blocks, dev, ring_copies(blocks.size, RING)))
        fns.append(lambda s, ring=rings[-1], tid=tid, k=k: mod.gguf_quant_gemm_forward(x, ring[s % len(ring)], k, tid, grid))
    step_bytes = sum(b.size for b in host_blocks)

    def step_eager(s):
        for fn in fns:
            fn(s)

    # Exactly --warmup untimed steps, then exactly --steps timed steps, REPEATS times over; the median repeat is reported.
    # Graph mode: one graph holds a chunk of consecutive steps (every step on the next ring slot); whole chunks are replayed
    # and a second graph holds the remainder, so that the number of steps run is the number asked for.
    chunk = min(args.steps, 4 * RING)
    replay, graphed = (None, False) if args.eager else capture(step_eager, chunk)
    rest = args.steps % chunk
    replay_rest = None
    if graphed and rest:
        replay_rest, ok = capture(step_eager, rest)
        graphed = graphed and ok
    for i in range(args.warmup):
        step_eager(i)
    torch.cuda.synchronize()
    repeats = []
    for _ in range(REPEATS):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if graphed:
            for _c in range(args.steps // chunk):
                replay()
            if replay_rest:
                replay_rest()
        else:
            for i in range(args.steps):
                step_eager(args.warmup + i)
        torch.cuda.synchronize()
        repeats.append(time.perf_counter() - t0)
    elapsed = float(np.median(repeats))
    ms_per_step = elapsed * 1e3 / args.steps
    value = step_bytes / (elapsed / args.steps) / 1e9

    # per-case launch durations with HIP events on the launch stream (torch's current stream): every case on its own ring of
    # at least 512 MB of weight copies, at least 200 launches per repeat, median of 5 repeats
    cases = []
    for (name, tid, n, k), fn, blocks, ring in zip(CASES, fns, host_blocks, rings):
        us, g = time_calls_us(fn, len(ring), eager=args.eager)
        hot, _ = time_calls_us(lambda _s, fn=fn: fn(0), RING, eager=args.eager)
        cases.append({"case": f"{name} matvec {n}x{k} T=1", "weight_bytes": int(blocks.size), "us_per_call": round(us, 3),
                      "gbs": round(blocks.size / us / 1e3, 1), "frac_hbm_peak": round(blocks.size / us / 1e3 / HBM_PEAK_GBS, 4),
                      "us_per_call_cache_hot": round(hot, 3), "ring_copies": len(ring), "graph": g})
    dom = cases[DOMINANT]
    # The roofline object describes the dominant launch of the step: the Q5_K 17408x5120 operator call, which is ONE kernel (every
    # wave quantizes the activation slices of its own blocks while its weights are in flight), so its event-timed duration above
    # is the kernel's launch duration.  The same matrix on a prepared activation image (the kernel behind calls of several rows)
    # is timed beside it.
    d_name, d_tid, d_n, d_k = CASES[DOMINANT]
    image = mod.quantize_activations(x, d_k // 256)
    d_ring = rings[DOMINANT]
    image_us, _ = time_calls_us(lambda s: mod.gguf_quant_gemm_prequantized(image, d_ring[s], d_tid), len(d_ring), eager=args.eager)
    kernel_us = dom["us_per_call"]
    kernel_gbs = host_blocks[DOMINANT].size / kernel_us / 1e3
    traffic, traced_us = None, None
    if os.path.exists(TRAFFIC_FILE):
        with open(TRAFFIC_FILE) as f:
            recorded = json.load(f)
        traffic = recorded.get("q5_k matvec 17408x5120 T=1")
        traced_us = recorded.get("q5_k matvec 17408x5120 T=1 rocprofv3 kernel-trace avg us")
    roofline = {"bound": "hbm", "achieved": round(kernel_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(kernel_gbs / HBM_PEAK_GBS, 4), "traffic": traffic,
                "traffic_source": "profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE of an earlier run, not measured in this run",
                "kernel": "wave_image_matvec_kernel<Q5K, 5, 4, true, false> = the q5_k matvec 17408x5120 operator call (one launch, activations quantized in the kernel)",
                "bytes_per_launch": dom["weight_bytes"], "us_per_launch": round(kernel_us, 3),
                "us_per_launch_on_prepared_image": round(image_us, 3),
                # begin-to-end duration of the same kernel in the committed kernel trace (profiles/): the event-timed figure above is
                # the period of back-to-back launches and carries the gap between graph nodes
                "us_per_launch_in_committed_kernel_trace": traced_us,
                "timed_launches_per_repeat": max(MIN_TIMED_LAUNCHES, len(d_ring)), "repeats": REPEATS}

    # parity of what was just timed, against the float-activation oracle (small case only: seconds)
    from oracle import gguf_oracle as O
    y_gpu = mod.gguf_quant_gemm_forward(x, rings[0][0], 5120, 3, grid, out_dtype=torch.float32).cpu().numpy()
    want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(host_blocks[0], "q4_k", 5120))
    parity = O.rel_l2(y_gpu, want)

    cpu, cpu_more = None, []
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(host_blocks[0], "q4_k", 5120, x.float().cpu().numpy())
        cpu_more = cpu_baselines_more(host_blocks[0], x.float().cpu().numpy())
    del rings, d_ring
    torch.cuda.empty_cache()
    headline = {c["case"]: {"us": c["us_per_call"], "frac": c["frac_hbm_peak"]} for c in cases}
    if not args.no_extra:
        cases += extra_cases(mod, dev)
    # the full table goes to stderr; the one line on stdout keeps the records of the BASELINE configurations
    print("bench.py all cases: " + json.dumps(cases), file=sys.stderr)
    keep = ("q4_k matvec", "q5_k matvec", "q8_0 matvec", "fp8_e4m3 matvec 17408x5120 T=1", "fused experts", "q4_k prefill", "q5_k prefill",
            "q4_k int8-MFMA", "q5_k int8-MFMA", "fp8_e4m3 prefill", "fp8_e4m3 x fp8_e4m3", "iq2_xxs matvec", "iq1_m matvec", "q2_k matvec",
            "MiniMaxBlock", "MiniMaxTransformer")
    short = [{k2: v for k2, v in c.items() if k2 in ("case", "us_per_call", "gbs", "frac_hbm_peak", "tflops", "frac_mfma_peak", "peak", "decode_tps", "prefill_tps",
                                                     "decode_us_per_token", "decode_tps_62_layers_blocks_only", "decode_tps_62_layers_extrapolated")}
             for c in cases if c["case"].startswith(keep)]

    out = {
        "metric": "decode matvec effective HBM GB/s (% of peak) + prefill TFLOPS, per quant type",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 dot (two int8 activation terms), f32 accumulate",
        "data": "synthetic (seeded N(0,0.02) weights quantized to Q4_K/Q5_K blocks, N(0,1) bf16 activations)",
        "config": {"workload": "BASELINE config 2: Q4_K + Q5_K decode matvec, 5120x5120 and 17408x5120, T=1, each case on a ring of >= 512 MB of weight copies",
                   "bytes_per_step": int(step_bytes), "calls_per_step": len(CASES), "hip_graph_replay": graphed,
                   "repeats": REPEATS, "ms_per_step_repeats": [round(r * 1e3 / args.steps, 5) for r in repeats],
                   "headline_cases": headline},
        "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "roofline": roofline,
        "cpu_baseline": cpu,
        "cpu_baselines_more": cpu_more,
        "cases": short,
        "parity_rel_l2_vs_float_oracle": parity,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
