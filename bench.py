#!/usr/bin/env python3
"""Benchmark of the raw-block quantized matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the decode matvec over the Q4_K / Q5_K weights of the Qwen3-27B-like shapes
(N x K = 5120 x 5120 and 17408 x 5120, one bf16 activation row): four operator calls, each on the
next copy in a ring of weight copies larger than the 256 MB last-level cache, so the bytes come from
HBM.  Inputs are synthetic (seeded N(0, 0.02) weights quantized by this package's encoders, N(0, 1)
activations) and resident in HBM before the timed region.  The one JSON line printed at the end
carries whole-step throughput (weight bytes / time), the roofline figures of the dominant kernel
measured with HIP events on the launch stream, and the CPU dequantize-then-matmul baseline.
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
RING_BYTES = 640 << 20

CASES = [  # (type name, type id, N, K)
    ("q4_k", 3, 5120, 5120),
    ("q4_k", 3, 17408, 5120),
    ("q5_k", 4, 5120, 5120),
    ("q5_k", 4, 17408, 5120),
]
DOMINANT = 3   # index into CASES: the launch the roofline object describes


def _encoders():
    from pocketllm_amd import block_codec as C
    return {"q4_k": C.quantize_q4_k, "q5_k": C.quantize_q5_k}


def build_case(name, n, k, seed, device):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))
    blocks = _encoders()[name](w)
    first = torch.from_numpy(blocks).to(device)
    copies = max(2, -(-RING_BYTES // first.numel()))
    ring = [first] + [first.clone() for _ in range(copies - 1)]
    return blocks, ring


def event_time_us(fn, ring, iters, warm):
    for i in range(warm):
        fn(ring[i % len(ring)])
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(iters):
        fn(ring[i % len(ring)])
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters


def cpu_baseline(blocks: np.ndarray, type_name: str, k: int, x: np.ndarray, budget_s: float = 15.0):
    """The reference's CPU path restated: numpy block decode to float32, then torch matmul."""
    from oracle import gguf_oracle as O
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    xt = torch.from_numpy(x.astype(np.float32))
    times = []
    t_begin = time.perf_counter()
    while len(times) < 5 and (time.perf_counter() - t_begin < budget_s or len(times) < 2):
        t0 = time.perf_counter()
        w = O.dequant_rows(blocks, type_name, k)
        t1 = time.perf_counter()
        y = torch.nn.functional.linear(xt, torch.from_numpy(w))
        t2 = time.perf_counter()
        times.append((t2 - t0, t1 - t0, t2 - t1))
    times = times[1:] if len(times) > 1 else times          # first call warms the page cache
    total = float(np.median([t[0] for t in times]))
    return {
        "value": blocks.size / total / 1e9,
        "unit": "GB/s",
        "cores": int(torch.get_num_threads()),
        "kind": "port",
        "sample": (f"{type_name} {blocks.shape[0]}x{k} matvec, numpy block decode ({np.median([t[1] for t in times]) * 1e3:.0f} ms, "
                   f"one thread) + torch F.linear fp32 ({np.median([t[2] for t in times]) * 1e3:.1f} ms, {torch.get_num_threads()} threads), "
                   f"median of {len(times)} calls"),
        "ms_per_call": total * 1e3,
    }, y.numpy()


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
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
    x_np = np.random.default_rng(2002).standard_normal((1, 5120), dtype=np.float32)
    x = torch.from_numpy(x_np).to(dev).to(torch.bfloat16)

    rings, host_blocks, fns = [], [], []
    for idx, (name, tid, n, k) in enumerate(CASES):
        blocks, ring = build_case(name, n, k, 1002 + idx, dev)
        host_blocks.append(blocks)
        rings.append(ring)
        fns.append(lambda b, tid=tid, k=k: mod.gguf_quant_gemm_forward(x, b, k, tid, grid))
    step_bytes = sum(b.size for b in host_blocks)

    def step(i):
        for ring, fn in zip(rings, fns):
            fn(ring[i % len(ring)])

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(args.warmup + i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    value = step_bytes / (elapsed / args.steps) / 1e9

    # per-case launch durations with HIP events on the launch stream (torch's current stream)
    cases = []
    for (name, tid, n, k), ring, fn, blocks in zip(CASES, rings, fns, host_blocks):
        us = event_time_us(fn, ring, max(50, args.steps), 10)
        hot = event_time_us(fn, ring[:1], max(50, args.steps), 10)
        cases.append({"type": name, "n": n, "k": k, "t": 1, "weight_bytes": int(blocks.size), "us_per_call": round(us, 3),
                      "gbs": round(blocks.size / us / 1e3, 1), "frac_hbm_peak": round(blocks.size / us / 1e3 / HBM_PEAK_GBS, 4),
                      "us_per_call_cache_hot": round(hot, 3)})
    dom = cases[DOMINANT]
    roofline = {"bound": "hbm", "achieved": dom["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(dom["gbs"] / HBM_PEAK_GBS, 4), "traffic": None,
                "kernel": f"{dom['type']} matvec {dom['n']}x{dom['k']}", "bytes_per_launch": dom["weight_bytes"],
                "us_per_launch": dom["us_per_call"]}

    # parity of what was just timed, against the float-activation oracle (small case only: seconds)
    from oracle import gguf_oracle as O
    y_gpu = mod.gguf_quant_gemm_forward(x, rings[0][0], 5120, 3, grid, out_dtype=torch.float32).cpu().numpy()
    want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(host_blocks[0], "q4_k", 5120))
    parity = O.rel_l2(y_gpu, want)

    cpu = None
    if not args.no_cpu_baseline:
        cpu, _ = cpu_baseline(host_blocks[0], "q4_k", 5120, x.float().cpu().numpy())

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
        "dtype": "int8 dot, f32 accumulate",
        "data": "synthetic (seeded N(0,0.02) weights quantized to Q4_K/Q5_K blocks, N(0,1) bf16 activations)",
        "config": {"workload": "Q4_K + Q5_K decode matvec, N x K = 5120x5120 and 17408x5120, T=1, weights rotated through a "
                               f"{RING_BYTES >> 20} MiB ring per case",
                   "bytes_per_step": int(step_bytes), "calls_per_step": len(CASES)},
        "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "roofline": roofline,
        "cpu_baseline": cpu,
        "cases": cases,
        "parity_rel_l2_vs_float_oracle": parity,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
