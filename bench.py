#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

Default workload (`decode_gemv`): BASELINE.json config 2 -- one decode token's
dense projections, batch 1, bf16 activations N(0,1):
    gate, up : Q4_K 12288 x 4096        down : Q4_K 4096 x 12288
    head     : Q6_K 151936 x 4096
Weights are seeded N(0, 0.02) f32 generated on the device and quantized by the
library's own quantizer (byte-identical to hf2q's CPU quantizers).  One "step"
is one pass over those four GEMVs.  Several distinct weight sets are rotated so
that no step finds its weights in the 256 MB Infinity Cache.

Prints ONE JSON line: metric = effective GB/s of packed weight bytes, with a
`roofline` object for the dominant kernel (the Q6_K head GEMV) from HIP-event
timings taken inside the timed region, a `kernels` table for the others, and a
`cpu_baseline` object (the scalar CPU port of hf2q's quantize -> dequantize ->
scalar matmul, timed on this host).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E peak


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="decode_gemv", choices=["decode_gemv"])
    ap.add_argument("--weight-sets", type=int, default=4, help="distinct FFN weight sets rotated per step")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    return ap.parse_args()


def cpu_baseline() -> dict:
    """hf2q's CPU path on BASELINE config 1 (Q4_K 4096x4096): quantize, dequantize, scalar f32 GEMV.
    This is the only place the benchmark touches the oracle: it is what is being timed here."""
    import numpy as np

    import oracle

    oracle.build()
    rng = np.random.default_rng(1234)
    n = k = 4096
    w = rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)
    x = np.random.default_rng(5678).standard_normal((1, k), dtype=np.float32)
    t0 = time.perf_counter()
    blocks = oracle.quantize(w, k, oracle.Q4_K, threads=1)
    t_quant = time.perf_counter() - t0
    reps = 10
    t0 = time.perf_counter()
    for _ in range(reps):
        wd = oracle.dequantize(blocks, oracle.Q4_K, threads=1)
    t_deq = (time.perf_counter() - t0) / reps
    t0 = time.perf_counter()
    for _ in range(reps):
        oracle.matmul_a_by_bt(x, wd, 1, k, n, threads=1)
    t_gemv = (time.perf_counter() - t0) / reps
    cores = os.cpu_count() or 1
    nt = min(cores, 16)
    t0 = time.perf_counter()
    for _ in range(reps):
        wd = oracle.dequantize(blocks, oracle.Q4_K, threads=nt)
        oracle.matmul_a_by_bt(x, wd, 1, k, n, threads=nt)
    t_mt = (time.perf_counter() - t0) / reps
    nbytes = blocks.size
    return {
        "value": round(nbytes / (t_deq + t_gemv) / 1e9, 4),
        "unit": "GB/s",
        "cores": 1,
        "kind": "port",
        "sample": (f"BASELINE config 1: Q4_K 4096x4096 ({nbytes} packed bytes), scalar C port of hf2q's CPU path, "
                   f"1 thread: quantize once {t_quant:.2f} s (set-up, not in value), then {reps}x "
                   f"[dequantize {t_deq * 1e3:.1f} ms + scalar f32 GEMV {t_gemv * 1e3:.2f} ms]; value = packed "
                   f"bytes / (dequantize + GEMV)"),
        "quantize_s": round(t_quant, 3),
        "dequant_ms": round(t_deq * 1e3, 3),
        "gemv_ms": round(t_gemv * 1e3, 3),
        "row_parallel": {"threads": nt, "host_cores": cores, "dequant_plus_gemv_ms": round(t_mt * 1e3, 3),
                         "value": round(nbytes / t_mt / 1e9, 4), "unit": "GB/s"},
    }


def main():
    a = parse()
    if a.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU (asked for --gpus {a.gpus}); the path is single-GPU by "
              "construction, there is no multi-GPU figure to report", file=sys.stderr)
        sys.exit(2)

    import torch

    from hf2q_amd import ops
    from hf2q_amd.ops import HQ_Q4_K, HQ_Q6_K, GgmlQuantizedMatmulParams

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    H, F, V = 4096, 12288, 151936
    shapes = {  # name -> (n, k, type)
        "gate": (F, H, HQ_Q4_K), "up": (F, H, HQ_Q4_K), "down": (H, F, HQ_Q4_K), "head": (V, H, HQ_Q6_K),
    }
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)

    def make_weight(n, k, t):
        w = torch.randn(n * k, generator=gen, device=dev, dtype=torch.float32).mul_(0.02)
        q = ops.quantize_ggml(w, k, t)
        del w
        return q

    n_sets = max(1, a.weight_sets)
    n_heads = 2
    sets = []
    for s in range(n_sets):
        sets.append({nm: make_weight(*shapes[nm]) for nm in ("gate", "up", "down")})
    heads = [make_weight(*shapes["head"]) for _ in range(n_heads)]
    torch.cuda.synchronize()

    gx = torch.Generator(device=dev)
    gx.manual_seed(5678)
    x_h = torch.randn(1, H, generator=gx, device=dev, dtype=torch.float32).to(torch.bfloat16)
    x_f = torch.randn(1, F, generator=gx, device=dev, dtype=torch.float32).to(torch.bfloat16)
    y = {nm: torch.empty(1, shapes[nm][0], device=dev, dtype=torch.float32) for nm in shapes}
    params = {nm: GgmlQuantizedMatmulParams(1, n, k, t) for nm, (n, k, t) in shapes.items()}
    nbytes = {nm: sets[0][nm].numel() if nm != "head" else heads[0].numel() for nm in shapes}
    step_bytes = sum(nbytes.values())

    def step(i, ev=None):
        ws = sets[i % n_sets]
        for j, nm in enumerate(("gate", "up", "down", "head")):
            w = heads[i % n_heads] if nm == "head" else ws[nm]
            xin = x_f if nm == "down" else x_h
            if ev is not None:
                ev[j][0].record()
            ops.quantized_matmul_ggml(xin, w, y[nm], params[nm])
            if ev is not None:
                ev[j][1].record()

    for i in range(a.warmup):
        step(i)
    torch.cuda.synchronize()

    # timed region: exactly K steps, with a HIP event pair around every kernel (same stream)
    evs = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(4)]
           for _ in range(a.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(a.warmup + i, evs[i])
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    names = ("gate", "up", "down", "head")
    kern_us = {nm: sum(evs[i][j][0].elapsed_time(evs[i][j][1]) for i in range(a.steps)) * 1e3 / a.steps
               for j, nm in enumerate(names)}
    kernels = {nm: {"us": round(kern_us[nm], 3), "bytes": nbytes[nm],
                    "GBps": round(nbytes[nm] / kern_us[nm] / 1e3, 1),
                    "frac_hbm_peak": round(nbytes[nm] / kern_us[nm] / 1e3 / HBM_PEAK_GBS, 4)} for nm in names}
    q4_bytes = nbytes["gate"] + nbytes["up"] + nbytes["down"]
    q4_us = kern_us["gate"] + kern_us["up"] + kern_us["down"]

    value = step_bytes * a.steps / elapsed / 1e9
    head_gbs = nbytes["head"] / kern_us["head"] / 1e3
    out = {
        "metric": "Q4_K/Q6_K GEMV eff. GB/s (% HBM peak)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(elapsed / a.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "decode_gemv: gate/up Q4_K 12288x4096, down Q4_K 4096x12288, head Q6_K 151936x4096, "
                               "batch 1, bf16 activations (BASELINE config 2)",
                   "bytes_per_step": step_bytes, "weight_sets": n_sets, "head_copies": n_heads,
                   "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4)},
        "roofline": {"bound": "hbm", "kernel": "gemv Q6_K head 151936x4096", "achieved": round(head_gbs, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(head_gbs / HBM_PEAK_GBS, 4),
                     "traffic": None, "us_per_launch": round(kern_us["head"], 3), "bytes_per_launch": nbytes["head"]},
        "kernels": kernels,
        "q4_k_gemv": {"GBps": round(q4_bytes / q4_us / 1e3, 1), "frac_hbm_peak": round(q4_bytes / q4_us / 1e3 / HBM_PEAK_GBS, 4)},
    }
    out["cpu_baseline"] = None if a.no_cpu_baseline else cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
