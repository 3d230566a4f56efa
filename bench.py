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

The K timed steps behind `value` are replayed from HIP graphs after the W warm-up
steps, a run of further untimed steps and the per-kernel measurements: the device
takes 100-200 ms of continuous work to reach its steady rate (the same K steps
timed right after set-up are reported as `config.us_per_step_first_region`).

Prints ONE JSON line: metric = effective GB/s of packed weight bytes, with a
`roofline` object for the dominant kernel (the Q6_K head GEMV) from HIP event
pairs around every head launch of host-launched steps, a `kernels` table for the others
(back-to-back launches of one kind, medians over graph replays), a
`workloads` object with the other BASELINE configurations (MoE decode at 1 and 8
tokens, its prefill-sized grouped mul_mat_id, the Q4_K and Q8_0 prefill GEMM, the
TQ attention), each with its own
roofline, and a `cpu_baseline` object (the scalar CPU port of hf2q's
quantize -> dequantize -> scalar matmul, timed on this host).
`--workload <name>` runs one of them alone and prints its own line.
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
SETTLE_STEPS = 2400  # untimed decode steps before the steady-state measurements of the decode workload (about 0.25 s)

# HBM bytes per launch of the dominant kernel of each workload, from rocprofv3 --pmc runs of this
# file (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter reads
# for a device copy of known size (--calibration-copy): FETCH_SIZE reads half the bytes (factor
# 2.0), WRITE_SIZE all of them (1.0).  The runs and their figures are in profiles/*_pmc_traffic.md.
PMC_TRAFFIC_BYTES = {
    # (FETCH_SIZE KiB x 2.0 + WRITE_SIZE KiB x 1.0) x 1024 per dispatch
    "gemv_head_q6_k_151936x4096": int(254476.8 * 2.0 * 1024 + 1187.0 * 1.0 * 1024),
    # activation pre-pass + tile GEMM, Q4_K, 2048 x 12288 x 4096 (the GEMM re-fetches the weights once per 256-token tile)
    "prefill_gemm_q4_k_2048x12288x4096": int((23301.6 + 132573.1) * 2.0 * 1024 + (16496.5 + 98311.8) * 1.0 * 1024),
    # split (with the q rotation) + merge (with the output rotation), 32K context, 2 kv heads, head_dim 256
    "tq_attention_32k_fused_chain": int((16897.5 + 1072.5) * 2.0 * 1024 + (2112.0 + 16.0) * 1.0 * 1024),
    # the one-launch MoE FFN block, hidden 2048, 256 experts x 512, top-8, 1 and 8 tokens
    "moe_ffn_decode_t1": int(8698.0 * 2.0 * 1024 + 108.3 * 1.0 * 1024),
    "moe_ffn_decode_t8": int(63320.4 * 2.0 * 1024 + 866.5 * 1.0 * 1024),
    # the same block with gate / up in Q5_K and down in Q6_K
    "moe_ffn_decode_t1_q5k_q6k": int(11157.5 * 2.0 * 1024 + 108.3 * 1.0 * 1024),
    "moe_ffn_decode_t8_q5k_q6k": int(82141.3 * 2.0 * 1024 + 866.5 * 1.0 * 1024),
    # Q8_0, 2048 x 12288 x 4096: tile GEMM + the plain call's pre-pass (that one worked out of a run that mixes plain and
    # kept-scales calls 1 : 2: 68,804 KiB fetched for the activations and every line of the weights, 16,464 written)
    "prefill_gemm_q8_0_2048x12288x4096": int((232529.5 + 68804.0 / 2.0) * 2.0 * 1024 + (98572.3 + 16464.2) * 1.0 * 1024),
    # grouped mul_mat_id, 2048 tokens x top-8 over 256 experts of 512 x 2048 Q4_K: pre-pass (sort, conversion, scan of the stack's
    # headers) + grouped tile GEMM (bench.py --workload moe_prefill --step-only)
    "moe_prefill_gate_up_2048x8": int((106321.0 + 69719.0) * 2.0 * 1024 + (32940.8 + 8788.0) * 1.0 * 1024),
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all",
                    choices=["all", "decode_gemv", "moe_decode", "moe_prefill", "prefill_gemm", "tq_attention"],
                    help="all (default) = the BASELINE config 2 headline plus configs 3, 4 and 5 under `workloads` in the "
                         "same JSON line; a single name runs that workload alone and prints its own line")
    ap.add_argument("--tokens", type=int, default=1, help="moe_decode: tokens per step (1 or 8)")
    ap.add_argument("--mix", action="store_true", help="moe_decode: gate / up Q5_K and down Q6_K instead of Q4_K")
    ap.add_argument("--wtype", default="q4_k", choices=["q4_k", "q8_0", "q6_k", "q5_k", "q4_0"], help="prefill_gemm: weight type")
    ap.add_argument("--weight-sets", type=int, default=6, help="distinct FFN weight sets rotated per step")
    ap.add_argument("--moe-layers", type=int, default=20, help="moe_decode: distinct MoE layers rotated per step")
    ap.add_argument("--no-graph", action="store_true",
                    help="moe_decode / moe_prefill / tq_attention: launch every kernel from the host instead of replaying a HIP "
                         "graph of the step (the steps are 4-12 launches of a few microseconds each)")
    ap.add_argument("--step-only", action="store_true", help="moe_prefill: only the workload's own step (the gate / up call)")
    ap.add_argument("--block-only", action="store_true",
                    help="moe_prefill: run only the whole-block part (for a kernel trace of the block's launches alone)")
    ap.add_argument("--kept-scales", action="store_true",
                    help="moe_prefill --block-only: the block with its weight-row scales kept from load time")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run three 256 MiB device-to-device copies first: the known-size kernel that scales "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run of this file")
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


def cpu_baselines_by_config() -> dict:
    """hf2q's CPU path (dequantize + scalar f32 matmul, ffn.rs:38-50; the scalar MoE block, ffn.rs:179-336) on bounded samples
    of BASELINE configs 2-5, one thread, in each config's own unit; a few seconds each.  The oracle is what is timed here."""
    import numpy as np

    import oracle

    oracle.build()
    rng = np.random.default_rng(1234)
    out = {}

    def gemv(n_full, k, t, rows, name):
        w = rng.standard_normal((rows, k), dtype=np.float32) * np.float32(0.02)
        x = np.random.default_rng(5678).standard_normal((1, k), dtype=np.float32)
        blocks = oracle.quantize(w, k, t, threads=min(os.cpu_count() or 1, 16))
        wd = oracle.dequantize(blocks, t, threads=1)  # (untimed: the first call pays for the pages of its output)
        reps = 3
        t0 = time.perf_counter()
        for _ in range(reps):
            wd = oracle.dequantize(blocks, t, threads=1)
        t_deq = (time.perf_counter() - t0) / reps
        t0 = time.perf_counter()
        for _ in range(reps):
            oracle.matmul_a_by_bt(x, wd, 1, k, rows, threads=1)
        t_mm = (time.perf_counter() - t0) / reps
        return {"value": round(blocks.size / (t_deq + t_mm) / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{name}: the first {rows} of {n_full} rows x {k}, dequantize {t_deq * 1e3:.1f} ms + scalar f32 GEMV {t_mm * 1e3:.1f} ms"}

    # config 2: the Q4_K gate / up shape and the Q6_K head, a slice of rows each
    out["config2_decode_gemv"] = {"q4_k_12288x4096": gemv(12288, 4096, oracle.Q4_K, 2048, "Q4_K 12288 x 4096"),
                                  "q6_k_head_151936x4096": gemv(151936, 4096, oracle.Q6_K, 2048, "Q6_K 151936 x 4096")}
    # config 3: the scalar MoE block at one token; 32 of the 256 experts resident (the block touches the 8 routed ones and the
    # shared one, the router over 32 instead of 256 rows), weights dequantised once as hf2q's CPU path does at load time
    H, E, K, I = 2048, 32, 8, 512
    mk = lambda n, k: oracle.dequantize(oracle.quantize(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02), k, oracle.Q4_K,  # noqa: E731
                                                        threads=min(os.cpu_count() or 1, 16)), oracle.Q4_K, threads=8).reshape(n, k)
    eg, eu, ed, sg, su, sd = mk(E * I, H), mk(E * I, H), mk(E * H, I), mk(I, H), mk(I, H), mk(H, I)
    router = rng.standard_normal((E, H), dtype=np.float32) * np.float32(0.1)
    sgl = rng.standard_normal(H, dtype=np.float32) * np.float32(0.05)
    x = rng.standard_normal((1, H), dtype=np.float32)
    reps = 5
    t0 = time.perf_counter()
    for _ in range(reps):
        oracle.moe_ffn(x, H, E, K, I, I, router, eg, eu, ed, sgl, sg, su, sd)
    t_layer = (time.perf_counter() - t0) / reps
    out["config3_moe_decode_t1"] = {"value": round(1.0 / (40 * t_layer), 3), "unit": "tok/s", "cores": 1, "kind": "port",
                                    "sample": f"scalar MoE block (moe_ffn_cpu_ref) at one token, hidden 2048, top-8 of 32 resident experts x 512 + "
                                              f"shared expert, f32 weights dequantised beforehand: {t_layer * 1e3:.1f} ms per layer, x 40 layers"}
    # config 4: scalar f32 matmul over the dequantised Q4_K weights, 2 of the 2048 tokens
    M, Kd, N = 2, 4096, 12288
    wd = mk(N, Kd)
    xs = rng.standard_normal((M, Kd), dtype=np.float32)
    t0 = time.perf_counter()
    oracle.matmul_a_by_bt(xs, wd, M, Kd, N, threads=1)
    t_mm = time.perf_counter() - t0
    out["config4_prefill_gemm"] = {"value": round(2.0 * M * N * Kd / t_mm / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
                                   "sample": f"matmul_a_by_bt over dequantised Q4_K weights, {M} of 2048 tokens x 4096 x 12288: {t_mm * 1e3:.0f} ms"}
    # config 5: scalar attention over the int8 cache, 2048 of the 32768 positions
    nh, nkv, hd, n = 16, 2, 256, 2048
    kc = rng.integers(-127, 128, (nkv, n, hd)).astype(np.int8).view(np.uint8)
    vc = rng.integers(-127, 128, (nkv, n, hd)).astype(np.int8).view(np.uint8)
    kn = rng.uniform(0.5, 2.0, (nkv, n, 1)).astype(np.float32)
    vn = rng.uniform(0.5, 2.0, (nkv, n, 1)).astype(np.float32)
    q = rng.standard_normal((nh, hd)).astype(np.float32)
    t0 = time.perf_counter()
    oracle.tq_attention(q, kc, kn, vc, vn, None, nh, nkv, hd, n, n, 1.0 / 16.0)
    t_at = time.perf_counter() - t0
    nbytes = 2 * nkv * n * (hd + 4)
    out["config5_tq_attention"] = {"value": round(nbytes / t_at / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                                   "sample": f"scalar C attention over the int8 cache (dequantise in the loop, f64 accumulate), {n} of 32768 "
                                             f"positions, 16 / 2 heads, d = 256: {t_at * 1e3:.1f} ms"}
    return out


MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 peak


def _events(n):
    import torch
    return [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]


def _timed_steps(a, step, n_variants):
    """Exactly a.steps calls of step(i) between two synchronisations; returns (wall seconds, device
    microseconds per step from one HIP event pair around the whole region).  Unless --no-graph, the steps
    are replayed from HIP graphs the way a decode loop that records its token step runs them: one graph
    holds a run of min(32, steps) consecutive steps (the rotated variants in turn), replayed steps // run
    times, and a second graph holds the remaining steps."""
    import torch

    run = min(32, a.steps)
    q, r = (0, a.steps) if a.no_graph else divmod(a.steps, run)
    if a.no_graph:
        calls = [lambda i=i: step(a.warmup + i) for i in range(a.steps)]
    else:
        side = torch.cuda.Stream()
        graphs = []
        with torch.cuda.stream(side):
            for count in (run, r):
                if not count:
                    continue
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=side):
                    for i in range(count):
                        step(i)
                graphs.append(g)
        torch.cuda.synchronize()
        calls = [graphs[0].replay] * q + ([graphs[1].replay] if r else [])
        for g in graphs:  # untimed: first replay of each graph
            g.replay()
    e0, e1 = _events(1)[0]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for c in calls:
        c()
    e1.record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    return elapsed, e0.elapsed_time(e1) * 1e3 / a.steps


def _launch_us(launches, reps=5):
    """Device time of one launch: the callables (each enqueues ONE kernel, over weights no other of them touches)
    are recorded into a HIP graph back to back and the graph is replayed `reps` times, each replay between a HIP
    event pair of its own on the replay stream; the median replay / len(launches) (a replay of a millisecond or
    two now and then takes three times as long as its neighbours; the median leaves such a one out).  A kernel of
    a few microseconds cannot be timed by an event pair of its own: the pair adds ~2.5 us."""
    import torch

    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            for f in launches:
                f()
    torch.cuda.synchronize()
    g.replay()
    pairs = _events(reps)
    torch.cuda.synchronize()
    for e0, e1 in pairs:
        e0.record()
        g.replay()
        e1.record()
    torch.cuda.synchronize()
    times = sorted(e0.elapsed_time(e1) for e0, e1 in pairs)
    return times[len(times) // 2] * 1e3 / len(launches)


def _finish(a, out):
    """A workload run alone prints its own line; as part of the default run its dict goes under `workloads`."""
    if a.workload == "all":
        return out
    out.setdefault("n_gpus", 1)
    out.update({"steps": a.steps, "warmup": a.warmup, "higher_is_better": True, "scaling": "weak",
                "vs_baseline": None, "data": "synthetic"})
    out["cpu_baseline"] = None if a.no_cpu_baseline else cpu_baseline()
    print(json.dumps(out))
    return out


_MOE_LAYERS = {}  # the layers of bench_moe_decode, shared by its T = 1 and T = 8 runs


def bench_moe_decode(a, tokens=None, mix=False):
    """BASELINE config 3: Qwen3.6-35B-A3B-style MoE FFN layer, hidden 2048, 256 experts (inter 512, Q4_K), one
    shared expert, top-8 from seeded router logits, batch 1 or 8, bf16 activations.  A step is one layer.
    mix: the types the reference's model file really holds, gate / up Q5_K and down Q6_K (docs/ADR-028...:4942-4946)."""
    import torch

    from hf2q_amd import ops
    from hf2q_amd.ops import HQ_Q4_K

    dev = torch.device("cuda:0")
    H, E, K, I, SI, T = 2048, 256, 8, 512, 512, tokens or a.tokens
    tg, td = (ops.HQ_Q5_K, ops.HQ_Q6_K) if mix else (HQ_Q4_K, HQ_Q4_K)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    rnd = lambda *s: torch.randn(*s, generator=gen, device=dev, dtype=torch.float32)  # noqa: E731
    qz = lambda n, k, t: ops.quantize_ggml(rnd(n * k).mul_(0.02), k, t)  # noqa: E731
    n_layers = max(1, a.moe_layers)  # distinct layers rotated: a token touches 17 MB (T=1) of a layer, and the
    # 256 MB Infinity Cache must not hold the experts a layer routes to from its previous turn
    if (n_layers, mix) not in _MOE_LAYERS:
        _MOE_LAYERS.clear()
        _MOE_LAYERS[(n_layers, mix)] = [ops.MoeFfnWeightsGpuQ(
            rnd(E, H).mul_(0.02).to(torch.bfloat16), qz(E * I, H, tg), qz(E * I, H, tg), qz(E * H, I, td),
            rnd(1, H).mul_(0.02).to(torch.bfloat16), qz(SI, H, tg), qz(SI, H, tg), qz(H, SI, td), tg, H, E, K, I, SI,
            down_type=None if td == tg else td)
            for _ in range(n_layers)]
    layers = _MOE_LAYERS[(n_layers, mix)]
    gx = torch.Generator(device=dev)
    gx.manual_seed(5678)
    x = torch.randn(T, H, generator=gx, device=dev, dtype=torch.float32).to(torch.bfloat16)
    scratch = ops.MoeFfnScratch(layers[0], T, dev)
    out = torch.empty(T, H, device=dev)
    gu_bytes, dn_bytes = I * ops.ggml_row_bytes(tg, H), H * ops.ggml_row_bytes(td, I)

    def step(i):
        ops.build_moe_ffn_layer_gpu_q_into(x, layers[i % n_layers], scratch, out)

    eager_step = step
    for i in range(max(a.warmup, 1)):
        step(i)
    torch.cuda.synchronize()
    elapsed, layer_us = _timed_steps(a, eager_step, n_layers)
    uniq = []
    for i in range(min(a.steps, n_layers)):  # distinct experts actually routed (after the timed region)
        eager_step(i)
        uniq.append(int(torch.unique(scratch.ids[:T * K]).numel()))
    u = sum(uniq) / len(uniq)
    step_bytes = (u + 1) * (2 * gu_bytes + dn_bytes) + (E + 1) * H * 2  # routed + shared experts + router (bf16)
    gbs = step_bytes / layer_us / 1e3
    return _finish(a, {
        "metric": "MoE decode tok/s (FFN-only, 40 MoE layers)", "value": round(T / (40 * elapsed / a.steps), 1),
        "unit": "tok/s", "ms_per_step": round(elapsed / a.steps * 1e3, 4), "dtype": "bf16",
        "config": {"workload": f"moe_decode: hidden 2048, 256 experts x inter 512 {'gate / up Q5_K, down Q6_K' if mix else 'Q4_K'}, shared expert, top-8, "
                               f"batch {T}, bf16 activations (BASELINE config 3); one step = one MoE FFN layer = ONE launch "
                               f"(hq_moe_ffn_decode: router + shared logit, top-k, gate / up with SwiGLU, down, weighted "
                               f"sum, handed between workgroups inside the launch), "
                               f"{'launched from the host' if a.no_graph else 'replayed as a HIP graph'}",
                   "distinct_experts_per_layer": round(u, 1), "bytes_per_layer": int(step_bytes),
                   "layers_rotated": n_layers},
        "roofline": {"bound": "hbm", "kernel": "MoE FFN layer (hq_moe_ffn_decode, one launch)", "achieved": round(gbs, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": PMC_TRAFFIC_BYTES.get(f"moe_ffn_decode_t{T}" + ("_q5k_q6k" if mix else "")),
                     "us_per_launch": round(layer_us, 3), "bytes_per_launch": int(step_bytes)}})


def bench_prefill_gemm(a, wtype=None):
    """BASELINE config 4: 2048 tokens x K=4096 x N=12288, Q4_K (or Q8_0) weights, bf16 activations, f32 out."""
    import torch

    from hf2q_amd import ops
    from hf2q_amd.ops import HQ_Q4_K, HQ_Q8_0, GgmlQuantizedMatmulParams

    dev = torch.device("cuda:0")
    M, K, N = 2048, 4096, 12288
    wtype = wtype or a.wtype
    t = {"q4_k": HQ_Q4_K, "q8_0": HQ_Q8_0, "q6_k": ops.HQ_Q6_K, "q5_k": ops.HQ_Q5_K, "q4_0": ops.HQ_Q4_0}[wtype]
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    w = ops.quantize_ggml(torch.randn(N * K, generator=gen, device=dev).mul_(0.02), K, t)
    gx = torch.Generator(device=dev)
    gx.manual_seed(5678)
    x = torch.randn(M, K, generator=gx, device=dev).to(torch.bfloat16)
    y = torch.empty(M, N, device=dev)
    p = GgmlQuantizedMatmulParams(M, N, K, t)
    # caller-owned scratch for the tile kernels' pre-pass (f16 activations, row scales): allocated once
    need = ops.quantized_matmul_workspace_bytes(p, torch.bfloat16)
    ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None
    flops = 2.0 * M * N * K
    # The same product with the weight-row scales kept from load time (hq_qmatmul_ggml_ws_prepared; same bits), for
    # `config`.  The first tens of calls after an idle gap run slower, and of two forms timed one after the other the
    # first looked 6-8 us worse: this one is run once before the workload's own timing (not reported) and timed after it.
    scales = ops.weight_row_scales_ggml(w, N, K, t) if need else None

    def time_prepared():
        if not need:
            return None
        for _ in range(max(a.warmup, 1)):
            ops.quantized_matmul_ggml(x, w, y, p, workspace=ws, w_row_scales=scales)
        torch.cuda.synchronize()
        evp = _events(a.steps)
        for i in range(a.steps):
            evp[i][0].record()
            ops.quantized_matmul_ggml(x, w, y, p, workspace=ws, w_row_scales=scales)
            evp[i][1].record()
        torch.cuda.synchronize()
        return round(sum(e0.elapsed_time(e1) for e0, e1 in evp) * 1e3 / a.steps, 2)

    time_prepared()
    for _ in range(a.warmup):
        ops.quantized_matmul_ggml(x, w, y, p, workspace=ws)
    torch.cuda.synchronize()
    ev = _events(a.steps)
    t0 = time.perf_counter()
    for i in range(a.steps):
        ev[i][0].record()
        ops.quantized_matmul_ggml(x, w, y, p, workspace=ws)
        ev[i][1].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    us = sum(e0.elapsed_time(e1) for e0, e1 in ev) * 1e3 / a.steps
    tf = flops / us / 1e6
    us_prepared = time_prepared()
    # For scale only (not part of the path, not in `value`): the vendor library's plain f16 GEMM of the same shape,
    # no dequantisation, through torch.matmul; the same event timing over the same number of launches.
    vendor = None
    try:
        xa = x.to(torch.float16)
        wb = [torch.randn(N, K, generator=gen, device=dev).mul_(0.02).to(torch.float16) for _ in range(3)]
        for i in range(max(3, a.warmup)):
            torch.matmul(xa, wb[i % 3].t())
        torch.cuda.synchronize()
        evv = _events(a.steps)
        for i in range(a.steps):
            evv[i][0].record()
            torch.matmul(xa, wb[i % 3].t())
            evv[i][1].record()
        torch.cuda.synchronize()
        vus = sum(e0.elapsed_time(e1) for e0, e1 in evv) * 1e3 / a.steps
        vendor = {"what": "torch.matmul f16 2048x4096 @ 4096x12288 (hipBLASLt), plain weights", "us_per_launch": round(vus, 2),
                  "TFLOP/s": round(flops / vus / 1e6, 1), "frac_mfma_peak": round(flops / vus / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
        del wb
    except Exception as e:  # the reference figure must never take the bench line down
        vendor = {"error": str(e)[:200]}
    # The same product over the F16 shadow of the weight (hq_matmul_f16_shadow: the reference's route for m > 8 when a
    # weight has one, forward_mlx.rs:9790-9817): 2 bytes per weight kept in memory, no dequantisation in the product.
    shadow_line = None
    try:
        shadow = ops.dequantize_ggml(w, N * K, t, dtype=torch.float16)
        sws = torch.empty(ops.matmul_f16_shadow_workspace_bytes(M, N, K), dtype=torch.uint8, device=dev)
        for _ in range(max(3, a.warmup)):
            ops.matmul_f16_shadow(x, shadow, y, M, N, K, sws)
        torch.cuda.synchronize()
        evs = _events(a.steps)
        for i in range(a.steps):
            evs[i][0].record()
            ops.matmul_f16_shadow(x, shadow, y, M, N, K, sws)
            evs[i][1].record()
        torch.cuda.synchronize()
        sus = sum(e0.elapsed_time(e1) for e0, e1 in evs) * 1e3 / a.steps
        shadow_line = {"what": "hq_matmul_f16_shadow: activations cast to f16 + the vendor library's dense GEMM over the weight's F16 shadow",
                       "us_per_step": round(sus, 2), "TFLOP/s": round(flops / sus / 1e6, 1),
                       "frac_mfma_peak": round(flops / sus / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4), "shadow_bytes": shadow.numel() * 2}
        del shadow, sws
    except Exception as e:
        shadow_line = {"error": str(e)[:200]}
    return _finish(a, {
        "metric": "prefill TFLOP/s", "value": round(flops * a.steps / elapsed / 1e12, 1), "unit": "TFLOP/s",
        "ms_per_step": round(elapsed / a.steps * 1e3, 4), "dtype": "f16" if need else "bf16",
        "config": {"workload": f"prefill_gemm: 2048 tokens x K=4096 x N=12288, {wtype.upper()} weights, bf16 "
                               f"activations, fp32 accumulate (BASELINE config 4)", "flop_per_step": flops,
                   "weight_bytes": w.numel(), "workspace_bytes": need,
                   "launches_per_step": 2 if need else 1, "us_per_step_with_weight_row_scales_kept_from_load_time": us_prepared,
                   "vendor_dense_gemm_same_shape": vendor, "f16_shadow_route": shadow_line},
        "roofline": {"bound": "mfma", "kernel": (f"activation pre-pass + f16 MFMA gemm {wtype}" if need else
                                                 f"bf16 MFMA gemm {wtype}"), "achieved": round(tf, 1),
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": PMC_TRAFFIC_BYTES.get(f"prefill_gemm_{wtype}_2048x12288x4096"),
                     "us_per_launch": round(us, 2), "flop_per_launch": flops}})


def bench_moe_prefill(a):
    """The prefill side of BASELINE config 3's layer: mul_mat_id over 2048 tokens x top-8 of 256 experts, Q4_K, bf16
    activations, f32 out -- the gate / up shape (expert 512 x 2048, one activation row per token) and the down shape
    (expert 2048 x 512, one activation row per routed row).  A step is one gate / up call: the expert sort, the
    activation conversion and the weight-row scales in one launch, then the grouped tile GEMM."""
    import torch

    from hf2q_amd import ops
    from hf2q_amd.ops import HQ_Q4_K, GgmlQuantizedMatmulIdParams

    dev = torch.device("cuda:0")
    E, K, T, H, I = 256, 8, 2048, 2048, 512
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    n_stacks = 3  # 151 MB each, rotated past the 256 MB Infinity Cache

    def shape(n, k, rows, top_k):
        stacks = [ops.quantize_ggml(torch.randn(E * n * k, generator=gen, device=dev).mul_(0.02), k, HQ_Q4_K)
                  for _ in range(n_stacks)]
        p = GgmlQuantizedMatmulIdParams(rows, top_k, n, k, E, n * ops.ggml_row_bytes(HQ_Q4_K, k), HQ_Q4_K)
        x = torch.randn(rows, k, generator=gen, device=dev).to(torch.bfloat16)
        ids = torch.randint(0, E, (T * K,), generator=gen, device=dev, dtype=torch.int32)
        y = torch.empty(T * K, n, device=dev)
        need = ops.quantized_matmul_id_workspace_bytes(p)
        assert need > 0, "this shape must take the grouped route"
        scratch = torch.empty(need, dtype=torch.uint8, device=dev)

        scales = [ops.weight_row_scales_ggml(w, E * n, k, HQ_Q4_K) for w in stacks]  # once per stack, as at load time

        def step(i):
            ops.quantized_matmul_id_ggml(x, stacks[i % n_stacks], ids, y, p, scratch=scratch)

        def step_prepared(i):
            ops.quantized_matmul_id_ggml(x, stacks[i % n_stacks], ids, y, p, scratch=scratch, w_row_scales=scales[i % n_stacks])

        if a.step_only:  # the plain call and nothing else
            for i in range(max(a.warmup, 1)):
                step(i)
            torch.cuda.synchronize()
            elapsed, us = _timed_steps(a, step, n_stacks)
            return elapsed, us, us, need
        for i in range(max(a.warmup, 1)):
            step(i)
            step_prepared(i)
        torch.cuda.synchronize()
        # (of two forms timed one after the other the first looks a few microseconds worse: the kept-scales form is
        # run once before the workload's own timing, not reported, and timed after it)
        _timed_steps(a, step_prepared, n_stacks)
        elapsed, us = _timed_steps(a, step, n_stacks)
        _, us_prepared = _timed_steps(a, step_prepared, n_stacks)
        return elapsed, us, us_prepared, need

    if getattr(a, "block_only", False):  # the whole block alone, launched as asked (see `layer` below for what it is)
        rnd = lambda *s: torch.randn(*s, generator=gen, device=dev, dtype=torch.float32)  # noqa: E731
        qz = lambda n, k: ops.quantize_ggml(rnd(n * k).mul_(0.02), k, HQ_Q4_K)  # noqa: E731
        ls = [ops.MoeFfnWeightsGpuQ(rnd(E, H).mul_(0.02).to(torch.bfloat16), qz(E * I, H), qz(E * I, H), qz(E * H, I),
                                    rnd(1, H).mul_(0.02).to(torch.bfloat16), qz(I, H), qz(I, H), qz(H, I), HQ_Q4_K, H, E, K, I, I)
              for _ in range(2)]
        if a.kept_scales:
            for l in ls:
                l.prepare_prefill()
        x = rnd(T, H).to(torch.bfloat16)
        sc = ops.MoeFfnScratch(ls[0], T, dev)
        out = torch.empty(T, H, device=dev)

        def step(i):
            ops.build_moe_ffn_layer_gpu_q_into(x, ls[i % 2], sc, out)

        for i in range(max(a.warmup, 1)):
            step(i)
        torch.cuda.synchronize()
        elapsed, us = _timed_steps(a, step, 2)
        return _finish(a, {
            "metric": "MoE prefill tok/s (FFN-only, 40 MoE layers)", "value": round(T / (40 * elapsed / a.steps), 0), "unit": "tok/s",
            "ms_per_step": round(elapsed / a.steps * 1e3, 4), "dtype": "f16",
            "config": {"workload": "moe_prefill --block-only: build_moe_ffn_layer_gpu_q_into at 2048 tokens, hidden 2048, 256 experts x "
                                   "512 Q4_K, top-8, one shared expert" + (", weight-row scales kept from load time" if a.kept_scales else ""),
                       "us_per_layer": round(us, 1)}})

    elapsed, us, us_prep, need = shape(I, H, T, K)
    if a.step_only:  # the workload's own step and nothing else: for counter passes, whose per-kernel averages would mix shapes
        flops = 2.0 * T * K * I * H
        return _finish(a, {"metric": "MoE prefill mul_mat_id eff. TFLOP/s", "value": round(flops * a.steps / elapsed / 1e12, 1), "unit": "TFLOP/s",
                           "ms_per_step": round(elapsed / a.steps * 1e3, 4), "dtype": "f16",
                           "config": {"workload": "moe_prefill --step-only: the gate / up mul_mat_id call alone", "us_per_step": round(us, 2)}})
    _, us_down, us_down_prep, _ = shape(H, I, T * K, 1)

    # gate, up and SwiGLU of the block: two calls and hq_silu_mul, against the one grouped call that does all three
    def block():
        gates = [ops.quantize_ggml(torch.randn(E * I * H, generator=gen, device=dev).mul_(0.02), H, HQ_Q4_K) for _ in range(2)]
        ups = [ops.quantize_ggml(torch.randn(E * I * H, generator=gen, device=dev).mul_(0.02), H, HQ_Q4_K) for _ in range(2)]
        p = GgmlQuantizedMatmulIdParams(T, K, I, H, E, I * ops.ggml_row_bytes(HQ_Q4_K, H), HQ_Q4_K)
        x = torch.randn(T, H, generator=gen, device=dev).to(torch.bfloat16)
        ids = torch.randint(0, E, (T * K,), generator=gen, device=dev, dtype=torch.int32)
        yg, yu, act = (torch.empty(T * K, I, device=dev) for _ in range(3))
        scratch = torch.empty(ops.quantized_matmul_id_swiglu_workspace_bytes(p), dtype=torch.uint8, device=dev)

        def separate(i):
            ops.quantized_matmul_id_ggml(x, gates[i % 2], ids, yg, p, scratch=scratch)
            ops.quantized_matmul_id_ggml(x, ups[i % 2], ids, yu, p, scratch=scratch)
            ops.dispatch_silu_mul(yg, yu, act)

        def fused(i):
            ops.quantized_matmul_id_swiglu_ggml(x, gates[i % 2], ups[i % 2], ids, act, p, scratch)

        gs = [ops.weight_row_scales_ggml(w, E * I, H, HQ_Q4_K) for w in gates]
        us_ = [ops.weight_row_scales_ggml(w, E * I, H, HQ_Q4_K) for w in ups]

        def fused_kept(i):
            ops.quantized_matmul_id_swiglu_ggml(x, gates[i % 2], ups[i % 2], ids, act, p, scratch, gs[i % 2], us_[i % 2])

        for i in range(max(a.warmup, 1)):
            separate(i)
            fused(i)
        torch.cuda.synchronize()
        _timed_steps(a, fused, 2)
        _, us_sep = _timed_steps(a, separate, 2)
        _, us_fused = _timed_steps(a, fused, 2)
        _, us_kept = _timed_steps(a, fused_kept, 2)
        return us_sep, us_fused, us_kept

    us_sep, us_fused, us_fused_kept = block()

    # the whole MoE FFN block of a prefill chunk (router, routing, routed and shared experts, weighted sum), as the
    # host-side mirror of build_moe_ffn_layer_gpu_q_into encodes it above 8 tokens
    def layer():
        rnd = lambda *s: torch.randn(*s, generator=gen, device=dev, dtype=torch.float32)  # noqa: E731
        qz = lambda n, k: ops.quantize_ggml(rnd(n * k).mul_(0.02), k, HQ_Q4_K)  # noqa: E731
        ls = [ops.MoeFfnWeightsGpuQ(rnd(E, H).mul_(0.02).to(torch.bfloat16), qz(E * I, H), qz(E * I, H), qz(E * H, I),
                                    rnd(1, H).mul_(0.02).to(torch.bfloat16), qz(I, H), qz(I, H), qz(H, I), HQ_Q4_K, H, E, K, I, I)
              for _ in range(2)]
        x = rnd(T, H).to(torch.bfloat16)
        sc = ops.MoeFfnScratch(ls[0], T, dev)
        out = torch.empty(T, H, device=dev)

        def step(i):
            ops.build_moe_ffn_layer_gpu_q_into(x, ls[i % 2], sc, out)

        for i in range(max(a.warmup, 1)):
            step(i)
        torch.cuda.synchronize()
        _, us_plain = _timed_steps(a, step, 2)
        for l in ls:
            l.prepare_prefill()
        for i in range(2):
            step(i)
        torch.cuda.synchronize()
        _, us_kept = _timed_steps(a, step, 2)
        return us_plain, us_kept

    us_layer, us_layer_kept = layer()
    flops = 2.0 * T * K * I * H
    tf = flops / us / 1e6
    return _finish(a, {
        "metric": "MoE prefill mul_mat_id eff. TFLOP/s", "value": round(flops * a.steps / elapsed / 1e12, 1), "unit": "TFLOP/s",
        "ms_per_step": round(elapsed / a.steps * 1e3, 4), "dtype": "f16",
        "config": {"workload": "moe_prefill: mul_mat_id, 2048 tokens x top-8 over 256 experts, expert 512 x 2048 Q4_K (gate / up "
                               "shape of BASELINE config 3's layer), bf16 activations, fp32 accumulate; one step = 2 launches "
                               "(expert sort + activation conversion + weight-row scales; grouped tile GEMM), "
                               + ("launched from the host" if a.no_graph else "replayed as a HIP graph"),
                   "flop_per_step": flops, "workspace_bytes": need, "stacks_rotated": n_stacks,
                   "with_weight_row_scales_kept_from_load_time": {
                       "what": "hq_qmatmul_id_ggml_prepared: the stack's row scales (a function of the weights alone) computed "
                               "once, the call's pre-pass skips their scan; same bits", "us_per_step": round(us_prep, 2),
                       "TFLOP/s": round(flops / us_prep / 1e6, 1)},
                   "gate_up_swiglu": {"what": "gate, up and SwiGLU of the block (2 x 34.4 GFLOP): two mul_mat_id calls + hq_silu_mul "
                                              "(5 launches) against hq_qmatmul_id_swiglu_ggml (2 launches), same bits",
                                      "separate_us": round(us_sep, 2), "one_call_us": round(us_fused, 2),
                                      "one_call_with_kept_scales_us": round(us_fused_kept, 2),
                                      "one_call_TFLOP/s": round(2 * flops / us_fused / 1e6, 1)},
                   "whole_block_2048_tokens": {"what": "build_moe_ffn_layer_gpu_q_into at 2048 tokens: router, softmax / top-8, gate / up / "
                                                       "SwiGLU and down of the routed experts (grouped), the shared expert, the weighted "
                                                       "sum; 12 launches", "us_per_layer": round(us_layer, 1),
                                               "us_per_layer_with_kept_scales": round(us_layer_kept, 1),
                                               "tok/s_over_40_layers": round(T / (40 * us_layer * 1e-6), 0)},
                   "down_shape_2048x512": {"us_per_step": round(us_down, 2), "TFLOP/s": round(flops / us_down / 1e6, 1),
                                           "us_per_step_with_kept_scales": round(us_down_prep, 2)}},
        "roofline": {"bound": "mfma", "kernel": "grouped pre-pass + grouped f16 MFMA gemm q4_k", "achieved": round(tf, 1),
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": PMC_TRAFFIC_BYTES["moe_prefill_gate_up_2048x8"], "us_per_launch": round(us, 2), "flop_per_launch": flops}})


def bench_tq_attention(a):
    """BASELINE config 5: decode attention over the 8-bit KV cache, 32K context, 16 q / 2 kv heads, d=256."""
    import torch

    from hf2q_amd import ops
    from hf2q_amd.ops import FlashAttnVecTqHbParams

    dev = torch.device("cuda:0")
    nh, nkv, hd, n = 16, 2, 256, 32768
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    n_caches = 12  # 34 MB each: rotate past the 256 MB Infinity Cache
    caches = []
    for _ in range(n_caches):
        kc, kn = ops.alloc_tq_kv(nkv, n, hd, dev)
        vc, vn = ops.alloc_tq_kv(nkv, n, hd, dev)
        ops.hadamard_quantize_kv(torch.randn(n, nkv, hd, generator=gen, device=dev), kc, kn, 0)
        ops.hadamard_quantize_kv(torch.randn(n, nkv, hd, generator=gen, device=dev), vc, vn, 0)
        caches.append((kc, kn, vc, vn))
    q = torch.randn(nh, hd, generator=gen, device=dev)
    out = torch.empty(nh, hd, device=dev)
    tmp = torch.empty(ops.tq_tmp_buffer_bytes(nh, hd, n) // 4, device=dev)
    p = FlashAttnVecTqHbParams(nh, nkv, hd, n, n, 1.0 / 16.0)
    nbytes = sum(t.numel() * t.element_size() for t in caches[0])

    pf = FlashAttnVecTqHbParams(nh, nkv, hd, n, n, 1.0 / 16.0, fuse_fwht_pre=1)

    def separate(i):  # the reference's decode chain as three dispatches: rotate q, attend, rotate the output back
        ops.dispatch_fwht_sign_premult_f32(q, nh, hd)
        ops.flash_attn_vec_tq_hb(q, *caches[i % n_caches], out, tmp, p)
        ops.dispatch_fwht_sign_undo_f32(out, nh, hd)

    def fused(i):  # the same chain with both rotations inside the attention call (bit-identical result)
        ops.flash_attn_vec_tq_hb(q, *caches[i % n_caches], out, tmp, pf, undo_rotation=True)

    def timed(step):
        for i in range(max(a.warmup, 1)):
            step(i)
        torch.cuda.synchronize()
        return _timed_steps(a, step, n_caches)

    _, us_sep = timed(separate)
    elapsed, us = timed(fused)
    gbs = nbytes / us / 1e3
    return _finish(a, {
        "metric": "TQ-KV decode attention eff. GB/s", "value": round(nbytes * a.steps / elapsed / 1e9, 1),
        "unit": "GB/s", "ms_per_step": round(elapsed / a.steps * 1e3, 4), "dtype": "f32",
        "config": {"workload": "tq_attention: 32768 context, 16 q heads / 2 kv heads, head_dim 256, int8 codes + f32 "
                               "norm per (token, head), batch 1 (BASELINE config 5); one step = rotate q, attend, rotate "
                               "the output back, as one call = 2 launches (split with the q rotation, merge with the "
                               "output rotation)", "bytes_per_step": nbytes, "caches_rotated": n_caches,
                   "separate_dispatch": {"launches": 4, "us_per_step": round(us_sep, 3),
                                         "GB/s": round(nbytes / us_sep / 1e3, 1)}},
        "roofline": {"bound": "hbm", "kernel": "tq attention split (+ q rotation) + merge (+ output rotation)",
                     "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": PMC_TRAFFIC_BYTES["tq_attention_32k_fused_chain"], "us_per_launch": round(us, 3),
                     "bytes_per_launch": nbytes}})


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
    if a.calibration_copy:
        src = torch.randint(0, 255, (256 << 20,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if a.workload not in ("all", "decode_gemv"):
        if a.workload == "moe_decode":
            return bench_moe_decode(a, mix=a.mix)
        return {"moe_prefill": bench_moe_prefill, "prefill_gemm": bench_prefill_gemm,
                "tq_attention": bench_tq_attention}[a.workload](a)
    out = bench_decode_gemv(a)
    if a.workload == "all":
        def brief(d):
            keep = ("metric", "value", "unit", "ms_per_step", "dtype", "config", "roofline")
            return {**{k: d[k] for k in keep if k in d}, "steps": a.steps}
        import copy
        import gc
        wl = {}
        # The other workloads' steps take 15 .. 290 us: timed over at least 256 of them whatever --steps says (a few
        # milliseconds each), so that a graph launch and the clock's ramp after an idle gap do not weigh on the figure.
        a = copy.copy(a)
        a.steps = max(a.steps, 256)
        for name, fn in (("moe_decode_t1", lambda: bench_moe_decode(a, 1)), ("moe_decode_t8", lambda: bench_moe_decode(a, 8)),
                         ("moe_decode_t1_q5k_q6k", lambda: bench_moe_decode(a, 1, mix=True)),
                         ("moe_decode_t8_q5k_q6k", lambda: bench_moe_decode(a, 8, mix=True)),
                         ("moe_prefill_2048x8", lambda: bench_moe_prefill(a)),
                         ("prefill_gemm_q4_k", lambda: bench_prefill_gemm(a, "q4_k")),
                         ("prefill_gemm_q8_0", lambda: bench_prefill_gemm(a, "q8_0")),
                         ("tq_attention_32k", lambda: bench_tq_attention(a))):
            gc.collect()
            torch.cuda.empty_cache()
            wl[name] = brief(fn())
            if name == "moe_decode_t8_q5k_q6k":
                _MOE_LAYERS.clear()
        out["workloads"] = wl
    out["cpu_baseline"] = None if a.no_cpu_baseline else cpu_baseline()
    if not a.no_cpu_baseline and a.workload == "all":
        out["cpu_baseline"]["by_config"] = cpu_baselines_by_config()
    print(json.dumps(out))


def bench_decode_gemv(a):
    """BASELINE config 2 (the headline): the four dense decode GEMVs of one token."""
    import torch

    from hf2q_amd import ops
    from hf2q_amd.ops import HQ_Q4_K, HQ_Q6_K, GgmlQuantizedMatmulParams

    dev = torch.device("cuda:0")
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

    def one(nm, w):
        return lambda: ops.quantized_matmul_ggml(x_f if nm == "down" else x_h, w, y[nm], params[nm])

    def step(i):
        ws = sets[i % n_sets]
        for nm in ("gate", "up", "down", "head"):
            one(nm, heads[i % n_heads] if nm == "head" else ws[nm])()

    # The same four products as a decode step dispatches them: gate and up read the same activations and
    # the reference encodes them without a barrier in between (gpu_ffn.rs:1236-1258), so they go to the
    # library as one batched launch; down and the head follow = three launches.
    def fused_step(i):
        ws = sets[i % n_sets]
        ops.quantized_matmul_batch_ggml([ops.QmatmulJob(x_h, ws["gate"], y["gate"], 1, F, H),
                                         ops.QmatmulJob(x_h, ws["up"], y["up"], 1, F, H)], HQ_Q4_K)
        ops.quantized_matmul_ggml(x_f, ws["down"], y["down"], params["down"])
        ops.quantized_matmul_ggml(x_h, heads[i % n_heads], y["head"], params["head"])

    for i in range(max(a.warmup, 1)):
        step(i)
        fused_step(i)
    torch.cuda.synchronize()

    # The same K steps as the region behind `value` below, timed here, a few milliseconds of work after set-up: the
    # device is not at its steady rate yet (the same steps get faster over the first 100-200 ms of continuous work
    # after an idle period: 108 -> 98 us per step in one process), so this figure is reported beside `value`, which
    # is measured after the per-kernel measurements that follow, as a decode loop of more than a second sees the device.
    first_region_us = None
    if not a.no_graph:
        el_first, _ = _timed_steps(a, fused_step, n_sets * n_heads)
        first_region_us = el_first / a.steps * 1e6
    for i in range(SETTLE_STEPS):  # untimed: about a quarter of a second of decode steps
        fused_step(i)
    torch.cuda.synchronize()

    # K steps launched one kernel at a time from the host (Python + ctypes per launch).
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(a.warmup + i)
    torch.cuda.synchronize()
    el_host = time.perf_counter() - t0
    host = {"ms_per_step": round(el_host / a.steps * 1e3, 4), "GBps": round(step_bytes * a.steps / el_host / 1e9, 1),
            "frac_hbm_peak": round(step_bytes * a.steps / el_host / 1e9 / HBM_PEAK_GBS, 4)}

    # Per-kernel durations behind `roofline` and `kernels`: HIP events around back-to-back launches of ONE kernel
    # over distinct matrices, see _launch_us.  The 28 MB shapes rotate over all 3 * n_sets FFN buffers (a buffer of
    # Q4_K blocks reads as 12288 x 4096 or as 4096 x 12288 alike): 510 MB between two uses of a buffer, twice the
    # 256 MB Infinity Cache -- over the six down matrices alone (170 MB) a kernel that fetches with ordinary loads
    # finds them there (4096 x 12288 with f32 activations: 7.7 instead of 8.6 us).
    ffn_bufs = [ws[nm] for ws in sets for nm in ("gate", "up", "down")]
    kern_us = {
        "gate_up_12288x4096": _launch_us([one("gate", b) for b in ffn_bufs] * 3),
        "down_4096x12288": _launch_us([one("down", b) for b in ffn_bufs] * 3),
        "head_151936x4096": _launch_us([one("head", h) for h in heads] * 8),
        "gate_and_up_one_launch": _launch_us([
            (lambda b0=b0, b1=b1: ops.quantized_matmul_batch_ggml([ops.QmatmulJob(x_h, b0, y["gate"], 1, F, H),
                                                                  ops.QmatmulJob(x_h, b1, y["up"], 1, F, H)], HQ_Q4_K))
            for b0, b1 in zip(ffn_bufs[0::2], ffn_bufs[1::2])] * 5),
    }
    kbytes = {"gate_up_12288x4096": nbytes["gate"], "down_4096x12288": nbytes["down"], "head_151936x4096": nbytes["head"],
              "gate_and_up_one_launch": nbytes["gate"] + nbytes["up"]}
    kernels = {nm: {"us": round(kern_us[nm], 3), "bytes": kbytes[nm], "GBps": round(kbytes[nm] / kern_us[nm] / 1e3, 1),
                    "frac_hbm_peak": round(kbytes[nm] / kern_us[nm] / 1e3 / HBM_PEAK_GBS, 4)} for nm in kern_us}
    # The same three matrices under f32 activations, the dtype the reference's call sites pass (gpu_full_attn.rs:835).
    x_h32, x_f32 = x_h.float(), x_f.float()

    def one32(nm, w):
        return lambda: ops.quantized_matmul_ggml(x_f32 if nm == "down" else x_h32, w, y[nm], params[nm])

    kern32_us = {
        "gate_up_12288x4096": _launch_us([one32("gate", b) for b in ffn_bufs] * 3),
        "down_4096x12288": _launch_us([one32("down", b) for b in ffn_bufs] * 3),
        "head_151936x4096": _launch_us([one32("head", h) for h in heads] * 8),
    }
    kernels_f32 = {nm: {"us": round(us, 3), "bytes": kbytes[nm], "GBps": round(kbytes[nm] / us / 1e3, 1),
                        "frac_hbm_peak": round(kbytes[nm] / us / 1e3 / HBM_PEAK_GBS, 4)} for nm, us in kern32_us.items()}
    q4_bytes = 2 * nbytes["gate"] + nbytes["down"]
    q4_us = 2 * kern_us["gate_up_12288x4096"] + kern_us["down_4096x12288"]
    q4_us_fewer = kern_us["gate_and_up_one_launch"] + kern_us["down_4096x12288"]

    # The dense FFN of the decode step as a chain (x bf16 -> gate, up -> SwiGLU in f32 -> down over the f32 activations,
    # the reference's dataflow, gpu_ffn.rs:1231-1306): three dispatches + hq_silu_mul, two launches (gate + up + SwiGLU as
    # one streaming launch, then down), and the whole block as one launch with an in-launch hand-over.
    gate_b, up_b, act_b = (torch.empty(1, F, device=dev) for _ in range(3))
    ffn_w = [ops.DenseFfnWeightsGpuQ(ws["gate"], ws["up"], ws["down"], HQ_Q4_K, H, F) for ws in sets]
    ffn_out = torch.empty(1, H, device=dev)
    ffn_scratch = torch.zeros(ops.dense_ffn_decode_scratch_bytes(ffn_w[0], torch.bfloat16), dtype=torch.uint8, device=dev)
    p_gu = GgmlQuantizedMatmulParams(1, F, H, HQ_Q4_K)

    def ffn_separate(w):
        ops.quantized_matmul_batch_ggml([ops.QmatmulJob(x_h, w.gate_q, gate_b, 1, F, H), ops.QmatmulJob(x_h, w.up_q, up_b, 1, F, H)], HQ_Q4_K)
        ops.dispatch_silu_mul(gate_b, up_b, act_b)
        ops.quantized_matmul_ggml(act_b, w.down_q, ffn_out, params["down"])

    def ffn_two(w):
        ops.quantized_matmul_swiglu_decode(x_h, w.gate_q, w.up_q, act_b, p_gu)
        ops.quantized_matmul_ggml(act_b, w.down_q, ffn_out, params["down"])

    def ffn_one(w):
        ops.dense_ffn_decode(x_h, w, ffn_out, ffn_scratch)

    ffn_bytes = q4_bytes
    ffn_us = {nm: _launch_us([(lambda w=w, f=f: f(w)) for w in ffn_w] * 5) for nm, f in
              (("separate_dispatches_4_launches", ffn_separate), ("two_launches", ffn_two), ("one_launch", ffn_one))}
    dense_ffn = {nm: {"us": round(us, 3), "GBps": round(ffn_bytes / us / 1e3, 1), "frac_hbm_peak": round(ffn_bytes / us / 1e3 / HBM_PEAK_GBS, 4)}
                 for nm, us in ffn_us.items()}
    dense_ffn["bytes"] = ffn_bytes
    dense_ffn["what"] = ("the FFN of the decode step as a chain, Q4_K 4096 -> 12288 -> 4096, bf16 input, f32 SwiGLU activations into the down "
                         "projection (gpu_ffn.rs:1231-1306); us per FFN, every form the same bits")
    del ffn_w, gate_b, up_b

    # The reference's own published decode shapes (docs/ADR-028...:5247, 5248, 4884, 8564), both activation
    # dtypes (its call sites pass f32, gpu_full_attn.rs:835): lm_head 262144 x 2816 in Q6_K and Q8_0, the 4096 x 2816 and
    # 2816 x 4096 projections in Q5_K.
    ref_shapes = {}
    for nm, (n, k, t) in (("q6_k_lm_head_262144x2816", (262144, 2816, HQ_Q6_K)), ("q8_0_lm_head_262144x2816", (262144, 2816, ops.HQ_Q8_0)),
                          ("q5_k_4096x2816", (4096, 2816, ops.HQ_Q5_K)), ("q5_k_2816x4096", (2816, 4096, ops.HQ_Q5_K))):
        copies = 2 if n > 100000 else 8
        wsr = [make_weight(n, k, t) for _ in range(copies)]
        yr = torch.empty(1, n, device=dev)
        pr = GgmlQuantizedMatmulParams(1, n, k, t)
        entry = {"bytes": wsr[0].numel()}
        for dt, dn in ((torch.bfloat16, "bf16"), (torch.float32, "f32")):
            xr = torch.randn(1, k, generator=gx, device=dev, dtype=torch.float32).to(dt)
            us = _launch_us([(lambda w=w: ops.quantized_matmul_ggml(xr, w, yr, pr)) for w in wsr] * (4 if copies == 2 else 4))
            entry[dn] = {"us": round(us, 3), "GBps": round(wsr[0].numel() / us / 1e3, 1),
                         "frac_hbm_peak": round(wsr[0].numel() / us / 1e3 / HBM_PEAK_GBS, 4)}
        if n > 100000:  # the lm_heads at a few bf16 rows (batched decode): one pass over the weights for all of them
            for m_ in (2, 8):
                xm = torch.randn(m_, k, generator=gx, device=dev, dtype=torch.float32).to(torch.bfloat16)
                ym = torch.empty(m_, n, device=dev)
                pm = GgmlQuantizedMatmulParams(m_, n, k, t)
                us = _launch_us([(lambda w=w: ops.quantized_matmul_ggml(xm, w, ym, pm)) for w in wsr] * 4)
                entry[f"bf16_rows_{m_}"] = {"us": round(us, 2), "GBps": round(wsr[0].numel() / us / 1e3, 1),
                                            "frac_hbm_peak": round(wsr[0].numel() / us / 1e3 / HBM_PEAK_GBS, 4)}
        ref_shapes[nm] = entry
        del wsr

    # A few activation rows at once (batched decode): one pass over the weights for all of them.  The head and the gate
    # matrix of the step above, and a 65536 x 4096 Q4_K matrix; us per launch, weight bytes / time.
    small_batch = {}
    big = [make_weight(65536, H, HQ_Q4_K) for _ in range(4)]
    for nm, mats, (n_, k_, t_) in (("head_q6_k_151936x4096", heads, shapes["head"]), ("q4_k_65536x4096", big, (65536, H, HQ_Q4_K)),
                                   ("gate_q4_k_12288x4096", ffn_bufs, shapes["gate"])):
        entry = {"bytes": mats[0].numel()}
        for m_ in (2, 4, 8):
            xm = torch.randn(m_, k_, generator=gx, device=dev, dtype=torch.float32).to(torch.bfloat16)
            ym = torch.empty(m_, n_, device=dev)
            pm = GgmlQuantizedMatmulParams(m_, n_, k_, t_)
            us = _launch_us([(lambda w=w: ops.quantized_matmul_ggml(xm, w, ym, pm)) for w in mats] * max(1, 12 // len(mats)))
            entry[f"rows_{m_}"] = {"us": round(us, 2), "GBps": round(mats[0].numel() / us / 1e3, 1),
                                   "frac_hbm_peak": round(mats[0].numel() / us / 1e3 / HBM_PEAK_GBS, 4)}
        # four f32 rows (the dtype of the reference's call sites): hi and lo parts staged in the space of eight bf16 rows
        xm = torch.randn(4, k_, generator=gx, device=dev, dtype=torch.float32)
        ym = torch.empty(4, n_, device=dev)
        pm = GgmlQuantizedMatmulParams(4, n_, k_, t_)
        us = _launch_us([(lambda w=w: ops.quantized_matmul_ggml(xm, w, ym, pm)) for w in mats] * max(1, 12 // len(mats)))
        entry["rows_4_f32"] = {"us": round(us, 2), "GBps": round(mats[0].numel() / us / 1e3, 1),
                               "frac_hbm_peak": round(mats[0].numel() / us / 1e3 / HBM_PEAK_GBS, 4)}
        small_batch[nm] = entry
    del big

    # What streaming these bytes costs on this device with no arithmetic at all (hq_stream_read_probe: plain 16-byte loads,
    # the same back-to-back timing over the same rotated buffers): the rate the figures above can be read against beside
    # the published peak.
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    probe = {}
    for nm, bufs, reps in (("head_510MB", heads, 8), ("gate_28MB", ffn_bufs, 3)):
        us = _launch_us([(lambda b=b: ops.stream_read_probe(b, sink)) for b in bufs] * reps)
        nb_ = bufs[0].numel()
        probe[nm] = {"us": round(us, 3), "bytes": nb_, "GBps": round(nb_ / us / 1e3, 1), "frac_hbm_peak": round(nb_ / us / 1e3 / HBM_PEAK_GBS, 4)}
    probe["what"] = ("one plain read of the same buffers, 16 bytes per lane, no arithmetic (hq_stream_read_probe), timed like `kernels`: the "
                     "streaming rate this device reaches; kernels[...].us / this us = how far a kernel is from it")

    # The head inside the step, behind `roofline`: host-launched steps with a HIP event pair around every head launch
    # (the pair reads the kernel's time plus the 2-4 us its two markers add).  A head launch that follows the step's
    # FFN kernels is faster than one that follows another head launch, which is what `kernels` times (kernel trace:
    # 80.1 us inside steps, 87.4 us back to back, under the profiler on one device), and the step is the workload.
    n_in = max(a.steps, 64)
    pairs_in = _events(n_in)
    torch.cuda.synchronize()
    for i in range(n_in):
        ws = sets[i % n_sets]
        ops.quantized_matmul_batch_ggml([ops.QmatmulJob(x_h, ws["gate"], y["gate"], 1, F, H),
                                         ops.QmatmulJob(x_h, ws["up"], y["up"], 1, F, H)], HQ_Q4_K)
        ops.quantized_matmul_ggml(x_f, ws["down"], y["down"], params["down"])
        pairs_in[i][0].record()
        ops.quantized_matmul_ggml(x_h, heads[i % n_heads], y["head"], params["head"])
        pairs_in[i][1].record()
    torch.cuda.synchronize()
    head_in_step = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in pairs_in)
    head_in_step_us = sum(head_in_step) / len(head_in_step)

    # The timed region behind `value`: exactly K steps replayed from HIP graphs of their three launches
    # (runs of consecutive steps over the rotated weight sets and heads), as a decode loop that records
    # its token step does; the host's per-launch cost (Python, ctypes) is then out of the way, like in
    # the other workloads.
    elapsed, step_us_events = el_host, None
    if not a.no_graph:
        elapsed, step_us_events = _timed_steps(a, fused_step, n_sets * n_heads)

    value = step_bytes * a.steps / elapsed / 1e9
    head_us = head_in_step_us
    head_gbs = nbytes["head"] / head_us / 1e3
    return {
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
                               "batch 1, bf16 activations (BASELINE config 2); one step = "
                               + ("the four GEMVs launched one by one from the host" if a.no_graph else
                                  "gate + up in one batched launch, down, head = 3 launches replayed as a HIP graph"),
                   "bytes_per_step": step_bytes, "weight_sets": n_sets, "head_copies": n_heads,
                   "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4),
                   "step_us_by_hip_events": None if step_us_events is None else round(step_us_events, 2),
                   "timed_after": f"{a.warmup} warm-up steps, {SETTLE_STEPS} more untimed steps and the per-kernel measurements of this line "
                                  "(the device at its steady rate)",
                   "us_per_step_first_region": None if first_region_us is None else round(first_region_us, 2)},
        "roofline": {"bound": "hbm", "kernel": "gemv Q6_K head 151936x4096", "achieved": round(head_gbs, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(head_gbs / HBM_PEAK_GBS, 4),
                     "traffic": PMC_TRAFFIC_BYTES["gemv_head_q6_k_151936x4096"],
                     "traffic_source": "recorded: rocprofv3 --pmc runs of this file, profiles/gemv_decode_config2_pmc_traffic.md",
                     "us_per_launch": round(head_us, 3), "bytes_per_launch": nbytes["head"]},
        "kernels": kernels,
        "head_in_step": {"us_avg": round(head_in_step_us, 3), "us_median": round(head_in_step[len(head_in_step) // 2], 3), "launches": n_in,
                         "what": "HIP event pair around each head launch of host-launched steps (roofline.us_per_launch); "
                                 "kernels.head_151936x4096 is head launches back to back"},
        "kernels_f32_activations": kernels_f32,
        "host_launched": host,
        "q4_k_gemv": {"GBps": round(q4_bytes / q4_us / 1e3, 1), "frac_hbm_peak": round(q4_bytes / q4_us / 1e3 / HBM_PEAK_GBS, 4),
                      "what": "gate, up, down as three launches of their own (bf16 activations each)",
                      "gate_and_up_as_one_launch": {"GBps": round(q4_bytes / q4_us_fewer / 1e3, 1),
                                                    "frac_hbm_peak": round(q4_bytes / q4_us_fewer / 1e3 / HBM_PEAK_GBS, 4)}},
        "dense_ffn_decode_chain": dense_ffn,
        "reference_shapes": ref_shapes,
        "stream_read_probe": probe,
        "small_batch_rows": small_batch,
    }


if __name__ == "__main__":
    main()
