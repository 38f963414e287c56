#!/usr/bin/env python3
"""Benchmark of the Q4_K grouped-MoE LoRA expert layer (forward + backward) on one MI355X.

Workload (BASELINE.json configs[2]): 4096 tokens, hidden 2048, 256 experts, top-8 routing from N(0,1)
router logits, per expert gate/up [512+512, 2048] and down [2048, 512] drawn from N(0, 0.02^2) and
quantized to Q4_K, rank-16 LoRA (alpha 32) on both projections, dY ~ N(0,1) bf16.  One step = routing
plan + gather + gate/up + SiLU gate + down + combine, and the whole backward (dHidden, dRoutingWeights,
dA/dB of both projections).  Inputs are resident in HBM before the timed region.

Prints one JSON line: whole-step throughput in algorithmic TFLOP/s (430.0 GFLOP per step), the roofline
of the dominant kernel (packed-weight tile kernel, timed with HIP events on its launch stream while the
timed steps run) and a CPU baseline (dequantize-then-matmul on the host cores, bounded sample).
"""

from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import torch

import __graft_entry__

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
HBM_PEAK_GBS = 8000.0

CFG = dict(tokens=4096, hidden=2048, inter=512, experts=256, top_k=8, rank=16, alpha=32.0)


def algorithmic_flops(cfg) -> dict:
    routes = cfg["tokens"] * cfg["top_k"]
    h, i, r = cfg["hidden"], cfg["inter"], cfg["rank"]
    base_gu = 2 * routes * (2 * i) * h          # one pass over gate+up
    base_d = 2 * routes * h * i
    lora = 3 * 2 * routes * r * ((h + 2 * i) + (i + h))   # fwd 2 GEMMs + bwd 4 GEMMs per projection
    return dict(gate_up=base_gu, down=base_d, base_total=2 * (base_gu + base_d), lora=lora, total=2 * (base_gu + base_d) + lora)


def packed_weight_bytes(cfg) -> int:
    return cfg["experts"] * (2 * cfg["inter"] * cfg["hidden"] + cfg["hidden"] * cfg["inter"]) * 144 // 256


def build_workload(pkg, dev, cfg, seed=19260817 + 2):
    g = torch.Generator(device=dev).manual_seed(seed)
    e, h, i, r = cfg["experts"], cfg["hidden"], cfg["inter"], cfg["rank"]
    G = pkg.gguf.GGUFQuantizedTensor

    def packed(shape):
        out = []
        for lo in range(0, e, 32):  # quantize in slices to bound the fp32 staging memory
            w = torch.randn((min(32, e - lo),) + shape, generator=g, device=dev) * 0.02
            out.append(pkg.gguf.quantize_q4_k(w))
        return torch.cat(out, dim=0)

    gate = G(packed((i, h)), 12, (e, i, h))
    up = G(packed((i, h)), 12, (e, i, h))
    down = G(packed((h, i)), 12, (e, h, i))
    experts = pkg.fast_moe_lora.GGUFExperts(gate, up, down)
    layer = pkg.fast_moe_lora.FastGGUFMoeLora(experts, r=r, lora_alpha=cfg["alpha"])
    with torch.no_grad():
        layer.lora_A["default"].weight.copy_((torch.randn(e, r, h, generator=g, device=dev) * h ** -0.5).to(torch.bfloat16))
        layer.lora_B["default"].weight.copy_((torch.randn(e, 2 * i, r, generator=g, device=dev) * 0.01).to(torch.bfloat16))
        layer.lora_A_down["default"].weight.copy_((torch.randn(e, r, i, generator=g, device=dev) * i ** -0.5).to(torch.bfloat16))
        layer.lora_B_down["default"].weight.copy_((torch.randn(e, h, r, generator=g, device=dev) * 0.01).to(torch.bfloat16))
    x = torch.randn(cfg["tokens"], h, generator=g, device=dev).to(torch.bfloat16).requires_grad_(True)
    logits = torch.randn(cfg["tokens"], e, generator=g, device=dev)
    top = torch.topk(logits, cfg["top_k"], dim=-1)
    idx = top.indices
    weights = torch.softmax(top.values, dim=-1).requires_grad_(True)
    dy = torch.randn(cfg["tokens"], h, generator=g, device=dev).to(torch.bfloat16)
    return layer, x, idx, weights, dy


def cpu_baseline(cfg, sample_experts=64, repeats=21):
    """Dequantize-then-matmul on the host (the reference's non-native shape of the path,
    fast_moe_lora.py:230-247): oracle decoders -> bf16 weights -> torch matmul + autograd per expert,
    on `sample_experts` experts with 128 rows each (the layer's mean load)."""
    import numpy as np

    from oracle import gguf_blocks as gb

    torch.set_num_threads(os.cpu_count() or 1)
    h, i, r = cfg["hidden"], cfg["inter"], cfg["rank"]
    rows = cfg["tokens"] * cfg["top_k"] // cfg["experts"]
    rng = np.random.default_rng(0)
    pg = gb.quantize((rng.standard_normal((sample_experts, 2 * i, h)) * 0.02).astype(np.float32), gb.Q4_K)
    pd = gb.quantize((rng.standard_normal((sample_experts, h, i)) * 0.02).astype(np.float32), gb.Q4_K)
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(sample_experts, rows, h, generator=gen).to(torch.bfloat16)
    dy = torch.randn(sample_experts, rows, h, generator=gen).to(torch.bfloat16)
    a_gu = (torch.randn(sample_experts, r, h, generator=gen) * h ** -0.5).to(torch.bfloat16).requires_grad_(True)
    b_gu = (torch.randn(sample_experts, 2 * i, r, generator=gen) * 0.01).to(torch.bfloat16).requires_grad_(True)
    a_d = (torch.randn(sample_experts, r, i, generator=gen) * i ** -0.5).to(torch.bfloat16).requires_grad_(True)
    b_d = (torch.randn(sample_experts, h, r, generator=gen) * 0.01).to(torch.bfloat16).requires_grad_(True)
    s = cfg["alpha"] / r

    def one_pass():
        for e in range(sample_experts):
            wgu = torch.from_numpy(gb.dequantize(pg[e], gb.Q4_K)).to(torch.bfloat16)
            wd = torch.from_numpy(gb.dequantize(pd[e], gb.Q4_K)).to(torch.bfloat16)
            xe = x[e].clone().requires_grad_(True)
            gu = torch.addmm(xe @ wgu.T, xe @ a_gu[e].T, b_gu[e].T, alpha=s)
            hmid = torch.nn.functional.silu(gu[:, :i]) * gu[:, i:]
            out = torch.addmm(hmid @ wd.T, hmid @ a_d[e].T, b_d[e].T, alpha=s)
            out.backward(dy[e])

    one_pass()
    times = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        one_pass()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    fl = algorithmic_flops(dict(cfg, tokens=sample_experts * rows // cfg["top_k"]))
    return dict(value=fl["total"] / med / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                sample=f"{sample_experts} of {cfg['experts']} experts x {rows} rows, dequantize (numpy oracle) + torch bf16 matmul/autograd, median of {repeats}, {med:.2f} s per pass")


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--graph", type=int, default=1, help="replay the step from a captured HIP graph (1) or run it eagerly (0)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (every box here has one MI355X); run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    pkg = __graft_entry__.import_package()
    lib = pkg._lib.load()
    dev = torch.device("cuda:0")
    cfg = CFG
    layer, x, idx, weights, dy = build_workload(pkg, dev, cfg)
    params = list(layer.parameters())

    def step():
        for p in params:
            p.grad = None
        x.grad = None
        weights.grad = None
        out = layer(x, idx, weights)
        out.backward(dy)
        return out

    # warm-up on a side stream (also what graph capture needs), then optionally capture the step
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(max(args.warmup, 1)):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = None
    if args.graph:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        torch.cuda.synchronize()

    def run_step():
        if graph is not None:
            graph.replay()
        else:
            step()

    for _ in range(args.warmup):
        run_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3

    # per-launch durations of the tile kernel, HIP events on the launch stream, eager steps
    lib.ggq_profile_begin()
    prof_steps = min(args.steps, 10)
    for _ in range(prof_steps):
        step()
    torch.cuda.synchronize()
    cap = 8192
    ms = (ctypes.c_float * cap)()
    qt = (ctypes.c_int * cap)()
    mode = (ctypes.c_int * cap)()
    epi = (ctypes.c_int * cap)()
    n = lib.ggq_profile_end(ms, qt, mode, epi, cap)
    fl = algorithmic_flops(cfg)
    per_mode = {0: [], 1: []}
    for j in range(max(n, 0)):
        per_mode[mode[j]].append(ms[j])
    names = {0: "mmq_direct_q4k_kernel (Q4_K, forward, store)", 1: "mmq_mixed_kernel<Q4_K, grad_input, store>"}
    dominant = max(per_mode, key=lambda m: sum(per_mode[m]))
    launches = len(per_mode[dominant])
    avg_ms = sum(per_mode[dominant]) / max(launches, 1)
    # each step launches the kernel twice per direction: gate/up (pair) and down
    flops_per_launch = (fl["gate_up"] + fl["down"]) / 2
    achieved = flops_per_launch / (avg_ms * 1e-3) / 1e12 if launches else 0.0
    kernel_ms_per_step = {names[m]: sum(v) / prof_steps for m, v in per_mode.items()}
    # HBM bytes per launch (fetched + written, average of the gate/up and down launches) from the FETCH_SIZE /
    # WRITE_SIZE counter runs summarised in profiles/mmq_direct_and_mixed_q4k_grouped_moe_lora_step.pmc_traffic.txt;
    # the counters are collected offline, so this figure only changes when that profile is redone.
    traffic_bytes = {0: 572.1e6 + 100.7e6, 1: 343.6e6 + 83.9e6}[dominant]

    result = {
        "metric": "fwd+bwd TFLOP/s and weight GB/s, Q4_K grouped-MoE LoRA; % of MI355X roofline",
        "value": fl["total"] / (ms_per_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "configs[2]: grouped-MoE Q4_K LoRA fwd+bwd, 4096 tokens x top-8 = 32768 routes, hidden 2048, 256 experts, gate_up [1024x2048], down [2048x512], r=16 alpha=32",
                   "launch": "hip-graph replay" if graph is not None else "eager"},
        "weight_gb_per_s": 2 * packed_weight_bytes(cfg) / (ms_per_step * 1e-3) / 1e9,
        "pct_of_mfma_peak": 100.0 * fl["total"] / (ms_per_step * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        "pct_of_hbm_peak_weights": 100.0 * 2 * packed_weight_bytes(cfg) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "roofline": {"bound": "mfma", "kernel": names[dominant], "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": traffic_bytes, "avg_launch_ms": avg_ms, "launches_timed": launches,
                     "flops_per_launch": flops_per_launch},
        "tile_kernel_ms_per_step": kernel_ms_per_step,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
