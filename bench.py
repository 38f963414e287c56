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


def other_workload(name, pkg, lib, dev, args):
    """The other BASELINE configurations, timed the same way (eager launches): not the headline line, but the same JSON
    shape, so that their kernels can be traced with the same command."""
    g = torch.Generator(device=dev).manual_seed(3)

    def bf(*shape, std=1.0):
        return (torch.randn(*shape, generator=g, device=dev) * std).to(torch.bfloat16)

    if name == "dense_q4k":  # configs[1]
        n, k, rows = 4096, 2048, 4096
        payload = pkg.gguf.quantize_q4_k(torch.randn(n, k, generator=g, device=dev) * 0.02)
        x, a, b = bf(rows, k).requires_grad_(True), bf(16, k, std=k ** -0.5).requires_grad_(True), bf(n, 16, std=0.01).requires_grad_(True)
        dy = bf(rows, n)
        flops = 2 * 2 * rows * n * k + 3 * 2 * rows * 16 * (n + k)
        launch_flops, launches_per_step = 2 * rows * n * k, 2
        workload = "configs[1]: dense Q4_K LoRA linear fwd+bwd, W [4096x2048], X [4096, 2048], r=16 alpha=32"
        metric = "fwd+bwd TFLOP/s, dense Q4_K LoRA linear"

        def step():
            x.grad = a.grad = b.grad = None
            pkg.fast_lora.lora_mmq(x, payload, 12, n, a, b, 2.0).backward(dy)
    elif name == "lmhead_q6k":  # configs[3]
        vocab, hidden, rows, chunk = 151936, 2048, 4096, args.chunk
        payload = torch.cat([pkg.gguf.quantize_q6_k(torch.randn(min(18992, vocab - lo), hidden, generator=g, device=dev) * 0.02)
                             for lo in range(0, vocab, 18992)], dim=0)
        hs = bf(rows, hidden).requires_grad_(True)
        labels = torch.randint(0, vocab, (rows,), device=dev, generator=g)
        labels[torch.rand(rows, device=dev, generator=g) < 0.05] = -100
        flops = 2 * 2 * rows * vocab * hidden
        launch_flops, launches_per_step = None, None   # launches of different sizes (statistics per chunk, one grad-input)
        workload = f"configs[3]: chunked cross-entropy through a Q6_K lm_head [151936x2048], 4096 rows, chunks of {chunk}, loss + dHidden"
        metric = "fwd+bwd TFLOP/s (two algorithmic GEMMs), chunked lm_head cross-entropy"

        def step():
            hs.grad = None
            pkg.gguf_liger_loss.packed_linear_cross_entropy(hs, payload, labels, 14, vocab, chunk).backward()
    elif name == "moe_iq2xxs":  # configs[4], routed experts
        tokens, hidden, inter, e, top_k, r = 2048, 4096, 2048, 256, 8, 16
        G = pkg.gguf.GGUFQuantizedTensor
        gate = G(pkg.gguf.random_iq2_xxs((e, inter, hidden), g, dev), 16, (e, inter, hidden))
        up = G(pkg.gguf.random_iq2_xxs((e, inter, hidden), g, dev), 16, (e, inter, hidden))
        down = G(pkg.gguf.random_iq2_xxs((e, hidden, inter), g, dev), 16, (e, hidden, inter))
        layer = pkg.fast_moe_lora.FastGGUFMoeLora(pkg.fast_moe_lora.GGUFExperts(gate, up, down), r=r, lora_alpha=32)
        with torch.no_grad():
            for pname, p in layer.named_parameters():
                p.copy_(bf(*p.shape, std=p.shape[-1] ** -0.5 if "lora_A" in pname else 0.01))
        x = bf(tokens, hidden).requires_grad_(True)
        top = torch.topk(torch.randn(tokens, e, generator=g, device=dev), top_k, dim=-1)
        idx, weights = top.indices, torch.softmax(top.values, dim=-1).requires_grad_(True)
        dy = bf(tokens, hidden)
        routes = tokens * top_k
        flops = 2 * 2 * routes * (2 * inter * hidden + hidden * inter) + 3 * 2 * routes * r * ((hidden + 2 * inter) + (inter + hidden))
        launch_flops, launches_per_step = 2 * routes * (2 * inter * hidden + hidden * inter) / 2, 4
        workload = "configs[4] routed experts: grouped-MoE IQ2_XXS LoRA fwd+bwd, 2048 tokens x top-8, hidden 4096, 256 experts, gate_up [4096x4096], down [4096x2048], r=16 alpha=32"
        metric = "fwd+bwd TFLOP/s, IQ2_XXS grouped-MoE LoRA"
        params = list(layer.parameters())

        def step():
            for p in params:
                p.grad = None
            x.grad = weights.grad = None
            layer(x, idx, weights).backward(dy)
    else:
        sys.exit(f"unknown workload {name!r}")

    for _ in range(max(args.warmup, 1)):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    lib.ggq_profile_begin()
    prof_steps = min(args.steps, 5)
    for _ in range(prof_steps):
        step()
    torch.cuda.synchronize()
    cap = 8192
    ms, qt, mode, epi = (ctypes.c_float * cap)(), (ctypes.c_int * cap)(), (ctypes.c_int * cap)(), (ctypes.c_int * cap)()
    n_l = max(lib.ggq_profile_end(ms, qt, mode, epi, cap), 0)
    tile_ms = sum(ms[j] for j in range(n_l)) / prof_steps
    roofline = None
    if launch_flops is not None and n_l:
        avg_ms = tile_ms / launches_per_step
        achieved = launch_flops / (avg_ms * 1e-3) / 1e12
        roofline = {"bound": "mfma", "kernel": "packed-weight tile kernels (all launches of the step)", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS,
                    "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": None, "avg_launch_ms": avg_ms, "launches_timed": n_l}
    print(json.dumps({
        "metric": metric, "value": flops / (ms_per_step * 1e-3) / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": workload, "launch": "eager"}, "roofline": roofline, "tile_kernel_ms_per_step": tile_ms, "tile_kernel_launches_per_step": n_l / prof_steps}))


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="moe_q4k", choices=["moe_q4k", "dense_q4k", "lmhead_q6k", "moe_iq2xxs"],
                    help="moe_q4k (default) is the headline configuration; the others are timed for reference")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--chunk", type=int, default=1024, help="lmhead_q6k: rows per chunk (1024 in the BASELINE configuration; from 4096 rows on the logits of a chunk are kept)")
    ap.add_argument("--graph", type=int, default=1, help="replay the step from a captured HIP graph (1) or run it eagerly (0)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (every box here has one MI355X); run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    pkg = __graft_entry__.import_package()
    lib = pkg._lib.load()
    dev = torch.device("cuda:0")
    if args.workload != "moe_q4k":
        other_workload(args.workload, pkg, lib, dev, args)
        return
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
