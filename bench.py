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
SEED = 19260817  # + the index of the BASELINE configuration; every input is drawn on the host from this seed

_TYPE_NAMES = {8: "Q8_0", 10: "Q2_K", 11: "Q3_K", 12: "Q4_K", 13: "Q5_K", 14: "Q6_K", 16: "IQ2_XXS"}


def kernel_name(qt: int, mode: int, epi: int, shape: int) -> str:
    """Name of the kernel a profiled launch ran, from the record ggq_profile_end returns for it."""
    direction = "forward" if mode == 0 else "grad_input"
    if shape == 3:
        return "mmq_direct8_q4k_kernel (Q4_K, forward)" if mode == 0 else "mmq_direct8_nn_q4k_kernel (Q4_K, grad_input)"
    if shape == 4:
        return f"mmq_mixed_kernel<{_TYPE_NAMES.get(qt, qt)}, {direction}, store>"
    if shape == 5:
        return "mmq_small_iq2xxs_kernel (IQ2_XXS, forward)"
    return f"mmq_tile_kernel<{_TYPE_NAMES.get(qt, qt)}, {direction}, {'store' if epi == 0 else 'accumulate_f32'}, {'tall' if shape == 0 else 'wide'}>"


def profiled_launches(lib, cap=8192):
    """[(kernel name, ms)] of the launches recorded since ggq_profile_begin."""
    ms, qt, mode, epi, shape = (ctypes.c_float * cap)(), (ctypes.c_int * cap)(), (ctypes.c_int * cap)(), (ctypes.c_int * cap)(), (ctypes.c_int * cap)()
    n = max(lib.ggq_profile_end(ms, qt, mode, epi, shape, cap), 0)
    return [(kernel_name(qt[j], mode[j], epi[j], shape[j]), ms[j]) for j in range(n)]


def measured_traffic(kernel: str):
    """(bytes per launch, source file) of a kernel's HBM traffic from the committed counter summaries: lines
    'bench.traffic_bytes <kernel name, spaces as written> = <bytes>' in profiles/*pmc_traffic.txt; (None, None) when the
    kernel that ran has no such line (the counters are collected offline, in runs of their own)."""
    import glob

    root = os.path.dirname(os.path.abspath(__file__))
    for path in sorted(glob.glob(os.path.join(root, "profiles", "*pmc_traffic.txt"))):
        with open(path) as f:
            for line in f:
                if line.startswith("bench.traffic_bytes ") and "=" in line:
                    name, value = line[len("bench.traffic_bytes "):].rsplit("=", 1)
                    if name.strip() == kernel:
                        return float(value), os.path.relpath(path, root)
    return None, None


def host_randn(gen, *shape, std=1.0, dtype=torch.float32, device=None):
    t = torch.randn(*shape, generator=gen) * std
    return t.to(dtype).to(device) if device is not None else t.to(dtype)


def device_ceilings(pkg, lib, dev, x_samples, w_samples):
    """What this box sustains, next to the nominal peaks: the bf16 MFMA rate of a register-only loop with operands drawn
    from the workload's activations and decoded weights (and with all-zero operands: the device is power limited and its
    clock depends on the data), and the rate of a device-to-device copy."""
    out = {}
    tf = ctypes.c_float()
    n = min(x_samples.numel(), w_samples.numel()) // 8 * 8
    a, b = x_samples.reshape(-1)[:n].contiguous(), w_samples.reshape(-1)[:n].contiguous()
    st = pkg._lib.stream_handle(dev)
    sink = torch.zeros(64, dtype=torch.float32, device=dev)  # 256 bytes the measuring kernel may write
    if lib.ggq_measure_mfma_ceiling(a.data_ptr(), b.data_ptr(), n, 20000, sink.data_ptr(), ctypes.byref(tf), st) == 0:
        out["mfma_bf16_tflops_workload_values"] = tf.value
    z = torch.zeros(n, dtype=torch.bfloat16, device=dev)
    if lib.ggq_measure_mfma_ceiling(z.data_ptr(), z.data_ptr(), n, 20000, sink.data_ptr(), ctypes.byref(tf), st) == 0:
        out["mfma_bf16_tflops_zero_values"] = tf.value
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    dst.copy_(src)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    out["device_copy_gb_per_s"] = 5 * 2 * src.numel() / (e0.elapsed_time(e1) * 1e-3) / 1e9  # bytes read + bytes written
    return out

def timed_tflops(fn, flops, iters=30):
    for _ in range(3):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return flops * iters / (e0.elapsed_time(e1) * 1e-3) / 1e12


def library_gemm_ceilings(pkg, dev, cfg, layer, x):
    """What the framework's tuned dense bf16 GEMMs (hipBLASLt through torch.matmul / torch.bmm) reach on this box with the
    workload's values and shapes, weights already DECODED to bf16: the share of the gap to the MFMA peak that belongs to the GEMM structure
    (operands through LDS, tile edges, 128-row groups), as opposed to decoding packed weights and ragged grouping.
    configs[2] as a batched product over equal groups of 128 rows (the packed-weight kernels see 128 +- 11 rows and decode
    as they go); configs[1] as one dense product.  Not part of the timed step."""
    out = {}
    e, h, i = cfg["experts"], cfg["hidden"], cfg["inter"]
    rows = cfg["tokens"] * cfg["top_k"] // e
    with torch.no_grad():
        base = layer.base_layer
        w_gate = pkg.gguf.dequantize_gguf_tensor(base.gate_proj, 12, torch.bfloat16)  # [e, i, h]
        w_up = pkg.gguf.dequantize_gguf_tensor(base.up_proj, 12, torch.bfloat16)
        w_gu = torch.cat([w_gate, w_up], dim=1)  # [e, 2i, h]
        del w_gate, w_up
        w_down = pkg.gguf.dequantize_gguf_tensor(base.down_proj, 12, torch.bfloat16)  # [e, h, i]
        xs = x.detach()[: e * rows // 8].repeat(8, 1).reshape(e, rows, h).contiguous()  # token rows, as the routed rows are
        dgu = torch.randn(e, rows, 2 * i, device=dev, dtype=torch.bfloat16)
        hs = torch.randn(e, rows, i, device=dev, dtype=torch.bfloat16)
        dys = torch.randn(e, rows, h, device=dev, dtype=torch.bfloat16)
        f_gu, f_d = 2.0 * e * rows * 2 * i * h, 2.0 * e * rows * h * i
        out["bmm_gate_up_forward_tflops"] = timed_tflops(lambda: torch.bmm(xs, w_gu.transpose(1, 2)), f_gu)
        out["bmm_gate_up_grad_input_tflops"] = timed_tflops(lambda: torch.bmm(dgu, w_gu), f_gu)
        out["bmm_down_forward_tflops"] = timed_tflops(lambda: torch.bmm(hs, w_down.transpose(1, 2)), f_d)
        out["bmm_down_grad_input_tflops"] = timed_tflops(lambda: torch.bmm(dys, w_down), f_d)
        out["bmm_shapes"] = f"{e} groups x {rows} rows: [{rows}x{h}]x[{h}x{2 * i}] and [{rows}x{i}]x[{i}x{h}], forward (weights [n][k]) and grad-input"
        # configs[1]: X [4096, 2048] x W [4096, 2048]^T and dY [4096, 4096] x W
        wd = w_gu.reshape(-1, h)[:4096].contiguous()
        xd = x.detach()[:4096].contiguous()
        dyd = torch.randn(4096, 4096, device=dev, dtype=torch.bfloat16)
        f = 2.0 * 4096 * 4096 * h
        out["matmul_dense_forward_tflops"] = timed_tflops(lambda: torch.matmul(xd, wd.t()), f)
        out["matmul_dense_grad_input_tflops"] = timed_tflops(lambda: torch.matmul(dyd, wd), f)
        out["matmul_shapes"] = "configs[1]: [4096x2048]x[2048x4096] forward, [4096x4096]x[4096x2048] grad-input"
    return out


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


def build_workload(pkg, dev, cfg, seed=SEED + 2):
    """Every value is drawn on the host from one CPU generator (the bytes are the same on every box) and copied over; the
    fp32 expert weights are quantized to Q4_K on the device in slices of 32 experts."""
    g = torch.Generator().manual_seed(seed)
    e, h, i, r = cfg["experts"], cfg["hidden"], cfg["inter"], cfg["rank"]
    G = pkg.gguf.GGUFQuantizedTensor

    def packed(shape):
        out = []
        for lo in range(0, e, 32):  # in slices, to bound the fp32 staging memory
            out.append(pkg.gguf.quantize_q4_k(host_randn(g, min(32, e - lo), *shape, std=0.02, device=dev)))
        return torch.cat(out, dim=0)

    gate = G(packed((i, h)), 12, (e, i, h))
    up = G(packed((i, h)), 12, (e, i, h))
    down = G(packed((h, i)), 12, (e, h, i))
    experts = pkg.fast_moe_lora.GGUFExperts(gate, up, down)
    layer = pkg.fast_moe_lora.FastGGUFMoeLora(experts, r=r, lora_alpha=cfg["alpha"])
    with torch.no_grad():
        layer.lora_A["default"].weight.copy_(host_randn(g, e, r, h, std=h ** -0.5, dtype=torch.bfloat16))
        layer.lora_B["default"].weight.copy_(host_randn(g, e, 2 * i, r, std=0.01, dtype=torch.bfloat16))
        layer.lora_A_down["default"].weight.copy_(host_randn(g, e, r, i, std=i ** -0.5, dtype=torch.bfloat16))
        layer.lora_B_down["default"].weight.copy_(host_randn(g, e, h, r, std=0.01, dtype=torch.bfloat16))
    x = host_randn(g, cfg["tokens"], h, dtype=torch.bfloat16, device=dev).requires_grad_(True)
    logits = host_randn(g, cfg["tokens"], e)
    top = torch.topk(logits, cfg["top_k"], dim=-1)  # on the host: ties (none in practice) resolve the same way everywhere
    idx = top.indices.to(dev)
    weights = torch.softmax(top.values, dim=-1).to(dev).requires_grad_(True)
    dy = host_randn(g, cfg["tokens"], h, dtype=torch.bfloat16, device=dev)
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
    g = torch.Generator().manual_seed(SEED + {"dense_q4k": 1, "lmhead_q6k": 3, "moe_iq2xxs": 4}.get(name, 0))  # host generator: same bytes on every box
    gd = torch.Generator(device=dev).manual_seed(SEED)  # only for the arbitrary-byte IQ2_XXS payloads (1.7 GB of them)

    def bf(*shape, std=1.0):
        return host_randn(g, *shape, std=std, dtype=torch.bfloat16, device=dev)

    if name == "dense_q4k":  # configs[1]
        n, k, rows = 4096, 2048, 4096
        payload = pkg.gguf.quantize_q4_k(host_randn(g, n, k, std=0.02, device=dev))
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
        payload = torch.cat([pkg.gguf.quantize_q6_k(host_randn(g, min(18992, vocab - lo), hidden, std=0.02, device=dev))
                             for lo in range(0, vocab, 18992)], dim=0)
        hs = bf(rows, hidden).requires_grad_(True)
        labels = torch.randint(0, vocab, (rows,), generator=g)
        labels[torch.rand(rows, generator=g) < 0.05] = -100
        labels = labels.to(dev)
        flops = 2 * 2 * rows * vocab * hidden
        launch_flops, launches_per_step = None, None   # launches of different sizes (statistics per chunk, one grad-input)
        workload = f"configs[3]: chunked cross-entropy through a Q6_K lm_head [151936x2048], 4096 rows, chunks of {chunk}, loss + dHidden"
        metric = "fwd+bwd TFLOP/s (two algorithmic GEMMs), chunked lm_head cross-entropy"

        def step():
            hs.grad = None
            pkg.gguf_liger_loss.packed_linear_cross_entropy(hs, payload, labels, 14, vocab, chunk).backward()
    elif name == "moe_iq2xxs":  # configs[4]: routed IQ2_XXS experts plus the shared Q8_0 expert
        tokens, hidden, inter, e, top_k, r, s_lora = 2048, 4096, 2048, 256, 8, 16, 2.0
        G = pkg.gguf.GGUFQuantizedTensor

        def quantized_experts(n_out, k_in):
            # every expert drawn from N(0, 0.02^2) on the device (1.6 G weights per projection) and quantized there by the
            # restatement of the oracle's IQ2_XXS quantizer (bit-checked against it in tests/test_gpu_dequant.py)
            # (--iq2-pool N < 256 quantizes N distinct experts and repeats them: every expert still has its own bytes in HBM)
            out = torch.empty(e, n_out, k_in // 256 * 66, dtype=torch.uint8, device=dev)
            pool = max(1, min(e, args.iq2_pool))
            for j in range(pool):
                out[j] = pkg.gguf.quantize_iq2_xxs(torch.randn(n_out, k_in, generator=gd, device=dev) * 0.02)
            for j in range(pool, e):
                out[j] = out[j % pool]
            return G(out, 16, (e, n_out, k_in))

        gate, up, down = quantized_experts(inter, hidden), quantized_experts(inter, hidden), quantized_experts(hidden, inter)
        layer = pkg.fast_moe_lora.FastGGUFMoeLora(pkg.fast_moe_lora.GGUFExperts(gate, up, down), r=r, lora_alpha=32)
        with torch.no_grad():
            for pname, p in layer.named_parameters():
                p.copy_(bf(*p.shape, std=p.shape[-1] ** -0.5 if "lora_A" in pname else 0.01))
        # the shared expert: gate / up / down of the same shapes in Q8_0, a rank-16 LoRA on each, run as a SiLU FFN on every token
        shared = {}
        for pname, (n_out, k_in) in (("gate", (inter, hidden)), ("up", (inter, hidden)), ("down", (hidden, inter))):
            shared[pname] = (pkg.gguf.quantize_q8_0(host_randn(g, n_out, k_in, std=0.02, device=dev)), n_out,
                             bf(r, k_in, std=k_in ** -0.5).requires_grad_(True), bf(n_out, r, std=0.01).requires_grad_(True))
        shared_params = [t for v in shared.values() for t in v[2:]]

        def shared_ffn(h):
            g_, u_ = (pkg.fast_lora.lora_mmq(h, shared[n][0], 8, shared[n][1], shared[n][2], shared[n][3], s_lora) for n in ("gate", "up"))
            return pkg.fast_lora.lora_mmq(pkg.fast_moe_lora.swiglu(g_, u_), shared["down"][0], 8, hidden, shared["down"][2], shared["down"][3], s_lora)

        x = bf(tokens, hidden).requires_grad_(True)
        top = torch.topk(host_randn(g, tokens, e), top_k, dim=-1)
        idx, weights = top.indices.to(dev), torch.softmax(top.values, dim=-1).to(dev).requires_grad_(True)
        dy = bf(tokens, hidden)
        routes = tokens * top_k
        per_row = 2 * inter * hidden + hidden * inter
        lora_per_row = 3 * 2 * r * ((hidden + 2 * inter) + (inter + hidden))
        flops_routed = 2 * 2 * routes * per_row + routes * lora_per_row
        flops_shared = 2 * 2 * tokens * per_row + tokens * lora_per_row
        flops = flops_routed + flops_shared
        launch_flops, launches_per_step = None, None  # routed and shared launches differ; per-kernel figures are in `by_kernel_ms_per_step`
        workload = ("configs[4]: grouped-MoE IQ2_XXS LoRA fwd+bwd, 2048 tokens x top-8, hidden 4096, 256 routed experts quantized from N(0, 0.02^2), gate_up [4096x4096], "
                    "down [4096x2048], plus the shared Q8_0 expert of the same shapes on every token, r=16 alpha=32 on all projections"
                    + ("" if args.iq2_pool >= e else f" ({args.iq2_pool} distinct experts, repeated)"))
        metric = "fwd+bwd TFLOP/s, IQ2_XXS grouped-MoE LoRA with the shared Q8_0 expert"
        params = list(layer.parameters())

        def step_routed():
            for p in params:
                p.grad = None
            x.grad = weights.grad = None
            layer(x, idx, weights).backward(dy)

        def step_shared():
            for p in shared_params:
                p.grad = None
            x.grad = None
            shared_ffn(x).backward(dy)

        def step():
            for p in params + shared_params:
                p.grad = None
            x.grad = weights.grad = None
            (layer(x, idx, weights) + shared_ffn(x)).backward(dy)

        def timed(fn, n):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / n * 1e3

        extra = {"routed_experts_ms_per_step": timed(step_routed, args.steps), "shared_expert_ms_per_step": timed(step_shared, args.steps),
                 "routed_experts_tflops": None, "shared_expert_tflops": None}
        # algorithmic flops of a direction's packed-weight launches per step, by the block format in the launch record
        extra["_direction_flops"] = {"IQ2_XXS": 2 * routes * per_row, "Q8_0": 2 * tokens * per_row}
        extra["routed_experts_tflops"] = flops_routed / (extra["routed_experts_ms_per_step"] * 1e-3) / 1e12
        extra["shared_expert_tflops"] = flops_shared / (extra["shared_expert_ms_per_step"] * 1e-3) / 1e12
    elif name == "moe_q4k_separated":  # configs[2] through the reference's own order: base launches + separate grouped LoRA products
        cfg = CFG
        layer, x, idx, weights, dy = build_workload(pkg, dev, cfg)
        layer.get_base_layer().experts_implementation = pkg.fast_moe_lora.SEPARATED_EXPERTS_IMPLEMENTATION
        fl = algorithmic_flops(cfg)
        flops = fl["total"]
        launch_flops, launches_per_step = fl["base_total"] / 4, 4
        workload = ("configs[2] in the reference's order (fast_moe_lora.py:685-770): packed-weight launches without the LoRA term, each LoRA delta as "
                    "two grouped bf16 products (gmm) added afterwards, factor gradients by ptgmm, gather / activation / combine as separate nodes")
        metric = "fwd+bwd TFLOP/s, Q4_K grouped-MoE LoRA, separated order"
        params = list(layer.parameters())

        def step():
            for p in params:
                p.grad = None
            x.grad = weights.grad = None
            layer(x, idx, weights).backward(dy)
    else:
        sys.exit(f"unknown workload {name!r}")

    extra = locals().get("extra", {})
    for _ in range(max(args.warmup, 1)):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    lib.ggq_set_factor_gradient_overlap(0)  # per-launch event times of a launch alone on its stream (see main())
    lib.ggq_profile_begin()
    prof_steps = min(args.steps, 5)
    for _ in range(prof_steps):
        step()
    torch.cuda.synchronize()
    launches = profiled_launches(lib)
    lib.ggq_set_factor_gradient_overlap(1 if args.overlap else 0)
    n_l = len(launches)
    tile_ms = sum(t for _, t in launches) / prof_steps
    by_kernel = {}
    for nm, t in launches:
        by_kernel.setdefault(nm, []).append(t)
    roofline = None
    direction_flops = extra.pop("_direction_flops", None)
    if direction_flops and by_kernel:
        # per kernel: the direction's algorithmic flops over the time its launches take per step; `roofline` = the dominant one
        fracs = {}
        for nm, ts in by_kernel.items():
            fl_dir = next((v for k, v in direction_flops.items() if f"{k}," in nm), None)
            if fl_dir and sum(ts) / prof_steps > 0.1:  # (a launch whose tile table came out empty on the device is no measurement)
                fracs[nm] = fl_dir / (sum(ts) / prof_steps * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS
        extra["kernel_frac_of_mfma_peak"] = fracs
        dominant = max(by_kernel, key=lambda k: sum(by_kernel[k]))
        if dominant in fracs:
            roofline = {"bound": "mfma", "kernel": dominant, "achieved": fracs[dominant] * MFMA_BF16_PEAK_TFLOPS, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                        "frac": fracs[dominant], "traffic": None, "avg_launch_ms": sum(by_kernel[dominant]) / len(by_kernel[dominant]), "launches_timed": len(by_kernel[dominant])}
    if launch_flops is not None and n_l:
        avg_ms = tile_ms / launches_per_step
        achieved = launch_flops / (avg_ms * 1e-3) / 1e12
        roofline = {"bound": "mfma", "kernel": " + ".join(sorted(by_kernel)), "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS,
                    "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": None, "avg_launch_ms": avg_ms, "launches_timed": n_l}
    print(json.dumps({
        "metric": metric, "value": flops / (ms_per_step * 1e-3) / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": workload, "launch": "eager"}, "roofline": roofline, "tile_kernel_ms_per_step": tile_ms, "tile_kernel_launches_per_step": n_l / prof_steps,
        "by_kernel_ms_per_step": {k: sum(v) / prof_steps for k, v in by_kernel.items()}, **extra}))


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="moe_q4k", choices=["moe_q4k", "dense_q4k", "lmhead_q6k", "moe_iq2xxs", "moe_q4k_separated"],
                    help="moe_q4k (default) is the headline configuration; the others are timed for reference")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--settle-ms", type=float, default=300.0, help="moe_q4k: milliseconds of untimed step replays ahead of the warm-up steps (0: none)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--chunk", type=int, default=1024, help="lmhead_q6k: rows per chunk (1024 in the BASELINE configuration; from 4096 rows on the logits of a chunk are kept)")
    ap.add_argument("--graph", type=int, default=1, help="replay the step from a captured HIP graph (1) or run it eagerly (0)")
    ap.add_argument("--iq2-pool", type=int, default=256, help="moe_iq2xxs: number of distinct experts drawn and quantized (the others repeat them)")
    ap.add_argument("--overlap", type=int, default=1, help="factor gradients of the grouped backward calls on the library's side stream (1, the library's default) or on the launch stream (0)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (every box here has one MI355X); run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    pkg = __graft_entry__.import_package()
    lib = pkg._lib.load()
    dev = torch.device("cuda:0")
    lib.ggq_set_factor_gradient_overlap(1 if args.overlap else 0)
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

    # Settle: the device comes out of the set-up above (host-paced quantization, capture) at idle clocks and cold
    # translation caches, and its first few dozen steps run 5-6 % slower than the ones after them; a training run spends
    # its life in the sustained state.  The step is replayed for --settle-ms milliseconds (untimed, like the warm-up steps
    # that follow) so that the timed region measures that state whatever --steps is.
    t_settle = time.perf_counter()
    settle_steps = 0
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        for _ in range(10):
            run_step()
        torch.cuda.synchronize()
        settle_steps += 10
    for _ in range(args.warmup):
        run_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3

    # per-launch durations of the packed-weight kernels, HIP events on the launch stream, eager steps.  For these steps the
    # factor gradients stay on the launch stream: forked (the default, and what the timed region above ran) they share the
    # compute units with the grad-input launch, whose event pair would then time both.
    lib.ggq_set_factor_gradient_overlap(0)
    lib.ggq_profile_begin()
    prof_steps = min(args.steps, 10)
    for _ in range(prof_steps):
        step()
    torch.cuda.synchronize()
    launches = profiled_launches(lib)
    lib.ggq_set_factor_gradient_overlap(1 if args.overlap else 0)
    fl = algorithmic_flops(cfg)
    by_kernel = {}
    for nm, t in launches:
        by_kernel.setdefault(nm, []).append(t)
    dominant = max(by_kernel, key=lambda k: sum(by_kernel[k])) if by_kernel else "none"
    n_launches = len(by_kernel.get(dominant, []))
    avg_ms = sum(by_kernel.get(dominant, [])) / max(n_launches, 1)
    # each step launches a direction's kernel twice: gate/up (pair) and down; the figure is their average
    flops_per_launch = (fl["gate_up"] + fl["down"]) / 2
    achieved = flops_per_launch / (avg_ms * 1e-3) / 1e12 if n_launches else 0.0
    kernel_ms_per_step = {k: sum(v) / prof_steps for k, v in by_kernel.items()}
    traffic_bytes, traffic_source = measured_traffic(dominant)
    # operands with the workload's statistics for the on-box MFMA ceiling: token activations and decoded expert weights
    with torch.no_grad():
        w_samples = pkg.gguf.dequantize_gguf_tensor(layer.base_layer.gate_proj.as_subclass(torch.Tensor)[0].contiguous(), 12, torch.bfloat16)
    ceilings = device_ceilings(pkg, lib, dev, x.detach(), w_samples)
    ceilings["library_bf16_gemm_on_decoded_weights"] = library_gemm_ceilings(pkg, dev, cfg, layer, x)

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
                   "launch": "hip-graph replay" if graph is not None else "eager",
                   "factor_gradients": "forked onto the library's side stream" if args.overlap else "on the launch stream",
                   "settle": f"{settle_steps} untimed steps ({args.settle_ms:.0f} ms) ahead of the {args.warmup} warm-up steps, so that the timed steps run at sustained clocks"},
        "weight_gb_per_s": 2 * packed_weight_bytes(cfg) / (ms_per_step * 1e-3) / 1e9,
        "pct_of_mfma_peak": 100.0 * fl["total"] / (ms_per_step * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        "pct_of_hbm_peak_weights": 100.0 * 2 * packed_weight_bytes(cfg) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "roofline": {"bound": "mfma", "kernel": dominant, "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": traffic_bytes, "traffic_source": traffic_source, "avg_launch_ms": avg_ms,
                     "launches_timed": n_launches, "flops_per_launch": flops_per_launch,
                     "timed_with": "HIP events around each launch, eager steps, factor gradients on the launch stream"},
        "tile_kernel_ms_per_step": kernel_ms_per_step,
        "ceilings_on_this_box": ceilings,
        "frac_of_measured_mfma_ceiling": achieved / ceilings["mfma_bf16_tflops_workload_values"] if ceilings.get("mfma_bf16_tflops_workload_values") else None,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
