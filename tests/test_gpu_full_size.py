"""The headline shapes at full size, checked through properties whose cost does not grow with the oracle's: token-order
equivariance of the expert layer (bit-exact: every output row is computed independently of its neighbours), a sample of
expert groups against an fp32 matmul on the decoded weights, and the lm_head loss against a chunked torch reference
(tolerances of the path: outputs and gradients max rel err <= 2e-2, loss abs err <= 1e-3)."""

import pytest
import torch

import bench
from helpers import assert_close_bf16, max_rel

pytestmark = pytest.mark.gpu


def _bf16(t):
    return t.to(torch.bfloat16).float()


def test_expert_layer_at_full_size_is_token_order_equivariant(pkg, dev):
    # 4096 tokens x top-8 over 256 Q4_K experts, hidden 2048, r = 16: the bench's workload
    cfg = bench.CFG
    layer, x, idx, weights, dy = bench.build_workload(pkg, dev, cfg)
    out = layer(x, idx, weights)
    out.backward(dy)
    assert torch.isfinite(out).all() and out.shape == x.shape
    params = dict(layer.named_parameters())
    grads = {k: p.grad.clone() for k, p in params.items()}
    order = torch.randperm(cfg["tokens"], generator=torch.Generator().manual_seed(5)).to(dev)
    for p in params.values():
        p.grad = None
    x2 = x.detach()[order].requires_grad_(True)
    w2 = weights.detach()[order].requires_grad_(True)
    out2 = layer(x2, idx[order], w2)
    out2.backward(dy[order])
    assert torch.equal(out2, out[order]), "layer output"
    assert torch.equal(x2.grad, x.grad[order]), "token gradient"
    assert torch.equal(w2.grad, weights.grad[order]), "routing-weight gradient"
    # the factor gradients sum over an expert's rows in another order: equal to rounding
    for k, p in params.items():
        assert_close_bf16(p.grad, grads[k].double(), k, ulps=2.0)
    # experts no token chose get exactly zero factor gradients
    unused = torch.ones(cfg["experts"], dtype=torch.bool, device=dev)
    unused[idx.reshape(-1)] = False
    for k, g in grads.items():
        assert torch.count_nonzero(g[unused]) == 0, k


def test_sampled_expert_groups_at_full_size_match_an_fp32_matmul(pkg, dev):
    cfg = bench.CFG
    layer, x, idx, weights, _ = bench.build_workload(pkg, dev, cfg)
    ml, mr, experts = pkg.fast_moe_lora, pkg.fast_moe_routing, layer.base_layer
    e_total, inter, s = cfg["experts"], cfg["inter"], cfg["alpha"] / cfg["rank"]
    plan = mr.prepare_expert_routing(x.detach(), idx, weights.detach(), e_total)
    sel = plan.selected_hidden_states
    ids = torch.arange(e_total, dtype=torch.int64, device=dev)
    a, b = layer.lora_A["default"].weight.detach(), layer.lora_B["default"].weight.detach()
    dy1 = torch.randn(sel.shape[0], inter, generator=torch.Generator(device=dev).manual_seed(9), device=dev).to(torch.bfloat16)
    dy2 = torch.randn(sel.shape[0], inter, generator=torch.Generator(device=dev).manual_seed(10), device=dev).to(torch.bfloat16)
    xs = sel.detach().requires_grad_(True)
    y1, y2 = ml.grouped_lora_mmq_pair(xs, experts.gate_proj, experts.up_proj, ids, plan.expert_end_offsets, 12, inter, a, b, s)
    torch.autograd.backward((y1, y2), (dy1, dy2))
    # the launch that reads the token rows through the permutation gives the same bits as the one on the copy
    z1, z2 = ml._RoutedGroupedLoraProjection.apply(x.detach(), plan.permutation, plan.inverse_permutation, cfg["top_k"], experts.gate_proj.as_subclass(torch.Tensor),
                                                   experts.up_proj.as_subclass(torch.Tensor), ids, plan.expert_end_offsets, 12, inter, a, b, s)
    assert torch.equal(z1, y1) and torch.equal(z2, y2)
    ends = plan.expert_end_offsets.cpu().tolist()
    counts = plan.expert_counts.cpu()
    sample = sorted({0, 17, 100, e_total - 1, int(counts.argmax()), int(torch.where(counts > 0, counts, 10 ** 6).argmin())})
    for e in sample:
        r0, r1 = (ends[e - 1] if e else 0), ends[e]
        if r1 == r0:
            continue
        xe = sel[r0:r1].float()
        wg = _bf16(pkg.gguf.dequantize_gguf_tensor(experts.gate_proj[e:e + 1], 12, torch.float32)[0])
        wu = _bf16(pkg.gguf.dequantize_gguf_tensor(experts.up_proj[e:e + 1], 12, torch.float32)[0])
        xa = _bf16(xe @ a[e].float().T)
        want1 = xe @ wg.T + s * (xa @ b[e, :inter].float().T)
        want2 = xe @ wu.T + s * (xa @ b[e, inter:].float().T)
        assert_close_bf16(y1[r0:r1], want1.double(), f"gate of expert {e}")
        assert_close_bf16(y2[r0:r1], want2.double(), f"up of expert {e}")
        d1, d2 = dy1[r0:r1].float(), dy2[r0:r1].float()
        dyb = _bf16(d1 @ b[e, :inter].float() + d2 @ b[e, inter:].float())
        want_dx = d1 @ wg + d2 @ wu + s * (dyb @ a[e].float())
        assert_close_bf16(xs.grad[r0:r1], want_dx.double(), f"dX of expert {e}")


@pytest.mark.parametrize("chunk", [1024, 4096])
def test_lm_head_loss_at_full_size_matches_a_chunked_torch_reference(pkg, dev, chunk):
    # Qwen's head: 151936 x 2048 in Q6_K, 4096 rows; chunks of 1024 rows (no logits kept: one sweep over the vocabulary with a running softmax) and of
    # 4096 rows (the chunk's logits kept and rewritten as their gradient)
    vocab, hidden, rows = 151936, 2048, 4096
    g = torch.Generator(device=dev).manual_seed(31)
    payload = torch.cat([pkg.gguf.quantize_q6_k(torch.randn(min(18992, vocab - lo), hidden, generator=g, device=dev) * 0.02)
                         for lo in range(0, vocab, 18992)], dim=0)
    assert payload.shape[0] == vocab
    hid = (torch.randn(rows, hidden, generator=g, device=dev)).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (rows,), generator=g, device=dev)
    labels[torch.rand(rows, generator=g, device=dev) < 0.1] = -100
    h = hid.clone().requires_grad_(True)
    loss = pkg.gguf_liger_loss.packed_linear_cross_entropy(h, payload, labels, 14, vocab, chunk, -100, "mean")
    loss.backward()
    w = pkg.gguf.dequantize_gguf_tensor(payload, 14, torch.bfloat16).float()      # the path's weights are the bf16-rounded decoded values
    n_valid = int((labels != -100).sum())
    total = torch.zeros((), dtype=torch.float64, device=dev)
    want_dh = torch.empty(rows, hidden, dtype=torch.float32, device=dev)
    for r0 in range(0, rows, 512):
        hc, lc = hid[r0:r0 + 512].float(), labels[r0:r0 + 512]
        logits = _bf16(hc @ w.T)                                                   # logits are bf16 values
        lse = torch.logsumexp(logits, dim=1)
        valid = lc != -100
        tgt = logits.gather(1, lc.clamp(min=0)[:, None])[:, 0]
        total += ((lse - tgt) * valid).double().sum()
        d = torch.softmax(logits, dim=1)
        d[torch.arange(d.shape[0], device=dev), lc.clamp(min=0)] -= 1.0
        d = _bf16(d * (valid[:, None] / n_valid))                                  # the gradient slab is stored as bf16
        want_dh[r0:r0 + 512] = d @ w
    want_loss = float(total / n_valid)
    assert abs(float(loss) - want_loss) <= 1e-3, (float(loss), want_loss)
    assert max_rel(h.grad, want_dh) <= 2e-2
    cos = torch.nn.functional.cosine_similarity(h.grad.double().reshape(-1), want_dh.double().reshape(-1), dim=0)
    assert float(cos) > 0.9999
    assert bool((h.grad[labels == -100] == 0).all())


def test_dense_q4k_lora_linear_at_attention_projection_shape(pkg, dev):
    # W [4096 out x 2048 in] in Q4_K, X [4 x 1024, 2048], r = 16, alpha = 32: every output against fp32 matmuls on the decoded weights
    n, k, rows, r, s = 4096, 2048, 4096, 16, 2.0
    g = torch.Generator(device=dev).manual_seed(77)
    payload = pkg.gguf.quantize_q4_k(torch.randn(n, k, generator=g, device=dev) * 0.02)
    x = torch.randn(rows, k, generator=g, device=dev).to(torch.bfloat16).requires_grad_(True)
    a = (torch.randn(r, k, generator=g, device=dev) * k ** -0.5).to(torch.bfloat16).requires_grad_(True)
    b = (torch.randn(n, r, generator=g, device=dev) * 0.01).to(torch.bfloat16).requires_grad_(True)
    dy = torch.randn(rows, n, generator=g, device=dev).to(torch.bfloat16)
    y = pkg.fast_lora.lora_mmq(x, payload, 12, n, a, b, s)
    y.backward(dy)
    w = pkg.gguf.dequantize_gguf_tensor(payload, 12, torch.bfloat16).float()
    xf, af, bf, df = x.detach().float(), a.detach().float(), b.detach().float(), dy.float()
    xa = _bf16(xf @ af.T)
    dyb = _bf16(df @ bf)
    assert_close_bf16(y, (xf @ w.T + s * (xa @ bf.T)).double(), "Y")
    assert_close_bf16(x.grad, (df @ w + s * (dyb @ af)).double(), "dX")
    assert_close_bf16(a.grad, (s * (dyb.T @ xf)).double(), "dA")
    assert_close_bf16(b.grad, (s * (df.T @ xa)).double(), "dB")


def test_iq2_xxs_expert_layer_with_a_q8_0_shared_expert_at_full_size(pkg, dev):
    # 2048 tokens x top-8 over 256 IQ2_XXS experts (gate_up [4096 x 4096], down [4096 x 2048]), r = 16, and one shared
    # expert of the same shapes in Q8_0: token-order equivariance of the routed layer, sampled groups and the shared expert's
    # projections against fp32 matmuls on the decoded weights
    tokens, hidden, inter, e_total, top_k, r, s = 2048, 4096, 2048, 256, 8, 16, 2.0
    g = torch.Generator(device=dev).manual_seed(41)
    G = pkg.gguf.GGUFQuantizedTensor
    gate = G(pkg.gguf.random_iq2_xxs((e_total, inter, hidden), g, dev), 16, (e_total, inter, hidden))
    up = G(pkg.gguf.random_iq2_xxs((e_total, inter, hidden), g, dev), 16, (e_total, inter, hidden))
    down = G(pkg.gguf.random_iq2_xxs((e_total, hidden, inter), g, dev), 16, (e_total, hidden, inter))
    layer = pkg.fast_moe_lora.FastGGUFMoeLora(pkg.fast_moe_lora.GGUFExperts(gate, up, down), r=r, lora_alpha=32)
    with torch.no_grad():
        for name, p in layer.named_parameters():
            fan = p.shape[-1] if "lora_A" in name else None
            p.copy_((torch.randn(p.shape, generator=g, device=dev) * (fan ** -0.5 if fan else 0.01)).to(torch.bfloat16))
    x = torch.randn(tokens, hidden, generator=g, device=dev).to(torch.bfloat16).requires_grad_(True)
    top = torch.topk(torch.randn(tokens, e_total, generator=g, device=dev), top_k, dim=-1)
    idx, weights = top.indices, torch.softmax(top.values, dim=-1).requires_grad_(True)
    dy = torch.randn(tokens, hidden, generator=g, device=dev).to(torch.bfloat16)
    out = layer(x, idx, weights)
    out.backward(dy)
    assert torch.isfinite(out).all()
    order = torch.randperm(tokens, generator=torch.Generator().manual_seed(6)).to(dev)
    x2 = x.detach()[order].requires_grad_(True)
    w2 = weights.detach()[order].requires_grad_(True)
    out2 = layer(x2, idx[order], w2)
    out2.backward(dy[order])
    assert torch.equal(out2, out[order]) and torch.equal(x2.grad, x.grad[order]) and torch.equal(w2.grad, weights.grad[order])
    # sampled groups of the gate/up launch
    ml, mr = pkg.fast_moe_lora, pkg.fast_moe_routing
    plan = mr.prepare_expert_routing(x.detach(), idx, weights.detach(), e_total)
    ids = torch.arange(e_total, dtype=torch.int64, device=dev)
    a, b = layer.lora_A["default"].weight.detach(), layer.lora_B["default"].weight.detach()
    y1, y2 = ml.grouped_lora_mmq_pair(plan.selected_hidden_states, gate, up, ids, plan.expert_end_offsets, 16, inter, a, b, s)
    ends = plan.expert_end_offsets.cpu().tolist()
    for e in (0, 101, e_total - 1, int(plan.expert_counts.argmax())):
        r0, r1 = (ends[e - 1] if e else 0), ends[e]
        if r1 == r0:
            continue
        xe = plan.selected_hidden_states[r0:r1].float()
        wg = pkg.gguf.dequantize_gguf_tensor(gate[e:e + 1], 16, torch.bfloat16)[0].float()
        wu = pkg.gguf.dequantize_gguf_tensor(up[e:e + 1], 16, torch.bfloat16)[0].float()
        xa = _bf16(xe @ a[e].float().T)
        assert_close_bf16(y1[r0:r1], (xe @ wg.T + s * (xa @ b[e, :inter].float().T)).double(), f"gate of expert {e}")
        assert_close_bf16(y2[r0:r1], (xe @ wu.T + s * (xa @ b[e, inter:].float().T)).double(), f"up of expert {e}")
    # the shared expert: dense Q8_0 projections of the same shapes, LoRA on each
    for n_out, k_in in ((2 * inter, hidden), (hidden, inter)):
        payload = pkg.gguf.quantize_q8_0(torch.randn(n_out, k_in, generator=g, device=dev) * 0.02)
        xs = torch.randn(tokens, k_in, generator=g, device=dev).to(torch.bfloat16).requires_grad_(True)
        la = (torch.randn(r, k_in, generator=g, device=dev) * k_in ** -0.5).to(torch.bfloat16).requires_grad_(True)
        lb = (torch.randn(n_out, r, generator=g, device=dev) * 0.01).to(torch.bfloat16).requires_grad_(True)
        d = torch.randn(tokens, n_out, generator=g, device=dev).to(torch.bfloat16)
        y = pkg.fast_lora.lora_mmq(xs, payload, 8, n_out, la, lb, s)
        y.backward(d)
        w = pkg.gguf.dequantize_gguf_tensor(payload, 8, torch.bfloat16).float()
        xf, df = xs.detach().float(), d.float()
        xa, dyb = _bf16(xf @ la.detach().float().T), _bf16(df @ lb.detach().float())
        assert_close_bf16(y, (xf @ w.T + s * (xa @ lb.detach().float().T)).double(), "shared Y")
        assert_close_bf16(xs.grad, (df @ w + s * (dyb @ la.detach().float())).double(), "shared dX")
        assert_close_bf16(la.grad, (s * (dyb.T @ xf)).double(), "shared dA")
        assert_close_bf16(lb.grad, (s * (df.T @ xa)).double(), "shared dB")


def _expert_rows(ends, e):
    return (ends[e - 1] if e else 0), ends[e]


def test_down_projection_and_factor_gradients_of_sampled_experts_at_full_size(pkg, dev):
    # the bench's workload again: for a sample of experts (first, last, largest, smallest, two in between) the down
    # projection's forward and input gradient and the dA / dB of both projections against fp32 matmuls on the decoded
    # weights; for a sample of tokens the hidden-state gradient of the launch that reads tokens in place, summed over the
    # token's eight routes
    cfg = bench.CFG
    layer, x, idx, weights, _ = bench.build_workload(pkg, dev, cfg)
    ml, mr, experts = pkg.fast_moe_lora, pkg.fast_moe_routing, layer.base_layer
    e_total, inter, hidden, top_k, s = cfg["experts"], cfg["inter"], cfg["hidden"], cfg["top_k"], cfg["alpha"] / cfg["rank"]
    plan = mr.prepare_expert_routing(x.detach(), idx, weights.detach(), e_total)
    sel, rows = plan.selected_hidden_states, plan.selected_hidden_states.shape[0]
    ids = torch.arange(e_total, dtype=torch.int64, device=dev)
    gen = torch.Generator().manual_seed(77)

    def cot(*shape):
        return torch.randn(*shape, generator=gen).to(torch.bfloat16).to(dev)

    def leaf(p):
        return p.weight.detach().clone().requires_grad_(True)

    a, b, ad, bd = leaf(layer.lora_A["default"]), leaf(layer.lora_B["default"]), leaf(layer.lora_A_down["default"]), leaf(layer.lora_B_down["default"])
    dy1, dy2, dyd = cot(rows, inter), cot(rows, inter), cot(rows, hidden)
    y1, y2 = ml.grouped_lora_mmq_pair(sel, experts.gate_proj, experts.up_proj, ids, plan.expert_end_offsets, 12, inter, a, b, s)
    torch.autograd.backward((y1, y2), (dy1, dy2))
    act = ml.swiglu(y1.detach(), y2.detach()).requires_grad_(True)
    yd = ml.grouped_lora_mmq(act, experts.down_proj, ids, plan.expert_end_offsets, 12, hidden, ad, bd, s)
    yd.backward(dyd)
    ends = plan.expert_end_offsets.cpu().tolist()
    counts = plan.expert_counts.cpu()
    sample = sorted({0, 63, 190, e_total - 1, int(counts.argmax()), int(torch.where(counts > 0, counts, 10 ** 6).argmin())})
    for e in sample:
        r0, r1 = _expert_rows(ends, e)
        if r1 == r0:
            continue
        f = lambda t: t.detach().float()
        xe, d1, d2 = f(sel[r0:r1]), f(dy1[r0:r1]), f(dy2[r0:r1])
        xa = _bf16(xe @ f(a[e]).T)
        dyb = _bf16(d1 @ f(b[e, :inter]) + d2 @ f(b[e, inter:]))
        assert_close_bf16(a.grad[e], (s * (dyb.T @ xe)).double(), f"gate/up dA of expert {e}")
        assert_close_bf16(b.grad[e], (s * (torch.cat([d1, d2], dim=1).T @ xa)).double(), f"gate/up dB of expert {e}")
        wd = _bf16(pkg.gguf.dequantize_gguf_tensor(experts.down_proj[e:e + 1], 12, torch.float32)[0])
        ae, dd = f(act[r0:r1]), f(dyd[r0:r1])
        xad = _bf16(ae @ f(ad[e]).T)
        dybd = _bf16(dd @ f(bd[e]))
        assert_close_bf16(yd[r0:r1], (ae @ wd.T + s * (xad @ f(bd[e]).T)).double(), f"down of expert {e}")
        assert_close_bf16(act.grad[r0:r1], (dd @ wd + s * (dybd @ f(ad[e]))).double(), f"down dX of expert {e}")
        assert_close_bf16(ad.grad[e], (s * (dybd.T @ ae)).double(), f"down dA of expert {e}")
        assert_close_bf16(bd.grad[e], (s * (dd.T @ xad)).double(), f"down dB of expert {e}")
    # dHidden of the in-place launch: every route's dX rounded to bf16, then the token's eight routes added up
    xr = x.detach().clone().requires_grad_(True)
    z1, z2 = ml._RoutedGroupedLoraProjection.apply(xr, plan.permutation, plan.inverse_permutation, top_k, experts.gate_proj.as_subclass(torch.Tensor),
                                                   experts.up_proj.as_subclass(torch.Tensor), ids, plan.expert_end_offsets, 12, inter, a.detach(),
                                                   b.detach(), s)
    torch.autograd.backward((z1, z2), (dy1, dy2))
    inverse = plan.inverse_permutation.cpu().reshape(-1, top_k)
    idx_cpu = idx.cpu()
    for t in (0, 1, 2047, 4095):
        want = torch.zeros(hidden, dtype=torch.float64, device=dev)
        magnitude = torch.zeros(hidden, dtype=torch.float64, device=dev)
        for k in range(top_k):
            row, e = int(inverse[t, k]), int(idx_cpu[t, k])
            wg = _bf16(pkg.gguf.dequantize_gguf_tensor(experts.gate_proj[e:e + 1], 12, torch.float32)[0])
            wu = _bf16(pkg.gguf.dequantize_gguf_tensor(experts.up_proj[e:e + 1], 12, torch.float32)[0])
            d1, d2 = dy1[row].float(), dy2[row].float()
            dyb = _bf16(d1 @ b[e, :inter].detach().float() + d2 @ b[e, inter:].detach().float())
            term = _bf16(d1 @ wg + d2 @ wu + s * (dyb @ a[e].detach().float())).double()
            want += term
            magnitude += term.abs()
        # each of the eight adds rounds a partial sum no larger than the summed magnitudes to bf16 (half an ulp = 2^-9),
        # and each term carries the half ulp of its own rounding
        err = (xr.grad[t].double() - want).abs()
        assert bool((err <= (top_k + 1) * 2.0 ** -9 * magnitude + 1e-6).all()), f"dHidden of token {t}: worst {float((err / magnitude.clamp(min=1e-9)).max()):.3e} of the summed magnitude"
        assert max_rel(xr.grad[t], want) <= 2e-2


def test_iq2_xxs_experts_quantized_from_gaussian_weights_and_the_shared_ffn_at_full_size(pkg, dev):
    # the DeepSeek-shaped block: 2048 tokens x top-8 over 256 IQ2_XXS experts (gate / up [2048 x 4096], down [4096 x 2048]),
    # r = 16, plus one shared expert in Q8_0 run as a SiLU FFN and added to the routed output.  Two experts carry weights
    # QUANTIZED from N(0, 0.02^2) by the oracle's IQ2_XXS quantizer (the others arbitrary-byte payloads of the same spread):
    # their device decode equals the oracle's bit for bit and their projections match fp32 matmuls; the whole block
    # (routed + shared) matches an fp32 evaluation on sampled tokens.
    import numpy as np

    from oracle import gguf_blocks as gb

    tokens, hidden, inter, e_total, top_k, r, s = 2048, 4096, 2048, 256, 8, 16, 2.0
    gd = torch.Generator(device=dev).manual_seed(43)
    gen = torch.Generator().manual_seed(44)
    G = pkg.gguf.GGUFQuantizedTensor
    payloads = {"gate": pkg.gguf.random_iq2_xxs((e_total, inter, hidden), gd, dev), "up": pkg.gguf.random_iq2_xxs((e_total, inter, hidden), gd, dev),
                "down": pkg.gguf.random_iq2_xxs((e_total, hidden, inter), gd, dev)}
    quantized = (3, 200)
    rng = np.random.default_rng(45)
    oracle_decoded = {}
    for e in quantized:
        for name, (n_out, k_in) in (("gate", (inter, hidden)), ("up", (inter, hidden)), ("down", (hidden, inter))):
            w = (rng.standard_normal((n_out, k_in)) * 0.02).astype(np.float32)
            packed = gb.quantize(w, gb.IQ2_XXS)
            payloads[name][e] = pkg.gguf.quantize_iq2_xxs(torch.from_numpy(w).to(dev))  # the device quantizer the bench uses ...
            assert np.array_equal(payloads[name][e].cpu().numpy(), packed), f"device IQ2_XXS quantizer differs from the oracle's on {name}[{e}]"  # ... is the oracle's, bit for bit
            oracle_decoded[(name, e)] = gb.dequantize_bf16(packed, gb.IQ2_XXS)
    gate, up, down = (G(payloads[n], 16, shape) for n, shape in (("gate", (e_total, inter, hidden)), ("up", (e_total, inter, hidden)),
                                                                  ("down", (e_total, hidden, inter))))
    for (name, e), want in oracle_decoded.items():
        got = pkg.gguf.dequantize_gguf_tensor(payloads[name][e:e + 1], 16, torch.bfloat16)[0]
        assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), gb.to_bf16_bits(want)), f"decode of {name}[{e}]"
    layer = pkg.fast_moe_lora.FastGGUFMoeLora(pkg.fast_moe_lora.GGUFExperts(gate, up, down), r=r, lora_alpha=32)
    with torch.no_grad():
        for name, p in layer.named_parameters():
            std = p.shape[-1] ** -0.5 if "lora_A" in name else 0.01
            p.copy_((torch.randn(p.shape, generator=gen) * std).to(torch.bfloat16))
    # the shared expert: Q8_0 gate / up / down of the same shapes, quantized from N(0, 0.02^2), each with its own LoRA
    shared = {}
    for name, (n_out, k_in) in (("gate", (inter, hidden)), ("up", (inter, hidden)), ("down", (hidden, inter))):
        payload = pkg.gguf.quantize_q8_0((torch.randn(n_out, k_in, generator=gen) * 0.02).to(dev))
        la = (torch.randn(r, k_in, generator=gen) * k_in ** -0.5).to(torch.bfloat16).to(dev).requires_grad_(True)
        lb = (torch.randn(n_out, r, generator=gen) * 0.01).to(torch.bfloat16).to(dev).requires_grad_(True)
        shared[name] = (payload, la, lb, n_out)

    def shared_ffn(h):
        g_, u_ = (pkg.fast_lora.lora_mmq(h, *shared[n][:1], 8, shared[n][3], shared[n][1], shared[n][2], s) for n in ("gate", "up"))
        return pkg.fast_lora.lora_mmq(pkg.fast_moe_lora.swiglu(g_, u_), shared["down"][0], 8, hidden, shared["down"][1], shared["down"][2], s)

    x = torch.randn(tokens, hidden, generator=gen).to(torch.bfloat16).to(dev).requires_grad_(True)
    top = torch.topk(torch.randn(tokens, e_total, generator=gen), top_k, dim=-1)
    idx, weights = top.indices.to(dev), torch.softmax(top.values, dim=-1).to(dev).requires_grad_(True)
    dy = torch.randn(tokens, hidden, generator=gen).to(torch.bfloat16).to(dev)
    out = layer(x, idx, weights) + shared_ffn(x)
    out.backward(dy)
    assert torch.isfinite(out).all() and torch.isfinite(x.grad).all()
    # the two quantized experts' launches against fp32 matmuls on the ORACLE's decode
    ml, mr = pkg.fast_moe_lora, pkg.fast_moe_routing
    plan = mr.prepare_expert_routing(x.detach(), idx, weights.detach(), e_total)
    ids = torch.arange(e_total, dtype=torch.int64, device=dev)
    a, b = layer.lora_A["default"].weight.detach(), layer.lora_B["default"].weight.detach()
    ad, bd = layer.lora_A_down["default"].weight.detach(), layer.lora_B_down["default"].weight.detach()
    sel = plan.selected_hidden_states
    rows = sel.shape[0]

    def leaf(t):
        return t.detach().clone().requires_grad_(True)

    al, bl, adl, bdl = leaf(a), leaf(b), leaf(ad), leaf(bd)
    sel_l = leaf(sel)
    dy1 = torch.randn(rows, inter, generator=gen).to(torch.bfloat16).to(dev)
    dy2 = torch.randn(rows, inter, generator=gen).to(torch.bfloat16).to(dev)
    y1, y2 = ml.grouped_lora_mmq_pair(sel_l, gate, up, ids, plan.expert_end_offsets, 16, inter, al, bl, s)
    torch.autograd.backward((y1, y2), (dy1, dy2))
    act = leaf(ml.swiglu(y1.detach(), y2.detach()))
    yd = ml.grouped_lora_mmq(act, down, ids, plan.expert_end_offsets, 16, hidden, adl, bdl, s)
    dyd = torch.randn(rows, hidden, generator=gen).to(torch.bfloat16).to(dev)
    yd.backward(dyd)
    dact = ml.grouped_mmq_grad_input(dyd, down, ids, plan.expert_end_offsets, 16, inter)
    ends = plan.expert_end_offsets.cpu().tolist()
    f = lambda t: t.detach().float()
    for e in quantized:
        r0, r1 = _expert_rows(ends, e)
        assert r1 > r0
        wg, wu, wd = (torch.from_numpy(oracle_decoded[(n, e)]).to(dev) for n in ("gate", "up", "down"))
        xe, d1, d2 = f(sel[r0:r1]), f(dy1[r0:r1]), f(dy2[r0:r1])
        xa = _bf16(xe @ f(a[e]).T)
        assert_close_bf16(y1[r0:r1], (xe @ wg.T + s * (xa @ f(b[e, :inter]).T)).double(), f"gate of quantized expert {e}")
        assert_close_bf16(y2[r0:r1], (xe @ wu.T + s * (xa @ f(b[e, inter:]).T)).double(), f"up of quantized expert {e}")
        # gate/up input gradient WITH the LoRA term, and the factor gradients of the pair
        dyb = _bf16(d1 @ f(b[e, :inter]) + d2 @ f(b[e, inter:]))
        assert_close_bf16(sel_l.grad[r0:r1], (d1 @ wg + d2 @ wu + s * (dyb @ f(a[e]))).double(), f"gate/up dX of quantized expert {e}")
        assert_close_bf16(al.grad[e], (s * (dyb.T @ xe)).double(), f"gate/up dA of quantized expert {e}")
        assert_close_bf16(bl.grad[e], (s * (torch.cat([d1, d2], dim=1).T @ xa)).double(), f"gate/up dB of quantized expert {e}")
        # down: forward, input gradient with and without the LoRA term, factor gradients
        ae, dd = f(act[r0:r1]), f(dyd[r0:r1])
        xad = _bf16(ae @ f(ad[e]).T)
        dybd = _bf16(dd @ f(bd[e]))
        assert_close_bf16(yd[r0:r1], (ae @ wd.T + s * (xad @ f(bd[e]).T)).double(), f"down of quantized expert {e}")
        assert_close_bf16(act.grad[r0:r1], (dd @ wd + s * (dybd @ f(ad[e]))).double(), f"down dX (with LoRA) of quantized expert {e}")
        assert_close_bf16(dact[r0:r1], (dd @ wd).double(), f"down dX of quantized expert {e}")
        assert_close_bf16(adl.grad[e], (s * (dybd.T @ ae)).double(), f"down dA of quantized expert {e}")
        assert_close_bf16(bdl.grad[e], (s * (dd.T @ xad)).double(), f"down dB of quantized expert {e}")
    # dHidden of the launch that reads the tokens in place, for tokens routed to a quantized expert: every route's dX
    # rounded to bf16 (the quantized experts on the ORACLE's decode), then the token's eight routes added up
    xr = leaf(x)
    z1, z2 = ml._RoutedGroupedLoraProjection.apply(xr, plan.permutation, plan.inverse_permutation, top_k, gate.as_subclass(torch.Tensor),
                                                   up.as_subclass(torch.Tensor), ids, plan.expert_end_offsets, 16, inter, a, b, s)
    assert torch.equal(z1, y1) and torch.equal(z2, y2)
    torch.autograd.backward((z1, z2), (dy1, dy2))
    inverse = plan.inverse_permutation.cpu().reshape(-1, top_k)
    idx_rows = idx.cpu()

    def decoded(name, t, e):
        if (name, e) in oracle_decoded:
            return torch.from_numpy(oracle_decoded[(name, e)]).to(dev)
        return pkg.gguf.dequantize_gguf_tensor(t[e:e + 1], 16, torch.bfloat16)[0].float()

    for q in quantized:
        t = int((idx_rows == q).any(dim=1).nonzero()[0])
        want = torch.zeros(hidden, dtype=torch.float64, device=dev)
        magnitude = torch.zeros(hidden, dtype=torch.float64, device=dev)
        for k in range(top_k):
            row, e = int(inverse[t, k]), int(idx_rows[t, k])
            d1, d2 = dy1[row].float(), dy2[row].float()
            dyb = _bf16(d1 @ f(b[e, :inter]) + d2 @ f(b[e, inter:]))
            term = _bf16(d1 @ decoded("gate", gate, e) + d2 @ decoded("up", up, e) + s * (dyb @ f(a[e]))).double()
            want += term
            magnitude += term.abs()
        err = (xr.grad[t].double() - want).abs()
        assert bool((err <= (top_k + 1) * 2.0 ** -9 * magnitude + 1e-6).all()), f"dHidden of token {t}"
        assert max_rel(xr.grad[t], want) <= 2e-2

    # the whole block on sampled tokens (one of them routed to a quantized expert), every stage rounded to bf16 where the
    # path stores bf16
    def dec(t, e, qt=16):
        return pkg.gguf.dequantize_gguf_tensor(t[e:e + 1], qt, torch.bfloat16)[0].float()

    def ffn(h, wg, wu, wd, la_g, lb_g, la_u, lb_u, la_d, lb_d):
        g_ = _bf16(h @ wg.T + s * (_bf16(h @ la_g.T) @ lb_g.T))
        u_ = _bf16(h @ wu.T + s * (_bf16(h @ la_u.T) @ lb_u.T))
        m = _bf16(torch.nn.functional.silu(g_) * u_)
        return _bf16(m @ wd.T + s * (_bf16(m @ la_d.T) @ lb_d.T))

    idx_cpu = idx.cpu()
    hit = int((idx_cpu == quantized[0]).any(dim=1).nonzero()[0])
    sw = {n: pkg.gguf.dequantize_gguf_tensor(shared[n][0], 8, torch.bfloat16).float() for n in shared}
    for t in (0, hit, tokens - 1):
        h = x[t].detach().float()
        routed = torch.zeros(hidden, device=dev)
        for k in range(top_k):
            e = int(idx_cpu[t, k])
            y = ffn(h, dec(gate, e), dec(up, e), dec(down, e), a[e].float(), b[e, :inter].float(), a[e].float(), b[e, inter:].float(),
                    ad[e].float(), bd[e].float())
            routed += weights[t, k].detach().float() * y
        sh = ffn(h, sw["gate"], sw["up"], sw["down"], *(shared[n][i].detach().float() for n in ("gate", "up", "down") for i in (1, 2)))
        assert_close_bf16(out[t], (_bf16(routed) + sh).double(), f"block output of token {t}", ulps=4.0)
