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
