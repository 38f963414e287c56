"""Seeded sweep over shapes of the grouped LoRA projection (block format, expert count, ragged and empty groups, output
widths that are not whole tiles, ranks, pair or single, every kernel shape) against fp32 matmuls on the decoded weights,
whose decoders are checked bit for bit elsewhere.  Tolerance of the path: max rel err <= 2e-2 plus the per-element bound of
assert_close_bf16."""

import random

import numpy as np
import pytest
import torch

from helpers import assert_close_bf16, max_rel
from oracle import gguf_blocks as gb

pytestmark = pytest.mark.gpu


def _bf16(t):
    return t.to(torch.bfloat16).float()


def _payload(pkg, dev, qt, e, n, k, g):
    if qt == gb.IQ2_XXS:
        return pkg.gguf.random_iq2_xxs((e, n, k), g, dev)
    w = torch.randn(e, n, k, generator=g, device=dev) * 0.02
    if qt in (gb.Q8_0, gb.Q4_K, gb.Q6_K):
        return pkg.gguf.quantize(w, qt)
    return torch.from_numpy(gb.quantize(w.cpu().numpy().reshape(e * n, k), qt)).reshape(e, n, -1).to(dev)


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_grouped_projection_over_random_shapes(pkg, dev, seed, force_grouped_shape):
    ml = pkg.fast_moe_lora
    rnd = random.Random(seed)
    for case in range(40):
        qt = rnd.choice([gb.Q8_0, gb.Q2_K, gb.Q3_K, gb.Q4_K, gb.Q4_K, gb.Q4_K, gb.Q5_K, gb.Q6_K, gb.IQ2_XXS])
        e = rnd.choice([1, 3, 8, 17])
        k = rnd.choice([256, 512, 768, 1024])
        n = rnd.choice([8, 64, 72, 128, 192, 256, 320, 520])
        r = rnd.choice([0, 0, 4, 8, 16, 16, 24, 64])
        pair = rnd.random() < 0.5
        shape = rnd.choice(["", "", "0", "1", "1", "3"])
        sizes = [rnd.choice([0, 1, 5, 31, 64, 100, 128, 129, 200, 260, 400]) for _ in range(e)]
        if sum(sizes) == 0:
            sizes[0] = 7
        what = f"case {case}: qt={qt} e={e} k={k} n={n} r={r} pair={pair} shape={shape!r} sizes={sizes}"
        print(what, flush=True)
        force_grouped_shape(shape)
        g = torch.Generator(device=dev).manual_seed(1000 * seed + case)
        rows, nseg = sum(sizes), 2 if pair else 1
        p1 = _payload(pkg, dev, qt, e, n, k, g)
        p2 = _payload(pkg, dev, qt, e, n, k, g) if pair else None
        x = torch.randn(rows, k, generator=g, device=dev).to(torch.bfloat16).requires_grad_(True)
        a = (torch.randn(e, r, k, generator=g, device=dev) * k ** -0.5).to(torch.bfloat16).requires_grad_(True) if r else None
        b = (torch.randn(e, nseg * n, r, generator=g, device=dev) * 0.02).to(torch.bfloat16).requires_grad_(True) if r else None
        dy = torch.randn(rows, nseg * n, generator=g, device=dev).to(torch.bfloat16)
        ids = torch.arange(e, dtype=torch.int64, device=dev)
        ends = torch.tensor(np.cumsum(sizes), dtype=torch.int32, device=dev)
        if pair:
            y = torch.cat(ml.grouped_lora_mmq_pair(x, p1, p2, ids, ends, qt, n, a, b, 2.0) if r else ml.grouped_mmq_pair(x, p1, p2, ids, ends, qt, n), dim=1)
        else:
            y = ml.grouped_lora_mmq(x, p1, ids, ends, qt, n, a, b, 2.0) if r else ml.grouped_mmq(x, p1, ids, ends, qt, n)
        y.backward(dy)
        w = pkg.gguf.dequantize_gguf_tensor(p1, qt, torch.bfloat16).float()
        if pair:
            w = torch.cat([w, pkg.gguf.dequantize_gguf_tensor(p2, qt, torch.bfloat16).float()], dim=1)
        want_y, want_dx = torch.zeros(rows, nseg * n, device=dev), torch.zeros(rows, k, device=dev)
        want_da = torch.zeros(a.shape, device=dev) if r else None
        want_db = torch.zeros(b.shape, device=dev) if r else None
        r0 = 0
        for ei, sz in enumerate(sizes):
            r1 = r0 + sz
            if sz:
                xe, de = x.detach()[r0:r1].float(), dy[r0:r1].float()
                want_y[r0:r1], want_dx[r0:r1] = xe @ w[ei].T, de @ w[ei]
                if r:
                    af, bfm = a.detach()[ei].float(), b.detach()[ei].float()
                    xa, dyb = _bf16(xe @ af.T), _bf16(de @ bfm)
                    want_y[r0:r1] += 2.0 * (xa @ bfm.T)
                    want_dx[r0:r1] += 2.0 * (dyb @ af)
                    want_da[ei], want_db[ei] = 2.0 * (dyb.T @ xe), 2.0 * (de.T @ xa)
            r0 = r1
        assert_close_bf16(y, want_y.double(), what + ": Y")
        assert_close_bf16(x.grad, want_dx.double(), what + ": dX")
        if r:
            assert_close_bf16(a.grad, want_da.double(), what + ": dA")
            assert_close_bf16(b.grad, want_db.double(), what + ": dB")


def _dense_payload(pkg, dev, qt, n, k, g):
    return _payload(pkg, dev, qt, 1, n, k, g)[0]


def test_dense_lora_linear_over_random_shapes(pkg, dev):
    # row counts on both sides of the sizes at which the factor gradients split their rows over workgroups
    rnd = random.Random(21)
    for case in range(36):
        qt = rnd.choice([gb.Q8_0, gb.Q2_K, gb.Q3_K, gb.Q4_K, gb.Q4_K, gb.Q5_K, gb.Q6_K, gb.IQ2_XXS])
        m = rnd.choice([1, 7, 64, 255, 256, 257, 700, 1024, 3000, 4096, 5000])
        k = rnd.choice([256, 512, 1024, 2048])
        n = rnd.choice([8, 72, 128, 520, 1024, 4096])
        r = rnd.choice([4, 8, 16, 16, 24, 64])
        what = f"case {case}: qt={qt} m={m} k={k} n={n} r={r}"
        print(what, flush=True)
        g = torch.Generator(device=dev).manual_seed(77 + case)
        p = _dense_payload(pkg, dev, qt, n, k, g)
        x = torch.randn(m, k, generator=g, device=dev).to(torch.bfloat16).requires_grad_(True)
        a = (torch.randn(r, k, generator=g, device=dev) * k ** -0.5).to(torch.bfloat16).requires_grad_(True)
        b = (torch.randn(n, r, generator=g, device=dev) * 0.02).to(torch.bfloat16).requires_grad_(True)
        dy = torch.randn(m, n, generator=g, device=dev).to(torch.bfloat16)
        y = pkg.fast_lora.lora_mmq(x, p, qt, n, a, b, 2.0)
        y.backward(dy)
        w = pkg.gguf.dequantize_gguf_tensor(p, qt, torch.bfloat16).float()
        xf, af, bfm, df = x.detach().float(), a.detach().float(), b.detach().float(), dy.float()
        xa, dyb = _bf16(xf @ af.T), _bf16(df @ bfm)
        assert_close_bf16(y, (xf @ w.T + 2 * (xa @ bfm.T)).double(), what + ": Y")
        assert_close_bf16(x.grad, (df @ w + 2 * (dyb @ af)).double(), what + ": dX")
        assert_close_bf16(a.grad, (2 * (dyb.T @ xf)).double(), what + ": dA")
        assert_close_bf16(b.grad, (2 * (df.T @ xa)).double(), what + ": dB")


def test_lm_head_loss_over_random_shapes(pkg, dev):
    # vocabularies around one 8192-column block, row counts around one chunk and around one 4096-row gradient block
    from helpers import max_rel

    rnd = random.Random(31)
    for case in range(14):
        qt = rnd.choice([gb.Q8_0, gb.Q4_K, gb.Q6_K, gb.Q6_K])
        rows = rnd.choice([1, 33, 256, 257, 1000, 4097, 6000])
        hidden = rnd.choice([256, 512, 2048])
        vocab = rnd.choice([37, 1000, 8192, 8193, 20000, 50000])
        chunk = rnd.choice([32, 256, 1024, 5000])
        red = rnd.choice(["mean", "sum"])
        what = f"case {case}: qt={qt} rows={rows} hidden={hidden} vocab={vocab} chunk={chunk} {red}"
        print(what, flush=True)
        g = torch.Generator(device=dev).manual_seed(177 + case)
        p = _dense_payload(pkg, dev, qt, vocab, hidden, g)
        hid = torch.randn(rows, hidden, generator=g, device=dev).to(torch.bfloat16)
        labels = torch.randint(0, vocab, (rows,), generator=g, device=dev)
        labels[torch.rand(rows, generator=g, device=dev) < 0.1] = -100
        h = hid.clone().requires_grad_(True)
        loss = pkg.gguf_liger_loss.packed_linear_cross_entropy(h, p, labels, qt, vocab, chunk, -100, red)
        loss.backward()
        w = pkg.gguf.dequantize_gguf_tensor(p, qt, torch.bfloat16).float()
        valid = labels != -100
        n_valid = max(int(valid.sum()), 1)
        scale = 1.0 / n_valid if red == "mean" else 1.0
        logits = _bf16(hid.float() @ w.T)
        lse = torch.logsumexp(logits, 1)
        tgt = logits.gather(1, labels.clamp(min=0)[:, None])[:, 0]
        want = float(((lse - tgt) * valid).double().sum() * scale)
        d = torch.softmax(logits, 1)
        d[torch.arange(rows, device=dev), labels.clamp(min=0)] -= 1.0
        want_dh = _bf16(d * (valid[:, None] * scale)) @ w
        assert abs(float(loss) - want) * (1.0 if red == "mean" else 1.0 / n_valid) <= 1e-3, (what, float(loss), want)
        if bool(valid.any()):
            assert max_rel(h.grad, want_dh) <= 2e-2, what
        assert bool((h.grad[~valid] == 0).all()), what


def test_expert_layer_equals_the_explicit_composition_bit_for_bit(pkg, dev, monkeypatch):
    # The module (token rows read in place by the gate/up launch) against routing plan -> gathered copy -> grouped pair ->
    # SwiGLU -> grouped down -> combine, over random layer geometries: outputs and every gradient are the same bits.
    ml, mr = pkg.fast_moe_lora, pkg.fast_moe_routing
    G = pkg.gguf.GGUFQuantizedTensor
    rnd = random.Random(9)
    for case in range(30):
        qt = rnd.choice([gb.Q8_0, gb.Q2_K, gb.Q4_K, gb.Q4_K, gb.Q4_K, gb.Q6_K, gb.IQ2_XXS])
        qd = rnd.choice([qt, gb.Q4_K, gb.Q2_K])
        e = rnd.choice([4, 8, 32, 64])
        top_k = min(rnd.choice([1, 2, 6, 8]), e)
        tokens, hidden, inter = rnd.choice([1, 5, 64, 300, 1000]), rnd.choice([256, 512, 1024]), rnd.choice([256, 512])
        r, limit, wdt = rnd.choice([0, 4, 16]), rnd.choice([None, None, 1.5]), rnd.choice([torch.float32, torch.bfloat16])
        what = f"case {case}: qt={qt}/{qd} e={e} top_k={top_k} tokens={tokens} hidden={hidden} inter={inter} r={r} limit={limit} {wdt}"
        print(what, flush=True)
        g = torch.Generator(device=dev).manual_seed(500 + case)
        gate = G(_payload(pkg, dev, qt, e, inter, hidden, g), qt, (e, inter, hidden))
        up = G(_payload(pkg, dev, qt, e, inter, hidden, g), qt, (e, inter, hidden))
        down = G(_payload(pkg, dev, qd, e, hidden, inter, g), qd, (e, hidden, inter))
        experts = ml.GGUFExperts(gate, up, down, swiglu_limit=limit)
        layer = ml.FastGGUFMoeLora(experts, r=r, lora_alpha=2 * r) if r else None
        params = list(layer.parameters()) if layer is not None else []
        with torch.no_grad():
            for name, p in (layer.named_parameters() if layer is not None else []):
                p.copy_((torch.randn(p.shape, generator=g, device=dev) * (p.shape[-1] ** -0.5 if "lora_A" in name else 0.02)).to(torch.bfloat16))
        x0 = torch.randn(tokens, hidden, generator=g, device=dev).to(torch.bfloat16)
        scores = torch.randn(tokens, e, generator=g, device=dev)
        scores[:, 0] += 1.0
        top = torch.topk(scores, top_k, dim=-1)
        idx, w0 = top.indices, torch.softmax(top.values, -1).to(wdt)
        dy = torch.randn(tokens, hidden, generator=g, device=dev).to(torch.bfloat16)

        def run(through_module):
            x, w = x0.clone().requires_grad_(True), w0.clone().requires_grad_(True)
            for p in params:
                p.grad = None
            if through_module:
                out = layer(x, idx, w) if layer is not None else experts(x, idx, w)
            else:
                lw = layer._active_lora_weights() if layer is not None else None
                s = lw.scaling if lw else 0.0
                plan = mr.prepare_expert_routing(x, idx, w, e)
                ids = torch.arange(e, dtype=torch.int64, device=dev)
                ga, u = ml._GroupedLoraProjection.apply(plan.selected_hidden_states, gate.as_subclass(torch.Tensor), up.as_subclass(torch.Tensor), ids,
                                                        plan.expert_end_offsets, qt, inter, lw.gate_up_a if lw else None, lw.gate_up_b if lw else None, s)
                o = ml._GroupedLoraProjection.apply(ml.swiglu(ga, u, limit), down.as_subclass(torch.Tensor), None, ids, plan.expert_end_offsets, qd, hidden,
                                                    lw.down_a if lw else None, lw.down_b if lw else None, s)
                out = mr.finalize_expert_routing(o, x, plan, None).reshape(x.shape)
            out.backward(dy)
            return [out.detach(), x.grad, w.grad] + [p.grad.clone() for p in params]

        explicit = run(False)
        monkeypatch.setattr(ml, "FUSE_GATED_DOWN_COMBINE", False)
        for i, (got, want) in enumerate(zip(run(True), explicit)):
            assert torch.equal(got, want), (what, i)
        # the module's default: activation + down projection + combine as one node whose backward applies the routing weight
        # after the grad-input matmul.  Same output bits; gradients equal up to where the two orders round
        monkeypatch.setattr(ml, "FUSE_GATED_DOWN_COMBINE", True)
        fused = run(True)
        assert torch.equal(fused[0], explicit[0]), (what, "fused output")
        for i, (got, want) in enumerate(zip(fused[1:], explicit[1:])):
            assert got.dtype == want.dtype and torch.isfinite(got.float()).all(), (what, i)
            err, bound = float((got.double() - want.double()).abs().max()), 2e-2 * float(want.double().abs().max())
            if i == 1:
                # a routing weight's gradient is one dot product of two hidden-sized vectors, which may cancel: the two
                # orders' bf16 roundings of those vectors move it by about 2^-9 of |dy| |expert output| / sqrt(hidden)
                bound += 2.0 ** -10 * float(dy.float().norm(dim=1).max() * explicit[0].float().norm(dim=1).max() / w0.float().min().clamp(min=1e-3))
            assert err <= bound, (what, "fused gradient", i, err, bound)
