"""Grouped expert projections and the full expert layer against the per-expert oracle loop
(relations of test_fast_moe_lora.py:133-279, 282-348, 406-511 and test_deepseek_v4_moe_lora.py:67-118)."""

import numpy as np
import pytest
import torch

from helpers import max_rel, ALL_TYPES, TYPE_NAMES, assert_close_bf16, bf16_randn, make_payload
from oracle import gguf_blocks as gb
from oracle import lora_matmul as ref
from oracle import routing as rref

pytestmark = pytest.mark.gpu


def _expert_payload(seed, qt, experts, n, k, kind="quantized"):
    return np.stack([make_payload(seed + e, qt, n, k, kind) for e in range(experts)])


def _to(dev, *ts):
    return [t.to(dev) for t in ts]


@pytest.mark.parametrize("qt", ALL_TYPES, ids=[TYPE_NAMES[q] for q in ALL_TYPES])
def test_grouped_pair_and_single_projection_jacobian(pkg, dev, qt):
    # experts [0, 2, 5], cumulative end offsets [2, 5, 6] (test_fast_moe_lora.py:136-137)
    ml = pkg.fast_moe_lora
    experts = torch.tensor([0, 2, 5], dtype=torch.int64)
    offsets = torch.tensor([2, 5, 6], dtype=torch.int32)
    gen = torch.Generator().manual_seed(2468)
    k, n = 2048, 64
    pg, pu = _expert_payload(10, qt, 8, n, k), _expert_payload(50, qt, 8, n, k)
    wg, wu = ref.weights_bf16(pg, qt), ref.weights_bf16(pu, qt)
    hidden = bf16_randn(gen, 6, k)
    g1, g2 = bf16_randn(gen, 6, n), bf16_randn(gen, 6, n)
    want_g = ref.grouped_lora_linear(hidden, wg, experts, offsets, dy=g1)
    want_u = ref.grouped_lora_linear(hidden, wu, experts, offsets, dy=g2)
    h = hidden.to(dev).requires_grad_(True)
    e_d, o_d = _to(dev, experts, offsets)
    pg_d, pu_d = torch.from_numpy(pg).to(dev), torch.from_numpy(pu).to(dev)
    gate, up = ml.grouped_mmq_pair(h, pg_d, pu_d, e_d, o_d, qt, n)
    torch.autograd.backward((gate, up), _to(dev, g1, g2))
    assert_close_bf16(gate, want_g["y"], "gate")
    assert_close_bf16(up, want_u["y"], "up")
    # both cotangents in one accumulator, rounded once (test_fast_moe_lora.py:199-203: atol 1e-4 there)
    assert_close_bf16(h.grad, want_g["dx"] + want_u["dx"], "pair dX")
    # pair == two single projections, bit for bit (test_fast_moe_lora.py:207-236)
    assert torch.equal(gate, ml.grouped_mmq(h.detach(), pg_d, e_d, o_d, qt, n))
    assert torch.equal(up, ml.grouped_mmq(h.detach(), pu_d, e_d, o_d, qt, n))
    # single projection backward (down-proj shape of the reference test: K = 512)
    pd = _expert_payload(90, qt, 8, 64, 512)
    wd = ref.weights_bf16(pd, qt)
    inter = bf16_randn(gen, 6, 512)
    gd = bf16_randn(gen, 6, 64)
    want_d = ref.grouped_lora_linear(inter, wd, experts, offsets, dy=gd)
    it = inter.to(dev).requires_grad_(True)
    out = ml.grouped_mmq(it, torch.from_numpy(pd).to(dev), e_d, o_d, qt, 64)
    out.backward(gd.to(dev))
    assert_close_bf16(out, want_d["y"], "down")
    assert_close_bf16(it.grad, want_d["dx"], "down dX")
    dx_op = ml.grouped_mmq_grad_input(gd.to(dev), torch.from_numpy(pd).to(dev), e_d, o_d, qt, 512)
    assert torch.equal(dx_op, it.grad)


def test_q4k_grouped_grad_input_decoding_waves(pkg, dev):
    # Q4_K, no LoRA term, contraction length 256 (pair: 2 x 256): forward and grad-input both run in the kernels
    # whose MFMA waves decode the weights themselves; ragged groups up to more than one 192-row tile
    ml = pkg.fast_moe_lora
    qt, k, n = gb.Q4_K, 512, 256
    sizes = [5, 0, 200, 33, 0, 129, 64, 1]
    experts = torch.arange(8, dtype=torch.int64)
    offsets = torch.tensor(np.cumsum(sizes), dtype=torch.int32)
    rows = sum(sizes)
    gen = torch.Generator().manual_seed(13579)
    pg, pu = _expert_payload(610, qt, 8, n, k), _expert_payload(650, qt, 8, n, k)
    wg, wu = ref.weights_bf16(pg, qt), ref.weights_bf16(pu, qt)
    hidden = bf16_randn(gen, rows, k)
    g1, g2 = bf16_randn(gen, rows, n), bf16_randn(gen, rows, n)
    want_g = ref.grouped_lora_linear(hidden, wg, experts, offsets, dy=g1)
    want_u = ref.grouped_lora_linear(hidden, wu, experts, offsets, dy=g2)
    h = hidden.to(dev).requires_grad_(True)
    e_d, o_d = _to(dev, experts, offsets)
    pg_d, pu_d = torch.from_numpy(pg).to(dev), torch.from_numpy(pu).to(dev)
    gate, up = ml.grouped_mmq_pair(h, pg_d, pu_d, e_d, o_d, qt, n)
    torch.autograd.backward((gate, up), _to(dev, g1, g2))
    assert_close_bf16(gate, want_g["y"], "gate")
    assert_close_bf16(up, want_u["y"], "up")
    assert_close_bf16(h.grad, want_g["dx"] + want_u["dx"], "pair dX")
    dx_single = ml.grouped_mmq_grad_input(g1.to(dev), pg_d, e_d, o_d, qt, k)
    assert_close_bf16(dx_single, want_g["dx"], "single dX")


def test_constant_byte_iq2_xxs_experts(pkg, dev):
    # test_deepseek_v4_moe_lora.py:55-118: payload of all bytes 32, experts [0,1], offsets [3,7]
    ml = pkg.fast_moe_lora
    payload = np.full((2, 256, 66), 32, dtype=np.uint8)
    w = ref.weights_bf16(payload, gb.IQ2_XXS)
    experts = torch.tensor([0, 1], dtype=torch.int64)
    offsets = torch.tensor([3, 7], dtype=torch.int32)
    gen = torch.Generator().manual_seed(5)
    hidden, gout = bf16_randn(gen, 7, 256), bf16_randn(gen, 7, 256)
    want = ref.grouped_lora_linear(hidden, w, experts, offsets, dy=gout)
    h = hidden.to(dev).requires_grad_(True)
    out = ml.grouped_mmq(h, torch.from_numpy(payload).to(dev), experts.to(dev), offsets.to(dev), gb.IQ2_XXS, 256)
    out.backward(gout.to(dev))
    torch.testing.assert_close(out.double().cpu(), want["y"], rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(h.grad.double().cpu(), want["dx"], rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("qt,r,shape,n", [(gb.Q4_K, 16, "", 192), (gb.Q4_K, 16, "", 256), (gb.Q4_K, 16, "3", 256), (gb.Q4_K, 16, "1", 256), (gb.Q4_K, 16, "0", 192),
                                          (gb.Q4_K, 16, "3", 128),  # the pair's grad-input: four steps, the fewest the decoding-wave kernel takes; the single projection's two: tiles
                                          (gb.Q4_K, 32, "3", 256),  # a rank beyond the 16 columns of the LoRA rows the kernels keep in LDS
                                          (gb.Q8_0, 4, "", 192), (gb.Q6_K, 8, "", 192), (gb.IQ2_XXS, 16, "", 192)])
def test_grouped_lora_projection_all_gradients(pkg, dev, qt, r, shape, n, force_grouped_shape):
    # ragged groups including empty experts, a group larger than one 128-row tile, and inactive planes.
    # Q4_K runs in the kernels whose MFMA waves decode the weights themselves (the grad-input one takes an even number of
    # whole 64-row contraction steps: n = 192 as a pair, n = 256); shape "1": the wide / tall tile mix, "0": tall tiles
    force_grouped_shape(shape)
    ml = pkg.fast_moe_lora
    e_total, k = 8, 512
    sizes = [0, 150, 3, 0, 129, 1, 64, 0]
    rows = sum(sizes)
    all_ids = torch.arange(e_total, dtype=torch.int64)
    ends = torch.tensor(np.cumsum(sizes), dtype=torch.int32)
    gen = torch.Generator().manual_seed(8642 + r)
    p1, p2 = _expert_payload(300, qt, e_total, n, k), _expert_payload(400, qt, e_total, n, k)
    w1, w2 = ref.weights_bf16(p1, qt), ref.weights_bf16(p2, qt)
    x = bf16_randn(gen, rows, k)
    a = bf16_randn(gen, e_total, r, k, std=k ** -0.5)
    b = bf16_randn(gen, e_total, 2 * n, r, std=0.02)
    dy = bf16_randn(gen, rows, 2 * n)
    s = 2.0
    want = ref.grouped_lora_linear(x, torch.cat([w1, w2], dim=1), all_ids, ends, a, b, s, dy)
    xd, ad, bd = (t.to(dev).requires_grad_(True) for t in (x, a, b))
    y1, y2 = ml.grouped_lora_mmq_pair(xd, torch.from_numpy(p1).to(dev), torch.from_numpy(p2).to(dev), all_ids.to(dev), ends.to(dev), qt, n, ad, bd, s)
    torch.autograd.backward((y1, y2), (dy[:, :n].contiguous().to(dev), dy[:, n:].contiguous().to(dev)))
    assert_close_bf16(torch.cat([y1, y2], dim=1), want["y"], "pair Y")
    assert_close_bf16(xd.grad, want["dx"], "pair dX")
    assert_close_bf16(ad.grad, want["da"], "dA")
    assert_close_bf16(bd.grad, want["db"], "dB")
    inactive = torch.tensor([sz == 0 for sz in sizes])
    assert torch.count_nonzero(ad.grad[inactive.to(dev)]) == 0 and torch.count_nonzero(bd.grad[inactive.to(dev)]) == 0
    # compact active-expert form gives the same bits as the full list with empty groups
    active = torch.tensor([e for e, sz in enumerate(sizes) if sz], dtype=torch.int64)
    active_ends = torch.tensor(np.cumsum([sz for sz in sizes if sz]), dtype=torch.int32)
    z1, z2 = ml.grouped_lora_mmq_pair(xd.detach(), torch.from_numpy(p1).to(dev), torch.from_numpy(p2).to(dev), active.to(dev), active_ends.to(dev), qt, n, ad.detach(), bd.detach(), s)
    assert torch.equal(z1, y1) and torch.equal(z2, y2)
    # single (down-like) projection with LoRA
    want1 = ref.grouped_lora_linear(x, w1, all_ids, ends, a, b[:, :n].contiguous(), s, dy[:, :n].contiguous())
    xd2, ad2, bd2 = (t.to(dev).requires_grad_(True) for t in (x, a, b[:, :n].contiguous()))
    y = ml.grouped_lora_mmq(xd2, torch.from_numpy(p1).to(dev), all_ids.to(dev), ends.to(dev), qt, n, ad2, bd2, s)
    y.backward(dy[:, :n].contiguous().to(dev))
    assert_close_bf16(y, want1["y"], "single Y")
    assert_close_bf16(xd2.grad, want1["dx"], "single dX")
    assert_close_bf16(ad2.grad, want1["da"], "single dA")
    assert_close_bf16(bd2.grad, want1["db"], "single dB")


@pytest.mark.parametrize("sizes,n,k,r,pair", [
    ([1, 32, 33, 64, 65, 96, 97, 128, 129, 0, 7], 256, 512, 16, True),   # every count of live 32-row blocks; 129 rows: a tall tile beside them
    ([64, 64, 50, 3], 72, 256, 0, False),                                    # one block of the contraction; columns end inside a wave's 32
    ([40, 100, 128], 520, 768, 32, False),                                   # three column tiles, the last one 8 wide; rank 32
    ([5, 90], 8, 1024, 4, True),                                             # fewer columns than one wave owns; rank padded to 16
    ([128] * 3 + [1] * 5, 512, 256, 64, False),                              # rank 64
])
@pytest.mark.parametrize("shape", ["", "1"])
def test_iq2xxs_forward_of_small_groups(pkg, dev, sizes, n, k, r, pair, shape, force_grouped_shape):
    # IQ2_XXS groups of at most 128 rows run the forward kernel whose MFMA waves decode the packed bytes themselves
    # (mmq_small_iq2xxs_kernel); larger groups of the same call stay on the tile kernel.  Against the oracle, with and
    # without LoRA, as a pair and as a single projection.  Shape "1": the same calls on wide / tall tiles only.
    force_grouped_shape(shape)
    ml = pkg.fast_moe_lora
    qt = gb.IQ2_XXS
    e_total, rows = len(sizes), sum(sizes)
    ids = torch.arange(e_total, dtype=torch.int64)
    ends = torch.tensor(np.cumsum(sizes), dtype=torch.int32)
    gen = torch.Generator().manual_seed(97 + n + k + r)
    segs = 2 if pair else 1
    payloads = [_expert_payload(700 + 100 * j, qt, e_total, n, k) for j in range(segs)]
    w = torch.cat([ref.weights_bf16(pl, qt) for pl in payloads], dim=1)
    x = bf16_randn(gen, rows, k)
    a = bf16_randn(gen, e_total, r, k, std=k ** -0.5) if r else None
    b = bf16_randn(gen, e_total, segs * n, r, std=0.02) if r else None
    want = ref.grouped_lora_linear(x, w, ids, ends, a, b, 2.0) if r else ref.grouped_lora_linear(x, w, ids, ends)
    pd = [torch.from_numpy(pl).to(dev) for pl in payloads]
    if pair and r:
        ys = ml.grouped_lora_mmq_pair(x.to(dev), pd[0], pd[1], ids.to(dev), ends.to(dev), qt, n, a.to(dev), b.to(dev), 2.0)
    elif pair:
        ys = ml.grouped_mmq_pair(x.to(dev), pd[0], pd[1], ids.to(dev), ends.to(dev), qt, n)
    elif r:
        ys = (ml.grouped_lora_mmq(x.to(dev), pd[0], ids.to(dev), ends.to(dev), qt, n, a.to(dev), b.to(dev), 2.0),)
    else:
        ys = (ml.grouped_mmq(x.to(dev), pd[0], ids.to(dev), ends.to(dev), qt, n),)
    assert_close_bf16(torch.cat(list(ys), dim=1), want["y"], "Y")


@pytest.mark.parametrize("top_k,rank,pair,qt,shape", [(8, 16, True, gb.Q4_K, ""), (3, 4, True, gb.Q4_K, ""), (1, 16, False, gb.Q4_K, ""),
                                                      (8, 0, True, gb.Q4_K, ""), (8, 16, True, gb.Q4_K, "1"), (3, 16, True, gb.Q4_K, "0"),
                                                      (2, 8, True, gb.Q4_K, "0"), (8, 16, True, gb.Q6_K, ""), (3, 4, False, gb.IQ2_XXS, "")])
def test_routed_projection_reads_tokens_in_place(pkg, dev, top_k, rank, pair, qt, shape, force_grouped_shape):
    # The gate/up launch that reads the token matrix through the routing permutation against the same launch on the
    # gathered copy: outputs, token gradients (summed over each token's routes) and factor gradients are the same bits.
    # Skewed routing: some experts receive no route, one receives more than a 192-row tile.  Every kernel shape of the
    # forward launch takes the index (the decoding-wave kernel by default for Q4_K, the tile kernels otherwise).
    force_grouped_shape(shape)
    ml, mr = pkg.fast_moe_lora, pkg.fast_moe_routing
    tokens, k, n, experts = 211, 512, 256, 12
    gen = torch.Generator().manual_seed(977 + top_k)
    x = bf16_randn(gen, tokens, k)
    scores = torch.rand(tokens, experts, generator=gen)
    scores[:, 5] = -1.0
    scores[:, 9] = -1.0
    scores[:, 2] += 0.9 if top_k > 1 else 0.4
    idx = scores.topk(top_k, dim=1).indices
    w = torch.full((tokens, top_k), 1.0 / top_k)
    p1, p2 = _expert_payload(31, qt, experts, n, k), _expert_payload(32, qt, experts, n, k)
    p1d, p2d = torch.from_numpy(p1).to(dev), (torch.from_numpy(p2).to(dev) if pair else None)
    nseg = 2 if pair else 1
    a = bf16_randn(gen, experts, rank, k, std=k ** -0.5) if rank else None
    b = bf16_randn(gen, experts, nseg * n, rank, std=0.02) if rank else None
    dy = [bf16_randn(gen, tokens * top_k, n).to(dev) for _ in range(nseg)]
    routes = tokens * top_k
    assert ml.routed_projection_reads_tokens_in_place(qt, routes, experts, tokens, k)
    assert not ml.routed_projection_reads_tokens_in_place(qt, routes, experts, 1 << 21, 1024)   # a 4 GiB token matrix
    assert not ml.routed_projection_reads_tokens_in_place(3, routes, experts, tokens, k)        # no kernels for this type

    def run(in_place):
        xd = x.to(dev).requires_grad_(True)
        ad, bd = (t.to(dev).requires_grad_(True) if t is not None else None for t in (a, b))
        plan = mr.prepare_expert_routing(xd, idx.to(dev), w.to(dev), experts, gather=not in_place)
        ids = torch.arange(experts, dtype=torch.int64, device=dev)
        if in_place:
            assert plan.selected_hidden_states is None
            out = ml._RoutedGroupedLoraProjection.apply(xd, plan.permutation, plan.inverse_permutation, top_k, p1d, p2d, ids,
                                                        plan.expert_end_offsets, qt, n, ad, bd, 2.0)
        else:
            out = ml._GroupedLoraProjection.apply(plan.selected_hidden_states, p1d, p2d, ids, plan.expert_end_offsets, qt, n, ad, bd, 2.0)
        out = out if pair else (out,)
        torch.autograd.backward(out, tuple(dy))
        return [*out, xd.grad] + ([ad.grad, bd.grad] if rank else [])

    got, want = run(True), run(False)
    for g, t, what in zip(got, want, ["y1", "y2", "d hidden", "dA", "dB"] if pair else ["y", "d hidden", "dA", "dB"]):
        assert torch.equal(g, t), what
    # and the result is the oracle's: the gathered rows through the grouped oracle
    _, perm, _ = rref.plan(idx)
    sel = rref.gather_forward(x, perm, top_k)
    ends = torch.cumsum(rref.expert_counts(idx, experts).to(torch.int64), 0).to(torch.int32)
    wcat = torch.cat([ref.weights_bf16(p1, qt)] + ([ref.weights_bf16(p2, qt)] if pair else []), dim=1)
    o = ref.grouped_lora_linear(sel, wcat, torch.arange(experts), ends, a, b, 2.0, torch.cat([d.cpu() for d in dy], dim=1))
    assert_close_bf16(torch.cat(got[:nseg], dim=1), o["y"], "in-place Y against the oracle")
    if rank:
        assert_close_bf16(got[-2], o["da"], "in-place dA against the oracle")


@pytest.mark.parametrize("shape", ["", "0", "1", "3"])
def test_q4k_grouped_identity_reproduces_decoded_rows_exactly(pkg, dev, shape, force_grouped_shape):
    # One-hot rows through every Q4_K kernel shape of the grouped launches (the decoding-wave kernels by default): each
    # output is a single product 1 * w, so the in-register decoders are compared with the oracle element by element, for
    # arbitrary block bytes (every 6-bit scale split), in forward (pair) and in grad-input.
    force_grouped_shape(shape)
    ml = pkg.fast_moe_lora
    e, n, k = 3, 256, 512
    p1, p2 = _expert_payload(71, gb.Q4_K, e, n, k, "random"), _expert_payload(72, gb.Q4_K, e, n, k, "random")
    w1 = torch.from_numpy(gb.dequantize_bf16(p1.reshape(e * n, -1), gb.Q4_K)).reshape(e, n, k)
    w2 = torch.from_numpy(gb.dequantize_bf16(p2.reshape(e * n, -1), gb.Q4_K)).reshape(e, n, k)
    ids = torch.arange(e, dtype=torch.int64, device=dev)
    # forward: expert g gets the k one-hot rows; groups of 512 rows (several row tiles each)
    x = torch.eye(k, dtype=torch.bfloat16, device=dev).repeat(e, 1)
    ends = torch.tensor([k, 2 * k, 3 * k], dtype=torch.int32, device=dev)
    y1, y2 = ml.grouped_mmq_pair(x, torch.from_numpy(p1).to(dev), torch.from_numpy(p2).to(dev), ids, ends, gb.Q4_K, n)
    for g in range(e):
        assert torch.equal(y1[g * k:(g + 1) * k].float().cpu(), w1[g].T.contiguous()), (g, "first of the pair")
        assert torch.equal(y2[g * k:(g + 1) * k].float().cpu(), w2[g].T.contiguous()), (g, "second of the pair")
    # grad-input: expert g gets the n one-hot cotangent rows
    dy = torch.eye(n, dtype=torch.bfloat16, device=dev).repeat(e, 1)
    ends_n = torch.tensor([n, 2 * n, 3 * n], dtype=torch.int32, device=dev)
    dx = ml.grouped_mmq_grad_input(dy, torch.from_numpy(p1).to(dev), ids, ends_n, gb.Q4_K, k)
    for g in range(e):
        assert torch.equal(dx[g * n:(g + 1) * n].float().cpu(), w1[g]), (g, "grad-input")


def _layer_case(seed, tokens, hidden, inter, experts, k, r, qt):
    gen = torch.Generator().manual_seed(seed)
    pg, pu = _expert_payload(seed, qt, experts, inter, hidden), _expert_payload(seed + 1000, qt, experts, inter, hidden)
    pd = _expert_payload(seed + 2000, qt, experts, hidden, inter)
    x = bf16_randn(gen, tokens, hidden)
    logits = torch.randn(tokens, experts, generator=gen)
    idx, w = rref.router_topk(logits, k)
    a_gu = bf16_randn(gen, experts, r, hidden, std=hidden ** -0.5)
    b_gu = bf16_randn(gen, experts, 2 * inter, r, std=0.01)
    a_d = bf16_randn(gen, experts, r, inter, std=inter ** -0.5)
    b_d = bf16_randn(gen, experts, hidden, r, std=0.01)
    dy = bf16_randn(gen, tokens, hidden)
    return pg, pu, pd, x, idx, w, a_gu, b_gu, a_d, b_d, dy


def _oracle_layer(pg, pu, pd, x, idx, w, a_gu, b_gu, a_d, b_d, dy, qt, s, experts, fused=False):
    tokens, k = idx.shape
    sorted_ids, perm, inv = rref.plan(idx)
    counts = rref.expert_counts(idx, experts)
    ends = torch.cumsum(counts.long(), 0).int()
    sel = rref.gather_forward(x, perm, k)
    weights = (ref.weights_bf16(pg, qt), ref.weights_bf16(pu, qt), ref.weights_bf16(pd, qt))
    if fused:
        # the order of the fused backward: the tokens' cotangent rows unweighted, the routing weight after the grad-input
        row_weight = rref.bf16(w).reshape(-1)[perm].double()  # the path applies routing weights at bf16 precision
        res = ref.expert_layer(sel, torch.arange(experts), ends, *weights, a_gu, b_gu, a_d, b_d, s, dy[perm // k], row_weight=row_weight)
        dw = torch.zeros(tokens * k, dtype=torch.float64)
        dw[perm] = res["dw"]
        dw = dw.reshape(tokens, k)
    else:
        # backward through combine first: dO rows for the sorted layout
        d_o = (dy.float()[perm // k] * rref.bf16(w).reshape(-1)[perm][:, None]).to(torch.bfloat16)
        res = ref.expert_layer(sel, torch.arange(experts), ends, *weights, a_gu, b_gu, a_d, b_d, s, d_o)
        _, dw = rref.combine_backward(dy, ref.bf16_round(res["out"]).to(torch.bfloat16), w, perm)
    out = rref.combine_forward(ref.bf16_round(res["out"]).to(torch.bfloat16), w, inv)
    dx_tok = rref.gather_backward(ref.bf16_round(res["dx"]).to(torch.bfloat16), inv, tokens, k)
    return out, dx_tok, dw, res


@pytest.mark.parametrize("qt,tokens,hidden,inter,experts,k,r", [
    (gb.Q4_K, 8, 2048, 512, 8, 4, 4),        # the reference's one-layer test geometry (test_fast_moe_lora.py:409-470)
    (gb.Q4_K, 300, 512, 256, 16, 8, 16),     # ragged groups, some experts idle, r = 16
    (gb.IQ2_XXS, 64, 512, 512, 8, 2, 16),
    (gb.Q8_0, 40, 256, 128, 4, 2, 8),
])
@pytest.mark.parametrize("fused", [True, False])
def test_expert_layer_forward_backward(pkg, dev, qt, tokens, hidden, inter, experts, k, r, fused, monkeypatch):
    # fused: activation + down projection + combine as one autograd node whose backward never forms the [routes, hidden]
    # cotangent; otherwise the three nodes of the reference's structure.  Both against the same oracle layer.
    ml, G = pkg.fast_moe_lora, pkg.gguf.GGUFQuantizedTensor
    monkeypatch.setattr(ml, "FUSE_GATED_DOWN_COMBINE", fused)
    s = 32.0 / r
    pg, pu, pd, x, idx, w, a_gu, b_gu, a_d, b_d, dy = _layer_case(97531, tokens, hidden, inter, experts, k, r, qt)
    want_out, want_dx, want_dw, res = _oracle_layer(pg, pu, pd, x, idx, w, a_gu, b_gu, a_d, b_d, dy, qt, s, experts, fused)
    mod = ml.GGUFExperts(G(torch.from_numpy(pg).to(dev), qt, (experts, inter, hidden)), G(torch.from_numpy(pu).to(dev), qt, (experts, inter, hidden)),
                         G(torch.from_numpy(pd).to(dev), qt, (experts, hidden, inter)))
    layer = ml.FastGGUFMoeLora(mod, r=r, lora_alpha=32)
    with torch.no_grad():
        layer.lora_A["default"].weight.copy_(a_gu.to(dev)); layer.lora_B["default"].weight.copy_(b_gu.to(dev))
        layer.lora_A_down["default"].weight.copy_(a_d.to(dev)); layer.lora_B_down["default"].weight.copy_(b_d.to(dev))
    xd = x.to(dev).requires_grad_(True)
    wd = w.to(dev).requires_grad_(True)
    out = layer(xd, idx.to(dev), wd)
    out.backward(dy.to(dev))
    assert out.shape == x.shape
    assert_close_bf16(out, want_out.double(), "layer output", ulps=4)
    assert_close_bf16(xd.grad, want_dx.double(), "dHidden", ulps=6)
    assert_close_bf16(wd.grad, want_dw, "dRoutingWeights", ulps=6)
    for name, param, key in (("dA_gate_up", layer.lora_A, "da_gu"), ("dB_gate_up", layer.lora_B, "db_gu"),
                             ("dA_down", layer.lora_A_down, "da_d"), ("dB_down", layer.lora_B_down, "db_d")):
        assert_close_bf16(param["default"].weight.grad, res[key], name, ulps=6)
    active = torch.unique(idx)
    inactive = torch.ones(experts, dtype=torch.bool)
    inactive[active] = False
    for p in layer.parameters():
        assert torch.count_nonzero(p.grad[inactive.to(dev)]) == 0
    for t in (mod.gate_proj, mod.up_proj, mod.down_proj):
        assert t.grad is None
    # a recomputed forward/backward (activation checkpointing) reproduces the same bits
    grads1 = [p.grad.clone() for p in layer.parameters()] + [xd.grad.clone()]
    for p in layer.parameters():
        p.grad = None
    xd.grad = None
    out2 = layer(xd, idx.to(dev), wd)
    out2.backward(dy.to(dev))
    assert torch.equal(out2, out)
    for g1, g2 in zip(grads1, [p.grad for p in layer.parameters()] + [xd.grad]):
        assert torch.equal(g1, g2)


def test_moe_guards(pkg, dev):
    ml = pkg.fast_moe_lora
    x = torch.zeros(6, 256, dtype=torch.bfloat16, device=dev)
    p = torch.zeros(4, 32, 144, dtype=torch.uint8, device=dev)
    ids = torch.tensor([0, 1], dtype=torch.int64, device=dev)
    offs = torch.tensor([3, 6], dtype=torch.int32, device=dev)
    with pytest.raises(TypeError):
        ml.grouped_mmq(x, p, ids.int(), offs, gb.Q4_K, 32)
    with pytest.raises(TypeError):
        ml.grouped_mmq(x, p, ids, offs.long(), gb.Q4_K, 32)
    with pytest.raises(ValueError):
        ml.grouped_mmq(x, p, ids, offs, 11, 32)
    with pytest.raises(ValueError):
        ml.grouped_mmq(x, p, ids, offs, gb.Q4_K, 33)
    with pytest.raises(RuntimeError):
        ml.grouped_mmq_pair(x, p, p[:, :16].contiguous(), ids, offs, gb.Q4_K, 32)
    sizes = ml._group_sizes_from_offsets(offs)
    assert sizes.tolist() == [3, 3]
    assert ml._complete_group_sizes(sizes, ids, 4).tolist() == [3, 3, 0, 0]
    with pytest.raises(ValueError):
        ml._group_sizes_from_offsets(offs.long())


@pytest.mark.parametrize("limit", [7.0, 0.05])
def test_clamped_swiglu_forward_and_gradients(pkg, dev, limit):
    # DeepSeek's expert activation (config.swiglu_limit): the probe of test_deepseek_v4_moe_lora.py:184-199 (inputs four
    # times the limit either way) and random inputs around the limit, against autograd of the clamp expression
    ml = pkg.fast_moe_lora
    gen = torch.Generator().manual_seed(4321)
    probe = torch.tensor([[limit * 4, -limit * 4] * 4], dtype=torch.bfloat16)
    gate = torch.cat([probe, bf16_randn(gen, 63, 8) * limit * 2]).to(torch.bfloat16)
    up = torch.cat([probe, bf16_randn(gen, 63, 8) * limit * 2]).to(torch.bfloat16)
    dh = bf16_randn(gen, 64, 8).to(torch.bfloat16)
    g64, u64 = gate.double().requires_grad_(True), up.double().requires_grad_(True)
    want = ref.silu_mul(g64, u64, limit)
    want.backward(dh.double())
    gd, ud = gate.to(dev).requires_grad_(True), up.to(dev).requires_grad_(True)
    h = ml.swiglu(gd, ud, limit)
    h.backward(dh.to(dev))
    assert_close_bf16(h, want.detach(), "clamped h")
    assert_close_bf16(gd.grad, g64.grad, "clamped dgate")
    assert_close_bf16(ud.grad, u64.grad, "clamped dup")
    # the clamped probe entries: h = silu(limit) * (+-limit), and no gradient reaches a clamped gate or up
    assert float(gd.grad[0, 0]) == 0.0 and float(ud.grad[0, 0]) == 0.0 and float(ud.grad[0, 1]) == 0.0
    with pytest.raises(ValueError):
        ml.swiglu(gd, ud, 0.0)


@pytest.mark.parametrize("limit", [None, 1.5])
@pytest.mark.parametrize("weights_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("qt,with_lora", [(gb.Q4_K, True), (gb.Q6_K, True), (gb.Q4_K, False)])
def test_fused_gated_down_combine_against_the_separate_nodes(pkg, dev, monkeypatch, limit, weights_dtype, qt, with_lora):
    # one autograd node for activation + down projection + combine against the three separate ones: the forward gives the
    # same bits, the gradients agree to rounding (the fused backward applies the routing weight after the grad-input matmul
    # instead of before it, and takes the weights' gradient from the 512-wide side of the projection)
    ml, G = pkg.fast_moe_lora, pkg.gguf.GGUFQuantizedTensor
    tokens, hidden, inter, experts, k, r = 200, 512, 256, 12, 4, 16
    pg, pu, pd, x, idx, w, a_gu, b_gu, a_d, b_d, dy = _layer_case(4242, tokens, hidden, inter, experts, k, r, qt)
    mod = ml.GGUFExperts(G(torch.from_numpy(pg).to(dev), qt, (experts, inter, hidden)), G(torch.from_numpy(pu).to(dev), qt, (experts, inter, hidden)),
                         G(torch.from_numpy(pd).to(dev), qt, (experts, hidden, inter)), swiglu_limit=limit)
    layer = ml.FastGGUFMoeLora(mod, r=r, lora_alpha=32)
    with torch.no_grad():
        layer.lora_A["default"].weight.copy_(a_gu.to(dev)); layer.lora_B["default"].weight.copy_(b_gu.to(dev))
        layer.lora_A_down["default"].weight.copy_(a_d.to(dev)); layer.lora_B_down["default"].weight.copy_(b_d.to(dev))
    layer.disable_adapters = not with_lora
    results = {}
    for fused in (True, False):
        monkeypatch.setattr(ml, "FUSE_GATED_DOWN_COMBINE", fused)
        for p in layer.parameters():
            p.grad = None
        xd = (3.0 * x).to(dev).requires_grad_(True)  # wide enough activations for the clamp to bite
        wd = w.to(weights_dtype).to(dev).requires_grad_(True)
        out = layer(xd, idx.to(dev), wd)
        out.backward(dy.to(dev))
        results[fused] = (out, xd.grad, wd.grad, [None if p.grad is None else p.grad.clone() for p in layer.parameters()])
    (out1, dx1, dw1, g1), (out0, dx0, dw0, g0) = results[True], results[False]
    assert torch.equal(out1, out0)
    assert dw1.dtype == weights_dtype
    # (each order is held to a few bf16 steps of its own oracle in test_expert_layer_forward_backward; the two orders round
    # at different places, so against each other only the path's tolerance holds)
    assert max_rel(dx1, dx0) <= 2e-2 and max_rel(dw1, dw0) <= 2e-2
    for a, b, (name, _) in zip(g1, g0, layer.named_parameters()):
        if with_lora:
            assert max_rel(a, b) <= 2e-2, name
        else:
            assert a is None and b is None


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("qt_gu,qt_d", [(gb.Q4_K, gb.Q4_K), (gb.Q4_K, gb.Q6_K), (gb.Q8_0, gb.Q4_K)])
def test_shared_group_tables_give_the_same_bits(pkg, dev, monkeypatch, fused, qt_gu, qt_d):
    # the row-tile tables built once per step (ggq_group_tables_build) against tables built by every call: same bits in
    # every output and gradient, also where only some of the calls run the kernels the tables serve
    ml, G = pkg.fast_moe_lora, pkg.gguf.GGUFQuantizedTensor
    monkeypatch.setattr(ml, "FUSE_GATED_DOWN_COMBINE", fused)
    tokens, hidden, inter, experts, k, r = 300, 512, 256, 16, 8, 16
    pg, pu, _, x, idx, w, a_gu, b_gu, a_d, b_d, dy = _layer_case(777, tokens, hidden, inter, experts, k, r, qt_gu)
    pd = _layer_case(778, tokens, hidden, inter, experts, k, r, qt_d)[2]
    mod = ml.GGUFExperts(G(torch.from_numpy(pg).to(dev), qt_gu, (experts, inter, hidden)), G(torch.from_numpy(pu).to(dev), qt_gu, (experts, inter, hidden)),
                         G(torch.from_numpy(pd).to(dev), qt_d, (experts, hidden, inter)))
    layer = ml.FastGGUFMoeLora(mod, r=r, lora_alpha=32)
    with torch.no_grad():
        layer.lora_A["default"].weight.copy_(a_gu.to(dev)); layer.lora_B["default"].weight.copy_(b_gu.to(dev))
        layer.lora_A_down["default"].weight.copy_(a_d.to(dev)); layer.lora_B_down["default"].weight.copy_(b_d.to(dev))
    results = []
    for shared in (True, False):
        monkeypatch.setattr(ml, "SHARE_GROUP_TABLES", shared)
        for p in layer.parameters():
            p.grad = None
        xd, wd = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
        out = layer(xd, idx.to(dev), wd)
        out.backward(dy.to(dev))
        results.append([out.detach(), xd.grad, wd.grad] + [p.grad.clone() for p in layer.parameters()])
    for a, b in zip(*results):
        assert torch.equal(a, b)
    lib = pkg._lib.load()
    ids = torch.arange(experts, dtype=torch.int64, device=dev)
    ends = torch.full((experts,), 10, dtype=torch.int32, device=dev).cumsum(0).int()
    need = lib.ggq_group_tables_bytes(160, experts, experts)
    buf = torch.empty(need + 16, dtype=torch.uint8, device=dev)
    assert lib.ggq_group_tables_build(ids.data_ptr(), ends.data_ptr(), experts, experts, 160, buf.data_ptr(), need - 1, None) == -6
    assert lib.ggq_group_tables_build(ids.data_ptr(), ends.data_ptr(), experts, experts, 160, buf.data_ptr() + 8, need, None) == -3
    assert lib.ggq_group_tables_bytes(-1, experts, experts) == -1
