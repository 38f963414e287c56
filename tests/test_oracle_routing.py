"""Pins oracle/routing.py: brute-force loops, closed forms the reference's tests use
(test_fast_moe_routing.py:64-67,146-150,211-214) and the worked offsets example of
test_fast_moe_lora.py:136-138."""

import torch

from oracle import routing as rt


def _bf16_add(a: float, b: float) -> float:
    return float(torch.tensor(a + b, dtype=torch.float32).to(torch.bfloat16))


def test_plan_is_a_stable_sort_with_its_inverse():
    gen = torch.Generator().manual_seed(2468)
    ids = torch.randint(0, 7, (13, 3), generator=gen)
    sorted_ids, perm, inv = rt.plan(ids)
    flat = ids.reshape(-1).tolist()
    want_perm = sorted(range(len(flat)), key=lambda i: (flat[i], i))  # ties keep route order
    assert perm.tolist() == want_perm
    assert sorted_ids.tolist() == [flat[i] for i in want_perm]
    assert torch.equal(inv[perm], torch.arange(len(flat)))
    assert torch.equal(perm[inv], torch.arange(len(flat)))
    assert sorted_ids.dtype == perm.dtype == inv.dtype == torch.int64


def test_counts_and_active_offsets_worked_example():
    ids = torch.tensor([[0, 2], [2, 5], [0, 2]])  # experts 0,2,5 with 2,3,1 rows
    counts = rt.expert_counts(ids, 6)
    assert counts.tolist() == [2, 0, 3, 0, 0, 1] and counts.dtype == torch.int32
    active, ends = rt.active_offsets(counts)
    assert active.tolist() == [0, 2, 5] and ends.tolist() == [2, 5, 6]
    assert active.dtype == torch.int64 and ends.dtype == torch.int32


def test_gather_forward_and_backward_brute_force():
    gen = torch.Generator().manual_seed(97531)
    t, k, h = 6, 3, 5
    ids = torch.randint(0, 4, (t, k), generator=gen)
    _, perm, inv = rt.plan(ids)
    hidden = torch.randn(t, h, generator=gen).to(torch.bfloat16)
    sel = rt.gather_forward(hidden, perm, k)
    for s_pos in range(t * k):
        assert torch.equal(sel[s_pos], hidden[int(perm[s_pos]) // k])
    grad_sel = torch.randn(t * k, h, generator=gen).to(torch.bfloat16)
    got = rt.gather_backward(grad_sel, inv, t, k)
    for tok in range(t):
        positions = sorted(int(inv[tok * k + j]) for j in range(k))
        for col in range(h):
            acc = 0.0
            for pos in positions:  # ascending sorted position, rounded after every add
                acc = _bf16_add(acc, float(grad_sel[pos, col]))
            assert float(got[tok, col]) == acc
    # k = 1: the backward is the inverse scatter
    ids1 = torch.randint(0, 4, (t, 1), generator=gen)
    _, perm1, inv1 = rt.plan(ids1)
    g1 = torch.randn(t, h, generator=gen).to(torch.bfloat16)
    assert torch.equal(rt.gather_backward(g1, inv1, t, 1), g1[inv1])


def test_combine_forward_and_backward():
    gen = torch.Generator().manual_seed(86420)
    t, k, h = 5, 4, 6
    ids = torch.randint(0, 8, (t, k), generator=gen)
    _, perm, inv = rt.plan(ids)
    o = torch.randn(t * k, h, generator=gen).to(torch.bfloat16)
    w = torch.softmax(torch.randn(t, k, generator=gen), dim=1)
    got = rt.combine_forward(o, w, inv)
    wb = w.to(torch.bfloat16).double()
    want = torch.einsum("tk,tkh->th", wb, o.double()[inv].reshape(t, k, h))  # test_fast_moe_routing.py:211-214
    assert (got.double() - want).abs().max() <= 2.0 ** -8 * want.abs().max()
    # rank-ordered fp32 accumulation, one rounding at the end
    for tok in range(t):
        acc = torch.zeros(h, dtype=torch.float32)
        for rank in range(k):
            acc = acc + o[int(inv[tok * k + rank])].float() * w[tok, rank].to(torch.bfloat16).float()
        assert torch.equal(got[tok], acc.to(torch.bfloat16))
    g = torch.randn(t, h, generator=gen).to(torch.bfloat16)
    d_o, d_w = rt.combine_backward(g, o, w, perm)
    for s_pos in range(t * k):
        route = int(perm[s_pos])
        want_row = (g[route // k].float() * w.reshape(-1)[route].to(torch.bfloat16).float()).to(torch.bfloat16)
        assert torch.equal(d_o[s_pos], want_row)
    wr = wb.clone().requires_grad_(True)
    torch.einsum("tk,tkh->th", wr, o.double()[inv].reshape(t, k, h)).backward(g.double())
    assert torch.allclose(d_w, wr.grad, rtol=1e-12, atol=1e-12)


def test_router_topk_tie_break_and_weights():
    ids, weights = rt.router_topk(torch.zeros(3, 9), 4)  # test_fast_moe_ranking.py:183-201
    assert ids.tolist() == [[0, 1, 2, 3]] * 3
    assert torch.allclose(weights, torch.full((3, 4), 0.25))
    logits = torch.tensor([[0.5, 2.0, 2.0, -1.0, 3.0]])
    ids, weights = rt.router_topk(logits, 3)
    assert ids.tolist() == [[4, 1, 2]]
    assert torch.allclose(weights, torch.softmax(torch.tensor([[3.0, 2.0, 2.0]]), dim=1))
