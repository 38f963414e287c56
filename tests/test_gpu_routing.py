"""Routing layout parity: plan indices, offsets and gather bit-exact; combine within one bf16 step
(relations of test_fast_moe_routing.py:125-167, 170-240)."""

import pytest
import torch

from oracle import routing as ref

pytestmark = pytest.mark.gpu


def _indices(seed, tokens, k, experts, dtype=torch.int64):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, experts, (tokens, k), generator=g, dtype=dtype)


@pytest.mark.parametrize("tokens,k,experts,dtype", [(2048, 8, 256, torch.int64), (333, 6, 256, torch.int32), (8, 4, 8, torch.int64),
                                                     (1, 1, 3, torch.int64), (4096, 8, 256, torch.int64), (700, 16, 1000, torch.int64)])
def test_route_plan_is_bit_exact(pkg, dev, tokens, k, experts, dtype):
    idx = _indices(19260817, tokens, k, experts, dtype)
    want_sorted, want_perm, want_inv = ref.plan(idx)
    want_counts = ref.expert_counts(idx, experts)
    want_active, want_ends = ref.active_offsets(want_counts)
    sorted_ids, perm, inv, counts, ends, active_ids, active_ends, status = pkg.fast_moe_routing.build_route_plan(idx.to(dev), experts)
    torch.cuda.synchronize()
    assert torch.equal(sorted_ids.cpu(), want_sorted)
    assert torch.equal(perm.cpu(), want_perm)
    assert torch.equal(inv.cpu(), want_inv)
    assert torch.equal(counts.cpu(), want_counts)
    assert torch.equal(ends.cpu(), torch.cumsum(want_counts.long(), 0).int())
    n_active = int(status[0])
    assert n_active == want_active.numel() and int(status[1]) == 0
    assert torch.equal(active_ids[:n_active].cpu(), want_active)
    assert torch.equal(active_ends[:n_active].cpu(), want_ends)
    # closed forms (test_fast_moe_routing.py:64-67)
    assert torch.equal(inv.cpu()[perm.cpu()], torch.arange(tokens * k))
    assert bool((sorted_ids[1:] >= sorted_ids[:-1]).all())


def test_route_plan_all_routes_to_one_expert_and_bad_ids(pkg, dev):
    idx = torch.full((300, 8), 5, dtype=torch.int64)
    sorted_ids, perm, inv, counts, ends, active_ids, active_ends, status = pkg.fast_moe_routing.build_route_plan(idx.to(dev), 16)
    assert torch.equal(perm.cpu(), torch.arange(2400)) and int(counts[5]) == 2400 and int(status[0]) == 1
    idx[7, 3] = 99  # outside [0, 16): clamped for memory safety and reported
    *_, status = pkg.fast_moe_routing.build_route_plan(idx.to(dev), 16)
    assert int(status[1]) == 1
    pkg.fast_moe_routing.VALIDATE_EXPERT_IDS = True  # the debugging switch turns the flag into an error (and a synchronisation)
    try:
        with pytest.raises(ValueError):
            pkg.fast_moe_routing.build_route_plan(idx.to(dev), 16)
    finally:
        pkg.fast_moe_routing.VALIDATE_EXPERT_IDS = False


@pytest.mark.parametrize("bad_routes", [[300], [70 * 256 + 5], [256 * c + (c % 7) for c in range(1, 70)], [256 * 63 + 255], [20479]])
def test_route_plan_reports_a_bad_id_in_any_chunk(pkg, dev, bad_routes):
    """The flag must be raised wherever the id sits: the sort works in chunks of 256 routes whose flags one workgroup
    gathers with a wave vote, so ids in chunks 1, 63, 70 and in every chunk of a run are tried, negative ones too."""
    idx = _indices(86420, 2560, 8, 16).reshape(-1)
    *_, status = pkg.fast_moe_routing.build_route_plan(idx.reshape(2560, 8).to(dev), 16)
    assert int(status[1]) == 0
    for n, r in enumerate(bad_routes):
        idx[r] = 16 if n % 2 == 0 else -1
    sorted_ids, *_, status = pkg.fast_moe_routing.build_route_plan(idx.reshape(2560, 8).to(dev), 16)
    assert int(status[1]) == 1
    assert int(sorted_ids.min()) >= 0 and int(sorted_ids.max()) < 16  # clamped: no access leaves the buffers


@pytest.mark.parametrize("tokens,k,hidden", [(2048, 8, 2048), (257, 6, 4096), (8, 4, 2048), (64, 8, 4096), (5, 1, 256)])
def test_gather_forward_backward_exact(pkg, dev, tokens, k, hidden):
    g = torch.Generator().manual_seed(2468)
    idx = _indices(2468, tokens, k, 256)
    hid = torch.randn(tokens, hidden, generator=g).to(torch.bfloat16)
    w = torch.softmax(torch.randn(tokens, k, generator=g), dim=-1)
    _, perm, inv = ref.plan(idx)
    h = hid.to(dev).requires_grad_(True)
    plan = pkg.fast_moe_routing.prepare_expert_routing(h, idx.to(dev), w.to(dev), 256)
    assert torch.equal(plan.selected_hidden_states.cpu(), ref.gather_forward(hid, perm, k))
    grad_sel = torch.randn(tokens * k, hidden, generator=g).to(torch.bfloat16)
    plan.selected_hidden_states.backward(grad_sel.to(dev))
    want = ref.gather_backward(grad_sel, inv, tokens, k)
    assert torch.equal(h.grad.cpu(), want), "gather backward must reproduce the per-add bf16 rounding order"


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tokens,k,hidden", [(2048, 8, 2048), (100, 6, 4096), (8, 4, 2048)])
def test_combine_forward_backward(pkg, dev, tokens, k, hidden, wdtype):
    g = torch.Generator().manual_seed(97531)
    idx = _indices(97531, tokens, k, 256)
    hid = torch.randn(tokens, hidden, generator=g).to(torch.bfloat16)
    w = torch.softmax(torch.randn(tokens, k, generator=g), dim=-1).to(wdtype)
    out = torch.randn(tokens * k, hidden, generator=g).to(torch.bfloat16)
    grad = torch.randn(tokens, hidden, generator=g).to(torch.bfloat16)
    _, perm, inv = ref.plan(idx)
    plan = pkg.fast_moe_routing.prepare_expert_routing(hid.to(dev), idx.to(dev), w.to(dev).requires_grad_(True), 256)
    o = out.to(dev).requires_grad_(True)
    res = pkg.fast_moe_routing.finalize_expert_routing(o, hid.to(dev), plan, None)
    want = ref.combine_forward(out, w, inv)
    # one bf16 step (test_fast_moe_routing.py:217 uses atol 2^-6 on O(1) values)
    err = (res.float().cpu() - want.float()).abs()
    assert float(err.max()) <= 2.0 ** -7 * max(1.0, float(want.float().abs().max()))
    assert float((err > 0).float().mean()) < 0.02, "more than 2% of elements differ from the fp32-accumulated oracle"
    res.backward(grad.to(dev))
    want_do, want_dw = ref.combine_backward(grad, out, w, perm)
    assert torch.equal(o.grad.cpu(), want_do), "combine dO must be exact"
    dw = plan.routing_weights.grad.double().cpu()
    rel_rmse = float(((dw - want_dw) ** 2).mean().sqrt() / (want_dw ** 2).mean().sqrt())
    assert rel_rmse < (1e-5 if wdtype == torch.float32 else 5e-3)


def test_routing_guards(pkg, dev):
    r = pkg.fast_moe_routing
    hid = torch.zeros(8, 64, dtype=torch.bfloat16, device=dev)
    idx = torch.zeros(8, 2, dtype=torch.int64, device=dev)
    w = torch.zeros(8, 2, device=dev)
    with pytest.raises(ValueError):
        r.prepare_expert_routing(hid[None], idx, w, 4)
    with pytest.raises(ValueError):
        r.prepare_expert_routing(hid, idx[:4], w[:4], 4)
    with pytest.raises(RuntimeError):
        r.prepare_expert_routing(hid.float(), idx, w, 4)
    with pytest.raises(RuntimeError):
        r.prepare_expert_routing(hid, idx.float(), w, 4)
    with pytest.raises(RuntimeError):
        r.prepare_expert_routing(hid, idx, w.half(), 4)
    plan = r.prepare_expert_routing(hid, idx, w, 4)
    with pytest.raises(RuntimeError):
        r.finalize_expert_routing(torch.zeros(16, 64, dtype=torch.bfloat16, device=dev), hid, plan, torch.ones(1, device=dev))
    with pytest.raises(RuntimeError):
        r.finalize_expert_routing(torch.zeros(15, 64, dtype=torch.bfloat16, device=dev), hid, plan, None)
