"""Pins oracle/lora_matmul.py without the reference: torch autograd on the same formulas, exact
small-integer cases (every bf16 rounding in the path is then the identity), and structural facts the
reference's tests state (inactive experts get exactly-zero factor gradients, test_fast_moe_lora.py:331-333)."""

import numpy as np
import torch

from oracle import gguf_blocks as gb
from oracle import lora_matmul as lm

from helpers import make_payload, max_rel


def _ints(gen, *shape, lo=-3, hi=4):
    return torch.randint(lo, hi, shape, generator=gen).to(torch.float64)


def test_lora_linear_matches_autograd_exactly_on_small_integers():
    gen = torch.Generator().manual_seed(1)
    m, k, n, r, s = 5, 8, 6, 2, 2.0
    x, w, a, b, dy = _ints(gen, m, k), _ints(gen, n, k), _ints(gen, r, k), _ints(gen, n, r), _ints(gen, m, n)
    xr, ar, br = x.clone().requires_grad_(True), a.clone().requires_grad_(True), b.clone().requires_grad_(True)
    y = xr @ w.T + s * ((xr @ ar.T) @ br.T)
    y.backward(dy)
    got = lm.lora_linear(x.to(torch.bfloat16), w, a.to(torch.bfloat16), b.to(torch.bfloat16), s, dy.to(torch.bfloat16))
    assert torch.equal(got["y"], y.detach())
    assert torch.equal(got["xa"], x @ a.T)
    assert torch.equal(got["dx"], xr.grad)
    assert torch.equal(got["da"], ar.grad)
    assert torch.equal(got["db"], br.grad)


def test_lora_linear_rounds_the_rank_r_intermediates_to_bf16_only():
    """With real-valued operands the only difference from exact autograd is the bf16 rounding of
    x.A^T and dy.B (fast_lora.py:49-55): relative 2^-9 on those factors."""
    gen = torch.Generator().manual_seed(2)
    m, k, n, r, s = 33, 64, 17, 4, 0.5
    x = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    dy = torch.randn(m, n, generator=gen).to(torch.bfloat16)
    a = (torch.randn(r, k, generator=gen) * k ** -0.5).to(torch.bfloat16)
    b = (torch.randn(n, r, generator=gen) * 0.1).to(torch.bfloat16)
    w = torch.randn(n, k, generator=gen).to(torch.bfloat16).double()
    xr, ar, br = (t.double().clone().requires_grad_(True) for t in (x, a, b))
    y = xr @ w.T + s * ((xr @ ar.T) @ br.T)
    y.backward(dy.double())
    got = lm.lora_linear(x, w, a, b, s, dy)
    assert max_rel(got["y"], y) < 2.0 ** -8
    assert max_rel(got["dx"], xr.grad) < 2.0 ** -8
    assert max_rel(got["da"], ar.grad) < 2.0 ** -7
    assert max_rel(got["db"], br.grad) < 2.0 ** -7
    # and the base-only call has no LoRA outputs
    base = lm.lora_linear(x, w, dy=dy)
    assert set(base) == {"y", "dx"} and torch.equal(base["dx"], dy.double() @ w)


def test_grouped_equals_per_expert_dense_and_zeroes_inactive_experts():
    gen = torch.Generator().manual_seed(3)
    e, k, n, r, s = 6, 32, 8, 2, 2.0
    experts, offsets = [0, 2, 5], [2, 5, 6]  # test_fast_moe_lora.py:136-137
    rows = offsets[-1]
    x, dy = _ints(gen, rows, k), _ints(gen, rows, n)
    w = _ints(gen, e, n, k)
    a, b = _ints(gen, e, r, k, lo=-1, hi=2), _ints(gen, e, n, r, lo=-1, hi=2)
    got = lm.grouped_lora_linear(x.to(torch.bfloat16), w, experts, offsets, a.to(torch.bfloat16), b.to(torch.bfloat16), s, dy.to(torch.bfloat16))
    ar, br, xr = a.clone().requires_grad_(True), b.clone().requires_grad_(True), x.clone().requires_grad_(True)
    row_expert = torch.tensor([0, 0, 2, 2, 2, 5])
    y = torch.stack([xr[i] @ w[row_expert[i]].T + s * ((xr[i] @ ar[row_expert[i]].T) @ br[row_expert[i]].T) for i in range(rows)])
    y.backward(dy)
    assert torch.equal(got["y"], y.detach())
    assert torch.equal(got["dx"], xr.grad)
    assert torch.equal(got["da"], ar.grad) and torch.equal(got["db"], br.grad)
    for inactive in (1, 3, 4):
        assert not got["da"][inactive].any() and not got["db"][inactive].any()
    assert lm.group_bounds(offsets) == [(0, 2), (2, 5), (5, 6)]


def test_expert_layer_matches_unrounded_autograd_within_bf16_tolerance():
    gen = torch.Generator().manual_seed(4)
    e, h, i, r, s = 3, 64, 32, 4, 2.0
    experts, offsets = [0, 2], [5, 9]
    rows = offsets[-1]
    rng = np.random.default_rng(4)
    wg, wu = (lm.weights_bf16(gb.quantize((rng.standard_normal((e * i, h)) * 0.1).astype(np.float32), gb.Q8_0), gb.Q8_0).reshape(e, i, h) for _ in range(2))
    wd = lm.weights_bf16(gb.quantize((rng.standard_normal((e * h, i)) * 0.1).astype(np.float32), gb.Q8_0), gb.Q8_0).reshape(e, h, i)
    x = torch.randn(rows, h, generator=gen).to(torch.bfloat16)
    dy = torch.randn(rows, h, generator=gen).to(torch.bfloat16)
    a_gu = (torch.randn(e, r, h, generator=gen) * h ** -0.5).to(torch.bfloat16)
    b_gu = (torch.randn(e, 2 * i, r, generator=gen) * 0.1).to(torch.bfloat16)
    a_d = (torch.randn(e, r, i, generator=gen) * i ** -0.5).to(torch.bfloat16)
    b_d = (torch.randn(e, h, r, generator=gen) * 0.1).to(torch.bfloat16)
    got = lm.expert_layer(x, experts, offsets, wg, wu, wd, a_gu, b_gu, a_d, b_d, s, dy)

    leaves = [t.double().clone().requires_grad_(True) for t in (x, a_gu, b_gu, a_d, b_d)]
    xr, agr, bgr, adr, bdr = leaves
    row_expert = [0] * 5 + [2] * 4
    outs = []
    for row, ex in enumerate(row_expert):
        gu = xr[row] @ torch.cat([wg[ex], wu[ex]]).T + s * ((xr[row] @ agr[ex].T) @ bgr[ex].T)
        hid = torch.nn.functional.silu(gu[:i]) * gu[i:]
        outs.append(hid @ wd[ex].T + s * ((hid @ adr[ex].T) @ bdr[ex].T))
    out = torch.stack(outs)
    out.backward(dy.double())
    assert max_rel(got["out"], out) < 2e-2
    assert max_rel(got["dx"], xr.grad) < 2e-2
    for name, leaf in (("da_gu", agr), ("db_gu", bgr), ("da_d", adr), ("db_d", bdr)):
        assert max_rel(got[name], leaf.grad) < 2e-2, name
        assert not got[name][1].any(), f"{name}: inactive expert 1 must stay zero"
    # SiLU derivative used by the oracle: d/dg [g*sigmoid(g)] = sig*(1 + g*(1 - sig))
    g = torch.linspace(-4, 4, 33, dtype=torch.float64, requires_grad=True)
    torch.nn.functional.silu(g).sum().backward()
    sig = torch.sigmoid(g.detach())
    assert torch.allclose(g.grad, sig * (1 + g.detach() * (1 - sig)), atol=1e-12)


def test_expert_layer_with_row_weights_matches_autograd_of_the_weighted_sum():
    # the order of the backward that folds the combine into the down projection: the cotangent arrives unweighted, the
    # weight is applied after the grad-input.  Pinned by autograd of sum_r w_r <dy_r, out_r> in float64 without roundings:
    # input and factor gradients within the bf16 tolerance, and the weight gradient <dh_unweighted, h> against d/dw_r.
    gen = torch.Generator().manual_seed(8)
    e, h, i, r, s = 3, 64, 32, 4, 2.0
    experts, offsets = [0, 2], [5, 9]
    rows = offsets[-1]
    rng = np.random.default_rng(8)
    wg, wu = (lm.weights_bf16(gb.quantize((rng.standard_normal((e * i, h)) * 0.1).astype(np.float32), gb.Q8_0), gb.Q8_0).reshape(e, i, h) for _ in range(2))
    wd = lm.weights_bf16(gb.quantize((rng.standard_normal((e * h, i)) * 0.1).astype(np.float32), gb.Q8_0), gb.Q8_0).reshape(e, h, i)
    x = torch.randn(rows, h, generator=gen).to(torch.bfloat16)
    dy = torch.randn(rows, h, generator=gen).to(torch.bfloat16)
    w = torch.rand(rows, generator=gen).double() + 0.1
    a_gu = (torch.randn(e, r, h, generator=gen) * h ** -0.5).to(torch.bfloat16)
    b_gu = (torch.randn(e, 2 * i, r, generator=gen) * 0.1).to(torch.bfloat16)
    a_d = (torch.randn(e, r, i, generator=gen) * i ** -0.5).to(torch.bfloat16)
    b_d = (torch.randn(e, h, r, generator=gen) * 0.1).to(torch.bfloat16)
    # the clamp is a discontinuity of the gradient: put the limit in the middle of the widest gap between the gate / up
    # magnitudes, so that the bf16 rounding of gate and up moves no value across it
    plain = lm.expert_layer(x, experts, offsets, wg, wu, wd, a_gu, b_gu, a_d, b_d, s)
    mags = torch.cat([plain["gate"].reshape(-1), plain["up"].reshape(-1)]).abs().sort().values
    mags = mags[(mags > 0.3) & (mags < 1.0)]
    gap = int((mags[1:] - mags[:-1]).argmax())
    limit = float((mags[gap] + mags[gap + 1]) / 2)
    assert float(mags[gap + 1] - mags[gap]) > 0.01  # bf16 rounding moves a value of this size by at most 0.002
    for lim in (None, limit):
        got = lm.expert_layer(x, experts, offsets, wg, wu, wd, a_gu, b_gu, a_d, b_d, s, dy, row_weight=w, limit=lim)
        leaves = [t.double().clone().requires_grad_(True) for t in (x, a_gu, b_gu, a_d, b_d, w)]
        xr, agr, bgr, adr, bdr, wr = leaves
        row_expert = [0] * 5 + [2] * 4
        total = 0.0
        for row, ex in enumerate(row_expert):
            gu = xr[row] @ torch.cat([wg[ex], wu[ex]]).T + s * ((xr[row] @ agr[ex].T) @ bgr[ex].T)
            hid = lm.silu_mul(gu[:i], gu[i:], lim)
            out = hid @ wd[ex].T + s * ((hid @ adr[ex].T) @ bdr[ex].T)
            total = total + wr[row] * (out * dy[row].double()).sum()
        total.backward()
        assert max_rel(got["dx"], xr.grad) < 2e-2
        assert max_rel(got["dw"], wr.grad) < 2e-2
        for name, leaf in (("da_gu", agr), ("db_gu", bgr), ("da_d", adr), ("db_d", bdr)):
            assert max_rel(got[name], leaf.grad) < 2e-2, (name, lim)
        # the same layer with the weight folded into the cotangent beforehand (the reference's order) agrees to rounding
        pre = lm.expert_layer(x, experts, offsets, wg, wu, wd, a_gu, b_gu, a_d, b_d, s, (dy.double() * w[:, None]).to(torch.bfloat16), limit=lim)
        for name in ("dx", "da_gu", "db_gu", "da_d", "db_d"):
            assert max_rel(got[name], pre[name]) < 2e-2, (name, lim)
    assert (got["gate"] > limit).any() or (got["up"].abs() > limit).any()  # the clamp was exercised


def test_grouped_mm_matches_autograd_of_the_group_loop():
    """The closed-form gradients of the grouped product (a transposed operand or a group boundary off by one fails here),
    rows no group covers included."""
    gen = torch.Generator().manual_seed(31)
    m, k, n, sizes = 11, 5, 4, [3, 0, 4, 2]  # two rows left over
    lhs = torch.randint(-4, 5, (m, k), generator=gen).double().requires_grad_(True)
    rhs = torch.randint(-4, 5, (len(sizes), k, n), generator=gen).double().requires_grad_(True)
    dy = torch.randint(-4, 5, (m, n), generator=gen).double()
    pieces, r0 = [], 0
    for e, size in enumerate(sizes):
        pieces.append(lhs[r0:r0 + size] @ rhs[e])
        r0 += size
    pieces.append(torch.zeros(m - r0, n, dtype=torch.float64))
    out = torch.cat(pieces)
    dlhs, drhs = torch.autograd.grad(out, (lhs, rhs), dy)
    got = lm.grouped_mm(lhs.detach(), rhs.detach(), sizes, dy)
    assert torch.equal(got["out"], out.detach())
    assert torch.equal(got["dlhs"], dlhs)
    assert torch.equal(got["drhs"], drhs)
    assert torch.count_nonzero(got["drhs"][1]) == 0 and torch.count_nonzero(got["dlhs"][r0:]) == 0
    # sizes running past the last row are clipped
    clipped = lm.grouped_mm(lhs.detach(), rhs.detach(), [3, 0, 4, 100], dy)
    assert torch.equal(clipped["out"][:7], out.detach()[:7]) and torch.equal(clipped["out"][7:], lhs.detach()[7:] @ rhs.detach()[3])
