"""The grouped bf16 products that stand for AITER's gmm / ptgmm (fast_moe_lora.py:22, 42-151) against the per-group loop,
through ctypes (``grouped_mm.gmm`` / ``ptgmm`` call ``ggq_gmm`` / ``ggq_ptgmm``); relations of test_fast_moe_lora.py:280-404.
AITER's own output is parity unpinned: it is not importable here and the reference holds no vectors of it."""

import pytest
import torch
from torch.utils.checkpoint import checkpoint

from helpers import MAX_REL, assert_close_bf16, bf16_randn, make_payload, max_rel
from oracle import gguf_blocks as gb
from oracle import lora_matmul as ref
from oracle import routing as rref

pytestmark = pytest.mark.gpu


def _assert_product(got, want, lhs_abs_rhs_abs, what):
    """One bf16 rounding of an fp32 sum: half an ulp of the value plus the sum's own rounding noise."""
    got64, want64 = got.double().cpu(), want
    assert got64.shape == want64.shape, f"{what}: shape {tuple(got64.shape)} vs {tuple(want64.shape)}"
    tol = 2.0 ** -8 * want64.abs() + 2.0 ** -18 * lhs_abs_rhs_abs + 1e-30
    bad = (got64 - want64).abs() > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} off (worst {float(((got64 - want64).abs() / tol).max()):.2f}x)"


CASES = [  # m, k, n, group sizes
    (6, 16, 4, [2, 0, 3, 0, 0, 1, 0, 0]),            # the reference test's shape (test_fast_moe_lora.py:282-311)
    (300, 64, 48, [130, 0, 1, 169]),                 # a group ending inside a tile, an empty one, a one-row one
    (257, 40, 136, [128, 129]),                      # k, n multiples of 8 but not of the step / tile
    (70, 37, 19, [33, 37]),                          # odd k and n: element loads and stores
    (513, 2048, 16, [200, 0, 313]),                  # x . A^T of an expert layer
    (513, 16, 1024, [200, 0, 313]),                  # (x A^T) . B^T
    (100, 128, 128, [30, 20]),                       # 50 rows no group covers: zero rows
    (64, 96, 80, [50, 50]),                          # sizes past the last row are clipped
    (1, 8, 8, [1]),
    (1500, 24, 40, [3, 0] * 500),                    # a thousand groups: the plan's threads walk several groups each
]


@pytest.mark.parametrize("m,k,n,sizes", CASES, ids=[f"{c[0]}x{c[1]}x{c[2]}" for c in CASES])
@pytest.mark.parametrize("k_contiguous", [True, False], ids=["rhs_nk", "rhs_kn"])
def test_gmm_and_ptgmm_against_the_group_loop(pkg, dev, m, k, n, sizes, k_contiguous):
    gm = pkg.grouped_mm
    gen = torch.Generator().manual_seed(m * 7 + k * 3 + n)
    experts = len(sizes)
    lhs, dy = bf16_randn(gen, m, k), bf16_randn(gen, m, n)
    planes = bf16_randn(gen, experts, k, n, std=0.5)
    gs = torch.tensor(sizes, dtype=torch.int32)
    want = ref.grouped_mm(lhs, planes, sizes, dy)
    lhs_d, dy_d, gs_d = lhs.to(dev), dy.to(dev), gs.to(dev)
    rhs_d = planes.transpose(1, 2).contiguous().to(dev).transpose(1, 2) if k_contiguous else planes.to(dev)
    assert rhs_d.shape == (experts, k, n)
    out = gm.gmm(lhs_d, rhs_d, gs_d, preferred_element_type=torch.bfloat16)
    mag = ref.grouped_mm(lhs.abs(), planes.abs(), sizes)["out"]
    _assert_product(out, want["out"], mag, "gmm")
    covered = min(m, sum(sizes))
    assert torch.count_nonzero(out[covered:]) == 0
    # the gradient of lhs is the same product against the transposed planes (fast_moe_lora.py:55-68)
    dlhs = gm.gmm(dy_d, rhs_d.transpose(1, 2), gs_d)
    _assert_product(dlhs, want["dlhs"], ref.grouped_mm(dy.abs(), planes.abs().transpose(1, 2), sizes)["out"], "gmm against transposed planes")
    if k_contiguous:
        return
    drhs = gm.ptgmm(lhs_d.T, dy_d, gs_d, preferred_element_type=torch.bfloat16)
    mag_w = ref.grouped_mm(lhs.abs(), planes.abs(), sizes, dy.abs())["drhs"]
    _assert_product(drhs, want["drhs"], mag_w, "ptgmm")
    r0 = 0
    for e, size in enumerate(sizes):
        if min(m, r0 + size) == r0:
            assert torch.count_nonzero(drhs[e]) == 0, f"plane {e} of a group without rows is not zero"
        r0 = min(m, r0 + size)


def test_half_precision_operands(pkg, dev):
    """The reference's wrapper admits fp16 as well (fast_moe_lora.py:116-119): same relations, fp16 roundings."""
    gm = pkg.grouped_mm
    gen = torch.Generator().manual_seed(17)
    m, k, n, sizes = 300, 72, 40, [130, 0, 1, 169]
    lhs = torch.randn(m, k, generator=gen).half()
    planes = (0.5 * torch.randn(len(sizes), k, n, generator=gen)).half()
    dy = torch.randn(m, n, generator=gen).half()
    want = ref.grouped_mm(lhs, planes, sizes, dy)
    gs = torch.tensor(sizes, dtype=torch.int32, device=dev)
    tol = lambda w, mag: 2.0 ** -11 * w.abs() + 2.0 ** -18 * mag + 1e-30  # half an fp16 ulp + the fp32 sum's noise

    def close(got, w, mag, what):
        assert got.dtype == torch.float16
        bad = (got.double().cpu() - w).abs() > tol(w, mag)
        assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} off"

    mag = ref.grouped_mm(lhs.abs(), planes.abs(), sizes, dy.abs())
    for rhs_d in (planes.to(dev), planes.transpose(1, 2).contiguous().to(dev).transpose(1, 2)):
        close(gm.gmm(lhs.to(dev), rhs_d, gs), want["out"], mag["out"], "gmm fp16")
    close(gm.gmm(dy.to(dev), planes.to(dev).transpose(1, 2), gs), want["dlhs"], ref.grouped_mm(dy.abs(), planes.abs().transpose(1, 2), sizes)["out"], "gmm fp16 transposed planes")
    close(gm.ptgmm(lhs.to(dev).T, dy.to(dev), gs), want["drhs"], mag["drhs"], "ptgmm fp16")
    lhs_d, planes_d = lhs.to(dev).requires_grad_(True), planes.to(dev).requires_grad_(True)
    out = gm.aiter_grouped_mm(lhs_d, planes_d, gs)
    out.backward(dy.to(dev))
    close(lhs_d.grad, want["dlhs"], ref.grouped_mm(dy.abs(), planes.abs().transpose(1, 2), sizes)["out"], "autograd d lhs fp16")
    close(planes_d.grad, want["drhs"], mag["drhs"], "autograd d planes fp16")


def test_degenerate_sizes(pkg, dev):
    """No rows, no contraction, no columns: nothing faults, and what is defined is zero."""
    gm = pkg.grouped_mm
    bf = lambda *shape: torch.ones(*shape, dtype=torch.bfloat16, device=dev)
    gs = torch.tensor([0, 0, 0], dtype=torch.int32, device=dev)
    assert gm.gmm(bf(0, 8), bf(3, 8, 5), gs).shape == (0, 5)
    assert gm.gmm(bf(4, 8), bf(3, 8, 0), torch.tensor([1, 2, 1], dtype=torch.int32, device=dev)).shape == (4, 0)
    out = gm.gmm(bf(4, 0), bf(3, 0, 5), torch.tensor([1, 2, 1], dtype=torch.int32, device=dev))   # an empty contraction sums to zero
    assert out.shape == (4, 5) and torch.count_nonzero(out) == 0
    planes = gm.ptgmm(bf(0, 8).T, bf(0, 5), gs)
    assert planes.shape == (3, 8, 5) and torch.count_nonzero(planes) == 0
    out = gm.gmm(bf(4, 8), bf(3, 8, 5), gs)                                                        # rows, but no group owns any
    assert torch.count_nonzero(out) == 0
    neg = gm.gmm(bf(4, 8), bf(2, 8, 5), torch.tensor([-3, 4], dtype=torch.int32, device=dev))      # a negative size counts as zero
    assert torch.equal(neg, (bf(4, 8).float() @ bf(8, 5).float()).to(torch.bfloat16))
    torch.cuda.synchronize()


def test_unaligned_bases_take_the_element_path(pkg, dev):
    gm = pkg.grouped_mm
    gen = torch.Generator().manual_seed(5)
    m, k, n, sizes = 90, 24, 40, [40, 50]
    lhs, planes = bf16_randn(gen, m, k), bf16_randn(gen, 2, k, n)
    want = ref.grouped_mm(lhs, planes, sizes)["out"]
    store = torch.empty(m * k + 1, dtype=torch.bfloat16, device=dev)
    lhs_d = store[1:].view(m, k)  # 2-byte aligned only
    lhs_d.copy_(lhs)
    pstore = torch.empty(2 * k * n + 3, dtype=torch.bfloat16, device=dev)
    planes_d = pstore[3:].view(2, k, n)
    planes_d.copy_(planes)
    out = gm.gmm(lhs_d, planes_d, torch.tensor(sizes, dtype=torch.int32, device=dev))
    _assert_product(out, want, ref.grouped_mm(lhs.abs(), planes.abs(), sizes)["out"], "gmm on unaligned operands")


def test_grouped_mm_autograd_full_and_compact_expert_lists_agree(pkg, dev):
    """test_fast_moe_lora.py:282-360: all planes with zero-sized groups == the active planes only, bit for bit; planes of
    inactive experts get exactly zero gradients; checkpoint replay reproduces the bits."""
    gm = pkg.grouped_mm
    gen = torch.Generator().manual_seed(11)
    active = torch.tensor([0, 2, 5], device=dev)
    full_sizes = torch.tensor([2, 0, 3, 0, 0, 1, 0, 0], dtype=torch.int32, device=dev)
    active_sizes = torch.tensor([2, 3, 1], dtype=torch.int32, device=dev)
    lhs = bf16_randn(gen, 6, 16).to(dev).requires_grad_(True)
    factor = bf16_randn(gen, 8, 4, 16).to(dev).requires_grad_(True)
    grad_output = bf16_randn(gen, 6, 4).to(dev)
    ref_lhs, ref_factor = lhs.detach().clone().requires_grad_(), factor.detach().clone().requires_grad_()
    output = gm.aiter_grouped_mm(lhs, factor.transpose(1, 2), full_sizes)
    reference = gm.aiter_grouped_mm(ref_lhs, ref_factor.index_select(0, active).transpose(1, 2), active_sizes)
    gradients = torch.autograd.grad(output, (lhs, factor), grad_output)
    reference_gradients = torch.autograd.grad(reference, (ref_lhs, ref_factor), grad_output)
    assert torch.equal(output, reference)
    for g, r in zip(gradients, reference_gradients):
        assert torch.equal(g, r)
    inactive = torch.ones(8, dtype=torch.bool, device=dev)
    inactive[active] = False
    assert torch.count_nonzero(gradients[1][inactive]) == 0
    # against the group loop
    want = ref.grouped_mm(lhs.detach().cpu(), factor.detach().cpu().transpose(1, 2), full_sizes.tolist(), grad_output.cpu())
    assert_close_bf16(output, want["out"], "out")
    assert_close_bf16(gradients[0], want["dlhs"], "d lhs")
    assert_close_bf16(gradients[1], want["drhs"].transpose(1, 2), "d factor")
    ck_lhs, ck_factor = lhs.detach().clone().requires_grad_(), factor.detach().clone().requires_grad_()
    ck_out = checkpoint(lambda a, b: gm.aiter_grouped_mm(a, b.transpose(1, 2), full_sizes), ck_lhs, ck_factor, use_reentrant=False)
    ck_grads = torch.autograd.grad(ck_out, (ck_lhs, ck_factor), grad_output)
    assert torch.equal(ck_out, output)
    for g, r in zip(ck_grads, gradients):
        assert torch.equal(g, r)


def test_grouped_mm_rejects_layout_repairs(pkg, dev):
    """test_fast_moe_lora.py:387-404."""
    gm = pkg.grouped_mm
    lhs = torch.randn(16, 6, device=dev, dtype=torch.bfloat16).T
    factor = torch.randn(3, 4, 16, device=dev, dtype=torch.bfloat16)
    sizes = torch.tensor([2, 2, 2], device=dev, dtype=torch.int32)
    with pytest.raises(ValueError, match="lhs must be row-major"):
        gm.aiter_grouped_mm(lhs, factor.transpose(1, 2), sizes)
    valid_lhs = torch.randn(6, 16, device=dev, dtype=torch.bfloat16, requires_grad=True)
    valid_factor = factor.detach().requires_grad_()
    output = gm.aiter_grouped_mm(valid_lhs, valid_factor.transpose(1, 2), sizes)
    strided = torch.randn(output.shape[1], output.shape[0], device=dev, dtype=torch.bfloat16).T
    with pytest.raises(ValueError, match="output gradient must be row-major"):
        torch.autograd.grad(output, (valid_lhs, valid_factor), strided)
    with pytest.raises(ValueError, match="contiguous int32"):
        gm.aiter_grouped_mm(valid_lhs, valid_factor.transpose(1, 2), sizes.long())
    with pytest.raises(TypeError, match="FP16/BF16"):
        gm.aiter_grouped_mm(valid_lhs.float(), valid_factor.float().transpose(1, 2), sizes)
    with pytest.raises(TypeError, match="FP16/BF16"):
        gm.aiter_grouped_mm(valid_lhs, valid_factor.half().transpose(1, 2), sizes)
    with pytest.raises(ValueError, match="K mismatch"):
        gm.aiter_grouped_mm(valid_lhs[:, :8].contiguous(), valid_factor.transpose(1, 2), sizes)
    with pytest.raises(ValueError, match="dense"):
        gm.gmm(valid_lhs, torch.randn(3, 16, 8, device=dev, dtype=torch.bfloat16)[:, :, ::2], sizes)
    lib = pkg._lib.load()
    assert lib.ggq_gmm(valid_lhs.data_ptr(), factor.data_ptr(), sizes.data_ptr(), output.data_ptr(), 6, 16, 4, 3, 1, 0, sizes.data_ptr(), 4, None) == -6
    assert b"workspace" in lib.ggq_last_error()


def _layer_inputs(gen, tokens, top_k, experts, hidden, inter, r):
    x = bf16_randn(gen, tokens, hidden)
    idx = torch.stack([torch.randperm(experts, generator=gen)[:top_k] for _ in range(tokens)]).to(torch.int64)
    wts = torch.softmax(torch.randn(tokens, top_k, generator=gen), dim=-1)
    a_gu, b_gu = bf16_randn(gen, experts, r, hidden, std=0.05), bf16_randn(gen, experts, 2 * inter, r, std=0.05)
    a_d, b_d = bf16_randn(gen, experts, r, inter, std=0.05), bf16_randn(gen, experts, hidden, r, std=0.05)
    dy = bf16_randn(gen, tokens, hidden)
    return x, idx, wts, (a_gu, b_gu, a_d, b_d), dy


def _run_layer(ml, module, dev, x, idx, wts, factors, dy, s):
    xd = x.to(dev).requires_grad_(True)
    fs = [f.to(dev).requires_grad_(True) for f in factors]
    lw = ml._ExpertLoraWeights(*fs, scaling=s)
    out = module(xd, idx.to(dev), wts.to(dev), lw)
    out.backward(dy.to(dev))
    return out.detach(), xd.grad, [f.grad for f in fs]


def _assert_layer_close(got, want, what):
    """The separated order rounds the base output, each delta and their sum on their own, so single elements stray further
    from the oracle (which rounds where the fused launches do) than a few ulps: the path's headline bar on the largest
    error, and a bar on the root-mean-square error at about twice what the roundings account for (measured: 0.5 - 0.6 %)."""
    got64, want64 = got.detach().double().cpu(), want.detach().double().cpu()
    assert got64.shape == want64.shape and torch.isfinite(got64).all(), what
    assert max_rel(got64, want64) <= MAX_REL, f"{what}: max rel err {max_rel(got64, want64):.3e}"
    rms = float((got64 - want64).pow(2).mean().sqrt() / want64.pow(2).mean().sqrt())
    assert rms <= 1.2e-2, f"{what}: rms err {rms:.3e} of the rms value"


def _oracle(x, idx, wts, factors, dy, s, experts, wg, wu, wd):
    """Sort the routes, run the oracle's expert layer on the sorted rows, combine (the reference's order of the backward)."""
    tokens, top_k = idx.shape
    _, perm, inv = rref.plan(idx)
    offsets = torch.cumsum(rref.expert_counts(idx, experts).long(), 0).int()
    xs = rref.gather_forward(x, perm, top_k)
    d_o = (dy.float()[perm // top_k] * rref.bf16(wts).reshape(-1)[perm][:, None]).to(torch.bfloat16)
    want = ref.expert_layer(xs, torch.arange(experts), offsets, wg, wu, wd, *factors, s, d_o)
    out = rref.combine_forward(ref.bf16_round(want["out"]).to(torch.bfloat16), wts, inv)
    dx = rref.gather_backward(ref.bf16_round(want["dx"]).to(torch.bfloat16), inv, tokens, top_k)
    return out.double(), dx.double(), want


def test_separated_implementation_matches_the_fused_one_on_packed_weights(pkg, dev):
    """The reference's order (separate base and LoRA products, every intermediate a bf16 tensor, fast_moe_lora.py:685-770)
    against the fused launches: same mathematics, different roundings."""
    ml = pkg.fast_moe_lora
    gen = torch.Generator().manual_seed(77)
    tokens, top_k, experts, hidden, inter, r, s = 96, 2, 8, 256, 256, 16, 0.5
    qt = gb.Q4_K
    import numpy as np
    pg = np.stack([make_payload(1 + e, qt, inter, hidden) for e in range(experts)])
    pu = np.stack([make_payload(21 + e, qt, inter, hidden) for e in range(experts)])
    pd = np.stack([make_payload(41 + e, qt, hidden, inter) for e in range(experts)])
    Q = pkg.gguf.GGUFQuantizedTensor
    mk = lambda: ml.GGUFExperts(Q(torch.from_numpy(pg).to(dev), qt, (experts, inter, hidden)), Q(torch.from_numpy(pu).to(dev), qt, (experts, inter, hidden)),
                                Q(torch.from_numpy(pd).to(dev), qt, (experts, hidden, inter)))
    fused, separated = mk(), mk()
    separated.experts_implementation = ml.SEPARATED_EXPERTS_IMPLEMENTATION
    x, idx, wts, factors, dy = _layer_inputs(gen, tokens, top_k, experts, hidden, inter, r)
    out_f, dx_f, df_f = _run_layer(ml, fused, dev, x, idx, wts, factors, dy, s)
    out_s, dx_s, df_s = _run_layer(ml, separated, dev, x, idx, wts, factors, dy, s)
    # each against the oracle's layer
    want_out, want_dx, want = _oracle(x, idx, wts, factors, dy, s, experts, ref.weights_bf16(pg, qt), ref.weights_bf16(pu, qt), ref.weights_bf16(pd, qt))
    _assert_layer_close(out_s, want_out, "separated out")
    _assert_layer_close(dx_s, want_dx, "separated dX")
    for name, got, key in zip(("dA gate/up", "dB gate/up", "dA down", "dB down"), df_s, ("da_gu", "db_gu", "da_d", "db_d")):
        _assert_layer_close(got, want[key], f"separated {name}")
    # and the two orders against each other at the path's headline tolerance
    assert max_rel(out_s.double().cpu(), out_f.double().cpu()) <= MAX_REL and max_rel(dx_s.double().cpu(), dx_f.double().cpu()) <= MAX_REL
    for a, b in zip(df_s, df_f):
        assert max_rel(a.double().cpu(), b.double().cpu()) <= MAX_REL


def test_separated_implementation_takes_floating_point_expert_weights(pkg, dev):
    """Expert planes that are plain bf16 tensors go through decode-free gmm (fast_moe_lora.py:239-247); checked against the
    oracle's expert layer on the same bf16 weights."""
    ml = pkg.fast_moe_lora
    gen = torch.Generator().manual_seed(78)
    tokens, top_k, experts, hidden, inter, r, s = 80, 2, 6, 128, 192, 8, 0.25
    wg, wu = bf16_randn(gen, experts, inter, hidden, std=0.05), bf16_randn(gen, experts, inter, hidden, std=0.05)
    wd = bf16_randn(gen, experts, hidden, inter, std=0.05)
    module = ml.GGUFExperts(wg.to(dev), wu.to(dev), wd.to(dev))
    with pytest.raises(RuntimeError, match="packed expert weights"):
        module(torch.zeros(4, hidden, dtype=torch.bfloat16, device=dev), torch.zeros(4, 2, dtype=torch.int64, device=dev),
               torch.ones(4, 2, device=dev), None)
    module.experts_implementation = ml.SEPARATED_EXPERTS_IMPLEMENTATION
    x, idx, wts, factors, dy = _layer_inputs(gen, tokens, top_k, experts, hidden, inter, r)
    out, dx, dfs = _run_layer(ml, module, dev, x, idx, wts, factors, dy, s)
    # oracle: sort the routes, run the expert layer on the sorted rows, combine
    want_out, want_dx, want = _oracle(x, idx, wts, factors, dy, s, experts, wg.double(), wu.double(), wd.double())
    _assert_layer_close(out, want_out, "out")
    _assert_layer_close(dx, want_dx, "dX")
    for name, got, key in (("dA gate/up", dfs[0], "da_gu"), ("dB gate/up", dfs[1], "db_gu"), ("dA down", dfs[2], "da_d"), ("dB down", dfs[3], "db_d")):
        _assert_layer_close(got, want[key], name)
