"""Router expert selection on the device against oracle/ranking.py: indices bit-exact for identity scoring
(ties to the smaller expert index, test_fast_moe_ranking.py:183-201), selections equivalent up to the kth
score for sqrt-softplus scoring (the reference's own acceptance rule, fast_moe_ranking.py:205-208), routing
weights within bf16 / fp32 rounding."""

import numpy as np
import pytest
import torch

from oracle import ranking as ref

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tokens,experts,top_k,dtype", [(4096, 256, 8, torch.bfloat16), (333, 256, 6, torch.float32), (5, 64, 8, torch.float32),
                                                         (1, 256, 1, torch.bfloat16), (32768, 256, 8, torch.bfloat16)])
def test_identity_selection_is_bit_exact(pkg, dev, tokens, experts, top_k, dtype):
    gen = torch.Generator().manual_seed(19260817 + tokens)
    logits = torch.randn(tokens, experts, generator=gen).to(dtype)  # bf16 logits of 256 experts tie often
    got = pkg.fast_moe_ranking.router_topk_indices(logits.to(dev), top_k)
    assert got.dtype == torch.int64 and got.shape == (tokens, top_k)
    assert torch.equal(got.cpu(), ref.router_topk(logits, top_k))


def test_ties_zeros_and_signed_zeros(pkg, dev):
    rk = pkg.fast_moe_ranking
    for dtype in (torch.float32, torch.bfloat16):
        got = rk.router_topk_indices(torch.zeros(7, 256, dtype=dtype, device=dev), 8)
        assert torch.equal(got.cpu(), torch.arange(8).expand(7, 8))
    gen = torch.Generator().manual_seed(5)
    few = torch.randint(-2, 3, (500, 256), generator=gen).to(torch.float32)
    assert torch.equal(rk.router_topk_indices(few.to(dev), 8).cpu(), ref.router_topk(few, 8))
    z = torch.tensor([[0.0, -0.0, 0.0, -0.0] * 64])
    assert torch.equal(rk.router_topk_indices(z.to(dev), 8).cpu(), ref.router_topk(z, 8))


def test_sqrt_softplus_selection_with_bias(pkg, dev):
    gen = torch.Generator().manual_seed(77)
    logits = torch.randn(2048, 256, generator=gen) * 3
    bias = torch.randn(256, generator=gen) * 0.05
    got = pkg.fast_moe_ranking.router_topk_indices(logits.to(dev), 6, correction_bias=bias.to(dev), score_function="sqrtsoftplus").cpu()
    want = ref.router_topk(logits, 6, bias, "sqrtsoftplus")
    scores = torch.from_numpy(ref.router_scores(logits, bias, "sqrtsoftplus"))
    # the two evaluations of exp / log / sqrt differ by an ulp or two: wherever the order differs the scores involved
    # must be that close, and every row must still hold six distinct experts
    same = (got == want).all(dim=1)
    assert same.float().mean() > 0.99
    gs, ws = scores.gather(1, got), scores.gather(1, want)
    assert torch.allclose(gs, ws, rtol=0, atol=4e-6)
    assert all(len(set(r.tolist())) == 6 for r in got[~same])


def test_router_forwards(pkg, dev):
    rk = pkg.fast_moe_ranking
    gen = torch.Generator().manual_seed(3)
    weight = (torch.randn(256, 512, generator=gen) * 0.05).to(torch.bfloat16)
    hidden = torch.randn(3, 100, 512, generator=gen).to(torch.bfloat16)
    logits, scores, indices = rk.qwen_router_forward(weight.to(dev), hidden.to(dev), 8)
    assert logits.shape == (300, 256) and scores.dtype == torch.bfloat16
    lc = logits.cpu()
    assert torch.equal(indices.cpu(), ref.router_topk(lc, 8))
    want = ref.qwen_router_weights(lc, indices.cpu())
    assert torch.allclose(scores.cpu().float(), want.float(), rtol=0, atol=2 ** -8)
    bias = torch.randn(256, generator=gen) * 0.05
    l2, w2, i2 = rk.deepseek_topk_router_forward(weight.to(dev), bias.to(dev), hidden.to(dev), 6, 2.5)
    assert l2.dtype == torch.float32 and w2.dtype == torch.float32
    want2 = ref.deepseek_router_weights(l2.cpu(), i2.cpu(), 2.5)
    assert torch.allclose(w2.cpu(), want2, rtol=1e-5, atol=1e-6)
    assert torch.allclose(w2.sum(-1).cpu(), torch.full((300,), 2.5), atol=1e-4)


def test_router_guards(pkg, dev):
    rk = pkg.fast_moe_ranking
    x = torch.zeros(4, 256, device=dev)
    with pytest.raises(ValueError):
        rk.router_topk_indices(x[0], 8)
    with pytest.raises(ValueError):
        rk.router_topk_indices(x, 8, score_function="softmax")
    with pytest.raises(ValueError):
        rk.router_topk_indices(x, 8, correction_bias=torch.zeros(256, device=dev))
    with pytest.raises(RuntimeError):
        rk.router_topk_indices(x, 9)
    with pytest.raises(RuntimeError):
        rk.router_topk_indices(x.to(torch.float16), 8)
    with pytest.raises(RuntimeError):
        rk.router_topk_indices(torch.zeros(4, 256), 8)
