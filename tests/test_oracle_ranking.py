"""Pins oracle/ranking.py (router expert selection) without the reference: brute force, torch.topk, the
reference test's all-zero tie case (test_fast_moe_ranking.py:183-201) and the key order of signed zeros."""

import numpy as np
import torch

from oracle import ranking


def _brute_force(scores: np.ndarray, top_k: int) -> np.ndarray:
    out = np.zeros((scores.shape[0], top_k), dtype=np.int64)
    for t in range(scores.shape[0]):
        taken = set()
        for r in range(top_k):
            best = None
            for e in range(scores.shape[1]):
                if e in taken:
                    continue
                if best is None or scores[t, e] > scores[t, best]:  # strict: the first index wins a tie
                    best = e
            taken.add(best)
            out[t, r] = best
    return out


def test_ties_go_to_the_smaller_expert_index():
    gen = torch.Generator().manual_seed(20260101)
    logits = torch.randint(-3, 4, (40, 64), generator=gen).to(torch.float32)  # seven distinct values: ties everywhere
    got = ranking.router_topk(logits, 8).numpy()
    assert np.array_equal(got, _brute_force(logits.numpy(), 8))
    assert np.array_equal(ranking.router_topk(logits.to(torch.bfloat16), 6).numpy(), _brute_force(logits.numpy(), 6))


def test_all_zero_logits_select_the_first_experts():
    for dtype in (torch.float32, torch.bfloat16):
        got = ranking.router_topk(torch.zeros(5, 256, dtype=dtype), 8)
        assert torch.equal(got, torch.arange(8).expand(5, 8))


def test_distinct_scores_match_torch_topk():
    gen = torch.Generator().manual_seed(7)
    logits = torch.randn(64, 256, generator=gen)
    want = torch.topk(logits, 8, dim=-1)
    got = ranking.router_topk(logits, 8)
    assert torch.equal(got, want.indices)
    bias = torch.randn(256, generator=gen) * 0.1
    scores = torch.from_numpy(ranking.router_scores(logits, bias, "sqrtsoftplus"))
    got = ranking.router_topk(logits, 6, bias, "sqrtsoftplus")
    assert torch.equal(scores.gather(1, got), torch.topk(scores, 6, dim=-1).values)
    ref = torch.sqrt(torch.nn.functional.softplus(logits.double())) + bias.double()
    assert torch.allclose(scores.double(), ref, rtol=0, atol=2e-6)


def test_key_orders_signed_zeros_and_is_monotone():
    v = np.array([-np.inf, -2.5, -1e-30, -0.0, 0.0, 1e-30, 3.0, np.inf], dtype=np.float32)
    k = ranking.float_key(v)
    assert np.all(k[1:] > k[:-1])
    logits = torch.tensor([[0.0, -0.0, 0.0, -0.0]])
    assert ranking.router_topk(logits, 4).tolist() == [[0, 2, 1, 3]]


def test_weights():
    gen = torch.Generator().manual_seed(11)
    logits = torch.randn(16, 256, generator=gen).to(torch.bfloat16)
    idx = ranking.router_topk(logits, 8)
    w = ranking.qwen_router_weights(logits, idx)
    assert w.dtype == torch.bfloat16 and torch.allclose(w.float().sum(-1), torch.ones(16), atol=2e-2)
    lf = logits.float()
    idx6 = ranking.router_topk(lf, 6, None, "sqrtsoftplus")
    w6 = ranking.deepseek_router_weights(lf, idx6, 2.5)
    assert torch.allclose(w6.sum(-1), torch.full((16,), 2.5), atol=1e-5)
