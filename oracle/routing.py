"""CPU oracle for the expert-sorted routing layout.

TEST INFRASTRUCTURE (see oracle/__init__.py).  Restates fast_moe_routing.py:

* plan (``prepare_expert_routing``, :379-428): sort the flat top-k expert ids, keep the sorted ids,
  the permutation (sorted position -> original route, route = token*k + rank) and its inverse
  (:88-98).  The reference calls ``torch.sort`` without ``stable=True``; its own test compares with
  the same call (test_fast_moe_routing.py:55-67).  The contract fixed here is the *stable* order
  (ties keep ascending route index), which is what a counting sort produces;
* gather forward (:101-123): selected[s] = hidden[perm[s] // k];
* gather backward (:126-159): per token, add its k routed rows in ascending sorted position,
  rounding the running sum to bf16 after every add;
* combine forward (:162-194): fp32 sum over rank of o[inv[t*k+rank]] * fp32(bf16(w[t,rank])), one
  rounding to bf16 at the store;
* combine backward (:197-226): dO[s] = bf16(g[t] * fp32(bf16(w))), dW[t,rank] = sum_h g*o in fp32;
* grouped offsets (fast_moe_lora.py:652-672 and the compact form of test_fast_moe_lora.py:136-138):
  active expert ids and cumulative END offsets.

Pinned by closed forms in tests/test_oracle_routing.py: inv[perm] = arange, sortedness, gather ==
hidden[perm // k], torch autograd of index_select for the unrounded sums, brute-force loops on tiny
inputs for the rounding order.
"""

from __future__ import annotations

import numpy as np
import torch


def bf16(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.float32).to(torch.bfloat16).to(torch.float32)


def plan(top_k_index: torch.Tensor):
    """[T,k] integer -> (sorted expert ids [R] int64, permutation [R] int64, inverse [R] int64)."""
    flat = top_k_index.reshape(-1).to(torch.int64)
    sorted_ids, perm = torch.sort(flat, stable=True)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(perm.numel(), dtype=torch.int64)
    return sorted_ids, perm, inv


def expert_counts(top_k_index: torch.Tensor, num_experts: int) -> torch.Tensor:
    return torch.bincount(top_k_index.reshape(-1).to(torch.int64), minlength=num_experts).to(torch.int32)


def active_offsets(counts: torch.Tensor):
    """counts [E] -> (active expert ids int64 [A], cumulative end offsets int32 [A])."""
    active = torch.nonzero(counts > 0).reshape(-1).to(torch.int64)
    return active, torch.cumsum(counts[active].to(torch.int64), 0).to(torch.int32)


def gather_forward(hidden: torch.Tensor, perm: torch.Tensor, k: int) -> torch.Tensor:
    return hidden[perm // k]


def gather_backward(grad_selected: torch.Tensor, inv: torch.Tensor, num_tokens: int, k: int) -> torch.Tensor:
    """bf16 [R,H] -> bf16 [T,H] with the reference's add order and per-add rounding."""
    pos = inv.reshape(num_tokens, k).sort(dim=1).values            # ascending sorted positions
    acc = torch.zeros(num_tokens, grad_selected.shape[1], dtype=torch.float32)
    g32 = grad_selected.to(torch.float32)
    for j in range(k):
        acc = bf16(acc + g32[pos[:, j]])
    return acc.to(torch.bfloat16)


def combine_forward(expert_out: torch.Tensor, weights: torch.Tensor, inv: torch.Tensor) -> torch.Tensor:
    """expert_out bf16 [R,H], weights [T,k] (bf16 or fp32) -> bf16 [T,H]."""
    t, k = weights.shape
    w = bf16(weights)
    acc = torch.zeros(t, expert_out.shape[1], dtype=torch.float32)
    o32 = expert_out.to(torch.float32)
    for rank in range(k):
        acc = acc + o32[inv.reshape(t, k)[:, rank]] * w[:, rank:rank + 1]
    return acc.to(torch.bfloat16)


def combine_backward(grad_out: torch.Tensor, expert_out: torch.Tensor, weights: torch.Tensor, perm: torch.Tensor):
    """-> (dO bf16 [R,H], dW [T,k] in float64 (the fp32 reduction order is unspecified))."""
    t, k = weights.shape
    tok = perm // k
    w = bf16(weights).reshape(-1)[perm]                             # weight of each sorted route
    g32 = grad_out.to(torch.float32)[tok]
    d_o = (g32 * w[:, None]).to(torch.bfloat16)
    dw_sorted = (g32.to(torch.float64) * expert_out.to(torch.float64)).sum(dim=1)
    dw = torch.empty(t * k, dtype=torch.float64)
    dw[perm] = dw_sorted
    return d_o, dw.reshape(t, k)


def router_topk(logits: torch.Tensor, k: int):
    """Top-k on raw logits with smaller-index tie-break, softmax over the k selected logits in fp32
    (fast_moe_ranking.py:208-211, 273-284).  -> (ids int64 [T,k] by descending logit, weights fp32)."""
    order = torch.argsort(-logits.to(torch.float32), dim=1, stable=True)[:, :k]
    picked = torch.gather(logits.to(torch.float32), 1, order)
    return order, torch.softmax(picked, dim=1)
