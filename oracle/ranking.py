"""CPU oracle for the router's expert selection.

TEST INFRASTRUCTURE (see oracle/__init__.py).  Restates fast_moe_ranking.py:

* ``router_topk`` (``router_topk_indices``, :197-271): the Triton kernel (:163-194) orders the experts of a
  token by the packed key ``float_key(score) << 16 | (256 - expert)`` (:71-80, :131-134) and keeps the top_k
  largest, best first (:160).  ``float_key`` maps the IEEE bits of a score to unsigned integers ordered like
  the values (negative: all bits flipped, otherwise the top bit set), so -0.0 sorts below +0.0 and equal
  scores go to the smaller expert index.  bf16 scores compare as the fp32 values they are (the map is
  monotone under that widening).  Score functions: the logit itself, or sqrt(softplus(logit)) in fp32 plus
  an optional per-expert bias (:88-102);
* ``qwen_router_weights`` (:273-284): softmax over the selected logits in fp32, cast to the logits' type;
* ``deepseek_router_weights`` (:287-303): sqrt(softplus(selected logits)) / (sum + 1e-20) * scaling.

Pinned in tests/test_oracle_ranking.py: a brute-force loop (repeatedly take the maximum, first index on
ties) on inputs full of ties, ``torch.topk`` values on distinct scores, the all-zero tie case of the
reference's own test (test_fast_moe_ranking.py:183-201: experts 0..k-1), and the -0.0 / +0.0 order of the
key.  **parity unpinned**: the rounding of sqrt(softplus()) — the reference evaluates it with Triton's exp
and log, this file with numpy's, the device kernel with HIP's; the three agree to an ulp or two, so
selections can differ where two scores are that close.  The tie rule itself is pinned.
"""

from __future__ import annotations

import numpy as np
import torch


def float_key(scores_f32: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(scores_f32, dtype=np.float32).view(np.uint32)
    return bits ^ np.where(bits & np.uint32(0x80000000), np.uint32(0xFFFFFFFF), np.uint32(0x80000000)).astype(np.uint32)


def sqrt_softplus(x: np.ndarray) -> np.ndarray:
    x = x.astype(np.float32)
    return np.sqrt(np.maximum(x, np.float32(0)) + np.log(np.float32(1) + np.exp(-np.abs(x)))).astype(np.float32)


def router_scores(logits: torch.Tensor, correction_bias: torch.Tensor | None = None, score_function: str = "identity") -> np.ndarray:
    x = logits.detach().to(torch.float32).cpu().numpy()
    if score_function == "identity":
        if correction_bias is not None:
            raise ValueError("Router correction bias is supported only with sqrt-softplus scoring.")
        return x
    if score_function != "sqrtsoftplus":
        raise ValueError(f"Unsupported router score function: {score_function!r}.")
    s = sqrt_softplus(x)
    if correction_bias is not None:
        s = (s + correction_bias.detach().to(torch.float32).cpu().numpy()[None, :]).astype(np.float32)
    return s


def router_topk(logits: torch.Tensor, top_k: int, correction_bias: torch.Tensor | None = None, score_function: str = "identity") -> torch.Tensor:
    scores = router_scores(logits, correction_bias, score_function)
    experts = scores.shape[1]
    packed = (float_key(scores).astype(np.uint64) << np.uint64(16)) | (np.uint64(256) - np.arange(experts, dtype=np.uint64))[None, :]
    order = np.argsort(packed, axis=1)[:, ::-1][:, :top_k]  # keys are distinct: any sort gives the same order
    return torch.from_numpy(np.ascontiguousarray(order).astype(np.int64))


def qwen_router_weights(logits: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    selected = logits.gather(1, indices)
    return torch.softmax(selected, dtype=torch.float32, dim=-1).to(logits.dtype)


def deepseek_router_weights(logits: torch.Tensor, indices: torch.Tensor, scaling: float) -> torch.Tensor:
    s = torch.from_numpy(sqrt_softplus(logits.float().gather(1, indices).numpy()))
    return s / (s.sum(dim=-1, keepdim=True) + 1e-20) * scaling
