"""Router expert selection for the MoE layers.

Host-side mirror of the reference's ``fast_moe_ranking.py``: ``router_topk_indices`` returns, per token, the
top-k experts of the router scores, best first, equal scores in ascending expert index (fast_moe_ranking.py:197-271;
the order is that of its packed keys, :71-80 and :119-160), and the two router forwards compute the routing weights
the way the reference's patched modules do (:273-303).  Selection and weights run in one device kernel
(``ggq_router_topk``); the router logits themselves are a plain ``torch.nn.functional.linear``.  Unlike the
reference (``_is_supported_router_geometry``) any expert count that is a multiple of 4 up to 256, any top-k up to 8
and any number of tokens is accepted.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from . import _lib

_SCORE_FUNCTIONS = {"identity": 0, "sqrtsoftplus": 1}


def _select(logits: torch.Tensor, top_k: int, correction_bias, score_function: str, weights_mode: int, scaling: float):
    if logits.ndim != 2:
        raise ValueError(f"Router logits must be [tokens,experts], got {logits.shape}.")
    if score_function not in _SCORE_FUNCTIONS:
        raise ValueError(f"Unsupported router score function: {score_function!r}.")
    num_tokens, num_experts = logits.shape
    if num_experts > 256 or num_experts % 4 or not 0 < top_k <= min(8, num_experts):
        raise RuntimeError("Router selection supports up to 256 experts (a multiple of 4) and top-k up to 8.")
    if logits.device.type != "cuda" or logits.dtype not in {torch.bfloat16, torch.float32}:
        raise RuntimeError("Optimized router selection requires CUDA/ROCm BF16 or FP32 logits.")
    if correction_bias is not None:
        if score_function != "sqrtsoftplus":
            raise ValueError("Router correction bias is supported only with sqrt-softplus scoring.")
        if correction_bias.shape != (num_experts,):
            raise ValueError(f"Router correction bias must have shape {(num_experts,)}, got {correction_bias.shape}.")
        if correction_bias.device != logits.device:
            raise ValueError("Router correction bias must be on the logits device.")
        correction_bias = correction_bias.to(torch.float32).contiguous()
    logits = logits.contiguous()
    indices = torch.empty((num_tokens, top_k), dtype=torch.long, device=logits.device)
    weights = None
    if weights_mode == 1:
        weights = torch.empty((num_tokens, top_k), dtype=logits.dtype, device=logits.device)
    elif weights_mode == 2:
        weights = torch.empty((num_tokens, top_k), dtype=torch.float32, device=logits.device)
    lib = _lib.load()
    _lib.check(lib.ggq_router_topk(logits.data_ptr(), int(logits.dtype == torch.bfloat16), num_tokens, num_experts, top_k,
                                   correction_bias.data_ptr() if correction_bias is not None else None,
                                   _SCORE_FUNCTIONS[score_function], indices.data_ptr(),
                                   weights.data_ptr() if weights is not None else None, weights_mode, float(scaling),
                                   _lib.stream_handle(logits.device)))
    return indices, weights


def router_topk_indices(logits: torch.Tensor, top_k: int, *, correction_bias: torch.Tensor | None = None,
                        score_function: str = "identity") -> torch.Tensor:
    """[tokens, experts] logits -> [tokens, top_k] int64 expert ids, best first; ties go to the smaller expert
    index (fast_moe_ranking.py:197-271)."""
    return _select(logits, top_k, correction_bias, score_function, 0, 1.0)[0]


def qwen_router_forward(weight: torch.Tensor, hidden_states: torch.Tensor, top_k: int):
    """(router_logits, router_scores, router_indices) as ``_qwen_router_forward`` returns them
    (fast_moe_ranking.py:273-284): scores = softmax over the selected logits in fp32, in the logits' type."""
    flat = hidden_states.reshape(-1, weight.shape[1])
    router_logits = F.linear(flat, weight)
    indices, scores = _select(router_logits, top_k, None, "identity", 1, 1.0)
    return router_logits, scores, indices


def deepseek_topk_router_forward(weight: torch.Tensor, e_score_correction_bias: torch.Tensor | None, hidden_states: torch.Tensor,
                                 top_k: int, routed_scaling_factor: float):
    """(logits, weights, indices) as ``_deepseek_topk_router_forward`` returns them (fast_moe_ranking.py:287-303):
    fp32 logits, selection on sqrt(softplus) + bias, weights = unbiased scores normalised, times the scaling."""
    flat = hidden_states.reshape(-1, weight.shape[1])
    logits = F.linear(flat.float(), weight.float())
    indices, weights = _select(logits, top_k, e_score_correction_bias, "sqrtsoftplus", 2, routed_scaling_factor)
    return logits, weights, indices
