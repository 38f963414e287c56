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
    (fast_moe_ranking.py:273-284): scores = softmax over the selected logits in fp32, in the logits' type.  Selection and
    scores come from one kernel when nothing differentiates through the logits; under autograd the scores are recomputed
    from the selected logits with framework operators, as the reference does, so that the gradient reaches the router's
    input (and its weight, when that trains)."""
    flat = hidden_states.reshape(-1, weight.shape[1])
    router_logits = F.linear(flat, weight)
    if router_logits.requires_grad and torch.is_grad_enabled():
        indices = _select(router_logits.detach(), top_k, None, "identity", 0, 1.0)[0]
        scores = torch.softmax(router_logits.gather(1, indices), dtype=torch.float32, dim=-1).to(router_logits.dtype)
        return router_logits, scores, indices
    indices, scores = _select(router_logits, top_k, None, "identity", 1, 1.0)
    return router_logits, scores, indices


def _sqrt_softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.sqrt(F.softplus(x))


def deepseek_topk_router_forward(weight: torch.Tensor, e_score_correction_bias: torch.Tensor | None, hidden_states: torch.Tensor,
                                 top_k: int, routed_scaling_factor: float):
    """(logits, weights, indices) as ``_deepseek_topk_router_forward`` returns them (fast_moe_ranking.py:287-303):
    fp32 logits, selection on sqrt(softplus) + bias, weights = unbiased scores normalised, times the scaling; under autograd
    the weights are recomputed from the selected logits with framework operators, like the Qwen router's."""
    flat = hidden_states.reshape(-1, weight.shape[1])
    logits = F.linear(flat.float(), weight.float())
    if logits.requires_grad and torch.is_grad_enabled():
        indices = _select(logits.detach(), top_k, e_score_correction_bias, "sqrtsoftplus", 0, 1.0)[0]
        scores = _sqrt_softplus(logits.gather(1, indices))
        return logits, scores / (scores.sum(dim=-1, keepdim=True) + 1e-20) * routed_scaling_factor, indices
    indices, weights = _select(logits, top_k, e_score_correction_bias, "sqrtsoftplus", 2, routed_scaling_factor)
    return logits, weights, indices


# ------------------------------------------------------------------------------------------------
# Model-level installation (fast_moe_ranking.py:273-380 of the reference): replacement forwards for the router modules of
# transformers' Qwen3.5-MoE and DeepSeek-V4 models, bound per module instance.
def _qwen_router_forward(self, hidden_states: torch.Tensor):
    """Replacement for ``Qwen3_5MoeTopKRouter.forward`` (fast_moe_ranking.py:273-284): logits, softmax over the selected
    logits (equal to the stock module's softmax over all experts renormalised over the selection), indices best first."""
    return qwen_router_forward(self.weight, hidden_states, self.top_k)


def _deepseek_topk_router_forward(self, hidden_states: torch.Tensor):
    """Replacement for ``DeepseekV4TopKRouter.forward`` (fast_moe_ranking.py:287-302)."""
    return deepseek_topk_router_forward(self.weight, self.e_score_correction_bias, hidden_states, self.top_k, float(self.routed_scaling_factor))


def _deepseek_hash_router_forward(self, hidden_states: torch.Tensor, input_ids: torch.Tensor):
    """Replacement for ``DeepseekV4HashRouter.forward`` (fast_moe_ranking.py:305-316): the experts come from the frozen
    token-id table, so there is nothing to select; framework operators, fp32 logits as in the reference."""
    flat = hidden_states.reshape(-1, self.hidden_dim)
    logits = F.linear(flat.float(), self.weight.float())
    indices = self.tid2eid[input_ids.reshape(-1)].long()
    scores = self.score_fn(logits.gather(1, indices))
    weights = scores / (scores.sum(dim=-1, keepdim=True) + 1e-20)
    return logits, weights * self.routed_scaling_factor, indices


def _is_a(module: torch.nn.Module, class_name: str) -> bool:
    return any(c.__name__ == class_name for c in type(module).__mro__)


def _selectable(module) -> bool:
    return module.num_experts <= 256 and module.num_experts % 4 == 0 and 0 < module.top_k <= min(8, module.num_experts)


def configure_fast_moe_ranking(model: torch.nn.Module, *, require_checkpoint_geometry: bool = False) -> dict:
    """Installs the device router selection on every router module of one model (fast_moe_ranking.py:319-380).  Router
    modules are recognised by class name (``Qwen3_5MoeTopKRouter``, ``DeepseekV4TopKRouter``, ``DeepseekV4HashRouter``
    anywhere in the MRO), a PEFT wrapper is unwrapped through ``get_base_model``.  The selection kernel takes up to 256
    experts (a multiple of 4) and top-k up to 8, and a module outside that fails the call; DeepSeek routers must score with
    sqrt-softplus.  ``require_checkpoint_geometry`` adds the reference's fail-closed checks for the two checkpoints it serves
    (Qwen 2048 / 256 / top-8 with 40 routers; DeepSeek 4096 / 256 / top-6 with 40 learned and 3 hash routers).
    Returns {"qwen": n, "deepseek_topk": n, "deepseek_hash": n, "paths": {...}}."""
    from types import MethodType

    get_base_model = getattr(model, "get_base_model", None)
    base = get_base_model() if callable(get_base_model) else model
    config = getattr(base, "config", None)
    model_type, scoring_func = getattr(config, "model_type", None), getattr(config, "scoring_func", None)
    paths: dict[str, list[str]] = {"qwen": [], "deepseek_topk": [], "deepseek_hash": []}
    for name, module in base.named_modules():
        if _is_a(module, "Qwen3_5MoeTopKRouter"):
            if not _selectable(module) or (require_checkpoint_geometry and (module.hidden_dim, module.num_experts, module.top_k) != (2048, 256, 8)):
                raise RuntimeError(f"Qwen router {name!r} does not match 2048/256/top-8." if require_checkpoint_geometry else
                                   f"Qwen router {name!r}: the selection kernel takes up to 256 experts (a multiple of 4) and top-k up to 8.")
            module.forward = MethodType(_qwen_router_forward, module)
            paths["qwen"].append(name)
        elif _is_a(module, "DeepseekV4TopKRouter") or _is_a(module, "DeepseekV4HashRouter"):
            hashed = _is_a(module, "DeepseekV4HashRouter")
            what = "DeepSeek hash router" if hashed else "DeepSeek router"
            if scoring_func != "sqrtsoftplus" or (not hashed and not _selectable(module)) or (
                    require_checkpoint_geometry and (module.hidden_dim, module.num_experts, module.top_k) != (4096, 256, 6)):
                raise RuntimeError(f"{what} {name!r} does not match 4096/256/top-6 sqrtsoftplus." if require_checkpoint_geometry else
                                   f"{what} {name!r} needs sqrtsoftplus scoring, up to 256 experts (a multiple of 4) and top-k up to 8.")
            module.forward = MethodType(_deepseek_hash_router_forward if hashed else _deepseek_topk_router_forward, module)
            paths["deepseek_hash" if hashed else "deepseek_topk"].append(name)
    if require_checkpoint_geometry:
        if model_type in {"qwen3_5_moe", "qwen3_5_moe_text"} and len(paths["qwen"]) != 40:
            raise RuntimeError(f"expected 40 Qwen routers, found {len(paths['qwen'])}")
        if model_type == "deepseek_v4" and (len(paths["deepseek_topk"]) != 40 or len(paths["deepseek_hash"]) != 3):
            raise RuntimeError(f"expected 40 learned and 3 hash DeepSeek routers, found {len(paths['deepseek_topk'])} and {len(paths['deepseek_hash'])}")
    return {"qwen": len(paths["qwen"]), "deepseek_topk": len(paths["deepseek_topk"]), "deepseek_hash": len(paths["deepseek_hash"]),
            "paths": {key: sorted(value) for key, value in paths.items()}}
