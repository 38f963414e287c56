"""DeepSeek-V4 twin of the expert LoRA surface (deepseek_v4_moe_lora.py:17-63 of the reference): the same packed expert
execution as ``fast_moe_lora`` behind DeepSeek's class names, with the clamped SwiGLU of its experts."""

from __future__ import annotations

from typing import Any

import torch

from .deepseek_v4_lora import DEEPSEEK_V4_TARGET_MODULES_PATTERN
from .fast_moe_lora import (ALL_GGUF_EXPERTS_FUNCTIONS, FastGGUFMoeLora, GGUFExperts, _ExpertLoraWeights, _register_expert_wrapper,
                            qwen3_5_moe_gguf_mmq_lora_forward)

EXPERTS_IMPLEMENTATION = "deepseek_v4_gguf_dequant_aiter_lora"


class DeepseekV4GGUFExperts(GGUFExperts):
    """Packed DeepSeek-V4 experts (stand-in for the fork's class of that name): split gate / up / down payloads and the
    model's ``swiglu_limit`` (the activation clamps gate to at most the limit and up to [-limit, limit])."""

    experts_implementation = EXPERTS_IMPLEMENTATION

    def __init__(self, gate_proj, up_proj, down_proj, swiglu_limit: float, compute_dtype: torch.dtype = torch.bfloat16):
        if not swiglu_limit or swiglu_limit <= 0:
            raise ValueError("DeepSeek V4 experts need a positive swiglu_limit.")
        super().__init__(gate_proj, up_proj, down_proj, compute_dtype=compute_dtype, swiglu_limit=float(swiglu_limit))


def deepseek_v4_gguf_dequant_aiter_lora_forward(self: Any, hidden_states: torch.Tensor, top_k_index: torch.Tensor, top_k_weights: torch.Tensor,
                                                _deepseek_v4_gguf_lora_weights: _ExpertLoraWeights | None = None) -> torch.Tensor:
    """The experts-implementation entry of the reference (deepseek_v4_moe_lora.py:44-63): type guard, then the shared
    packed expert forward."""
    if not isinstance(self, DeepseekV4GGUFExperts):
        raise TypeError(f"{EXPERTS_IMPLEMENTATION} requires DeepseekV4GGUFExperts, got {type(self).__name__}.")
    return qwen3_5_moe_gguf_mmq_lora_forward(self, hidden_states, top_k_index, top_k_weights, _deepseek_v4_gguf_lora_weights)


ALL_GGUF_EXPERTS_FUNCTIONS[EXPERTS_IMPLEMENTATION] = deepseek_v4_gguf_dequant_aiter_lora_forward


def register_deepseek_v4_moe_lora(lora_config, model: torch.nn.Module):
    """Registers DeepSeek's expert forward and its config-local wrapper (deepseek_v4_moe_lora.py:66-95): a string
    ``target_modules`` must be the exact DeepSeek pattern (which already names "experts"), a collection gets "experts" added."""
    return _register_expert_wrapper(lora_config, model, EXPERTS_IMPLEMENTATION, deepseek_v4_gguf_dequant_aiter_lora_forward, DeepseekV4GGUFExperts,
                                    DeepseekV4GGUFMoeLora, "DeepSeek V4 GGUF MoE LoRA", exact_pattern=DEEPSEEK_V4_TARGET_MODULES_PATTERN)


class DeepseekV4GGUFMoeLora(FastGGUFMoeLora):
    """LoRA wrapper for all gate, up and down transforms of one DeepSeek-V4 MoE layer (deepseek_v4_moe_lora.py:21-41)."""

    def forward(self, hidden_states: torch.Tensor, top_k_index: torch.Tensor, top_k_weights: torch.Tensor) -> torch.Tensor:
        experts = self.base_layer
        if not isinstance(experts, DeepseekV4GGUFExperts):
            raise TypeError(f"DeepSeek V4 expert LoRA requires DeepseekV4GGUFExperts, got {type(experts).__name__}.")
        return deepseek_v4_gguf_dequant_aiter_lora_forward(experts, hidden_states, top_k_index, top_k_weights, self._active_lora_weights())
