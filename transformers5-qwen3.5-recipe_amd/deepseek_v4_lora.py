"""DeepSeek-V4 twin of the dense LoRA surface (deepseek_v4_lora.py:52-124, :165-175 of the reference): the packed LoRA linear
under DeepSeek's class name and the frozen eight-group output projection that runs as ``fixed_grouped_mmq``."""

from __future__ import annotations

import re
from types import MethodType
from typing import Any

import torch

from .fast_lora import FastGGUFLoraLinear, FastLoraLinear, GGUFLinear, fixed_grouped_mmq
from .gguf import GGUFQuantizedTensor

_ADAPTER_PARAMETER = re.compile(r"\.lora_[AB](?:_down)?\.")

# the one target pattern DeepSeek-V4 adapters use (deepseek_v4_lora.py:25-28): the seven ordinary projections and the expert
# modules, anywhere but under the attention compressor's indexer
DEEPSEEK_V4_TARGET_MODULES_PATTERN = (
    r"^(?!.*\.self_attn\.compressor\.indexer\.)(?:.*\.)?"
    r"(?:q_a_proj|q_b_proj|kv_proj|o_b_proj|gate_proj|up_proj|down_proj|experts)$"
)


class DeepseekV4LoraLinear(FastLoraLinear):
    """The float LoRA linear under DeepSeek's class name (deepseek_v4_lora.py:52-53)."""


class DeepseekV4GGUFLoraLinear(FastGGUFLoraLinear):
    """The packed LoRA linear for DeepSeek-V4's ordinary projections (deepseek_v4_lora.py:56-57)."""


class _RejectedDeepseekV4GroupedLora(DeepseekV4GGUFLoraLinear):
    """What a grouped output projection maps to: constructing it fails, so that a target pattern that reaches ``o_a_proj``
    stops the injection instead of training an adapter the grouped kernel does not carry (deepseek_v4_lora.py:60-65)."""

    def __init__(self, *args: Any, **kwargs: Any) -> None:
        del args, kwargs
        raise RuntimeError("DeepSeek V4 grouped o_a_proj LoRA is unsupported; keep GGUFGroupedLinear frozen.")


class GGUFGroupedLinear(torch.nn.Module):
    """Frozen grouped projection ``[..., n_groups, in_features] -> [..., n_groups, out_features / n_groups]`` whose packed
    weight is one flattened ``[out_features, row bytes]`` payload, group after group (stand-in for the fork's class; exposes
    what deepseek_v4_lora.py:91-124 reads)."""

    def __init__(self, in_features: int, out_features: int, n_groups: int, weight: GGUFQuantizedTensor, compute_dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        if out_features % n_groups:
            raise ValueError("out_features must be a whole number of groups")
        if tuple(weight.logical_shape) != (out_features, in_features):
            raise ValueError(f"weight logical shape {weight.logical_shape} != ({out_features}, {in_features})")
        self.in_features, self.out_features, self.n_groups = in_features, out_features, n_groups
        self.weight = weight
        self.compute_dtype = compute_dtype
        self.input_permutation = None
        self.output_permutation = None

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return _deepseek_v4_fixed_grouped_mmq_forward(self, input)


def _deepseek_v4_fixed_grouped_mmq_forward(self: GGUFGroupedLinear, input: torch.Tensor) -> torch.Tensor:
    """The reference's replacement forward for ``GGUFGroupedLinear`` (deepseek_v4_lora.py:91-124), with its guards and
    messages: the flattened payload is viewed as ``[n_groups, out_features / n_groups, bytes]`` and handed to the fixed
    grouped operator, so the group boundary survives and no logical matrix is materialised; the result comes back in the
    input's dtype."""
    if self.compute_dtype != torch.bfloat16:
        raise RuntimeError("DeepSeek fixed grouped MMQ requires BF16 compute_dtype.")
    if not (self.input_permutation is None and self.output_permutation is None):
        raise RuntimeError("DeepSeek fixed grouped MMQ does not support layout permutations.")
    rows_per_group = self.out_features // self.n_groups
    payload = self.weight.as_subclass(torch.Tensor)
    if payload.ndim != 2 or payload.shape[0] != self.n_groups * rows_per_group:
        raise RuntimeError("DeepSeek fixed grouped MMQ expects a flattened grouped payload with "
                           f"{self.n_groups * rows_per_group} rows, got {tuple(payload.shape)}.")
    x = input.to(torch.bfloat16)
    if x.storage_offset() or not x.is_contiguous():
        x = x.contiguous()
    block_format = int(getattr(self.weight, "quant_type", 8))
    y = fixed_grouped_mmq(x, payload.view(self.n_groups, rows_per_group, payload.shape[1]), block_format)
    return y if y.dtype == input.dtype else y.to(input.dtype)


def register_deepseek_v4_lora(lora_config):
    """Registers DeepSeek's linear wrappers on one config (deepseek_v4_lora.py:68-88); the config must use the exact target
    pattern above."""
    register = getattr(lora_config, "_register_custom_module", None)
    if register is None:
        raise RuntimeError("This PEFT version has no LoraConfig._register_custom_module API.")
    if lora_config.target_modules != DEEPSEEK_V4_TARGET_MODULES_PATTERN:
        raise ValueError("DeepSeek V4 target_modules must use the exact indexer-excluding pattern "
                         f"{DEEPSEEK_V4_TARGET_MODULES_PATTERN!r}.")
    register({GGUFGroupedLinear: _RejectedDeepseekV4GroupedLora, GGUFLinear: DeepseekV4GGUFLoraLinear, torch.nn.Linear: DeepseekV4LoraLinear})
    return lora_config


def configure_deepseek_v4_grouped_mmq(model: torch.nn.Module, *, require_checkpoint_geometry: bool = False) -> dict[str, Any]:
    """Installs the fixed grouped forward on every ``GGUFGroupedLinear`` of one model instance (deepseek_v4_lora.py:127-162);
    the modules stay frozen and unwrapped.  The kernel takes any group count, width and natively supported block format;
    ``require_checkpoint_geometry`` restores the reference's fail-closed check for the one geometry its checkpoint has
    (Q8_0, 8 groups, 4096 -> 1024 per group).  Returns {"enabled": count, "paths": sorted paths}."""
    get_base_model = getattr(model, "get_base_model", None)
    base = get_base_model() if callable(get_base_model) else model
    paths: list[str] = []
    for name, module in base.named_modules():
        if not isinstance(module, GGUFGroupedLinear):
            continue
        if not isinstance(module.weight, GGUFQuantizedTensor):
            raise TypeError(f"DeepSeek grouped projection {name!r} is not GGUF-quantized.")
        if require_checkpoint_geometry and not (int(module.weight.quant_type) == 8 and module.n_groups == 8 and module.in_features == 4096
                                                and module.out_features == 8 * 1024):
            raise RuntimeError(f"DeepSeek grouped projection does not match the fixed eight-group Q8_0 4096->1024 contract: {name!r}.")
        if not getattr(module, "_deepseek_v4_grouped_mmq_enabled", False):
            module.forward = MethodType(_deepseek_v4_fixed_grouped_mmq_forward, module)
            module._deepseek_v4_grouped_mmq_enabled = True
        paths.append(name)
    return {"enabled": len(paths), "paths": sorted(paths)}


def normalize_peft_path(path: str) -> str:
    """The pre-PEFT model path of a module or parameter (the mapping of deepseek_v4_lora.py:165-175): wrapper prefixes are
    dropped one after the other, and a path that then starts at ``layers.`` gets its ``model.`` back."""
    for wrapper_prefix in ("base_model.model.", "model."):
        if path.startswith(wrapper_prefix):
            path = path[len(wrapper_prefix):]
    if path.startswith("layers."):
        path = "model." + path
    return path


def is_adapter_parameter(name: str) -> bool:
    """Whether a parameter name belongs to a LoRA factor (the pattern of deepseek_v4_lora.py:49)."""
    return _ADAPTER_PARAMETER.search(name) is not None
