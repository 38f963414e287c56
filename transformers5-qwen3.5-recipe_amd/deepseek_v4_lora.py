"""DeepSeek-V4 twin of the dense LoRA surface (deepseek_v4_lora.py:52-124, :165-175 of the reference): the packed LoRA linear
under DeepSeek's class name and the frozen eight-group output projection that runs as ``fixed_grouped_mmq``."""

from __future__ import annotations

import re

import torch

from .fast_lora import FastGGUFLoraLinear, fixed_grouped_mmq
from .gguf import GGUFQuantizedTensor

_ADAPTER_PARAMETER = re.compile(r"\.lora_[AB](?:_down)?\.")


class DeepseekV4GGUFLoraLinear(FastGGUFLoraLinear):
    """The packed LoRA linear for DeepSeek-V4's ordinary projections (deepseek_v4_lora.py:56-57)."""


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
