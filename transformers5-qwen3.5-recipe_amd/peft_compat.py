"""What the registration functions need from PEFT, for processes that do not have it.

The reference installs its wrappers through PEFT: a ``LoraConfig`` takes a mapping {base module class: wrapper class}
(``LoraConfig._register_custom_module``, fast_lora.py:178-200, fast_moe_lora.py:773-802) and ``get_peft_model`` then replaces
every targeted module by ``wrapper(target, adapter_name, config=..., r=..., lora_alpha=..., **kwargs)`` and freezes the rest
(train_qwen3.5_35b.py:96-118).  The registration functions of this package are written against that interface only, so a
real ``peft.LoraConfig`` works with them.  This module holds the two pieces a PEFT-free process lacks: a config object with
the fields those functions read, and the injection walk.  Nothing here is needed when PEFT is installed, and nothing here
was checked against PEFT itself (it is not importable where this package is tested).
"""

from __future__ import annotations

import re
from dataclasses import dataclass, field
from typing import Any, Iterable

import torch


@dataclass
class LoraConfig:
    """The fields of ``peft.LoraConfig`` the registration functions and wrappers read (train_qwen3.5_35b.py:96-110)."""

    r: int = 8
    lora_alpha: float = 8
    target_modules: Any = None          # a collection of module-name suffixes, or one regular expression (full match)
    target_parameters: Any = None
    lora_dropout: float = 0.0
    use_rslora: bool = False
    use_dora: bool = False
    lora_bias: bool = False
    init_lora_weights: Any = True
    alora_invocation_tokens: Any = None
    inference_mode: bool = False
    _custom_modules: dict | None = field(default=None, repr=False)

    def _register_custom_module(self, mapping: dict[type, type]) -> None:
        """Base-module class -> wrapper class; earlier registrations keep their place in the order of lookup."""
        if self._custom_modules is None:
            self._custom_modules = {}
        self._custom_modules.update(mapping)


def _is_target(name: str, target_modules) -> bool:
    if isinstance(target_modules, str):
        return re.fullmatch(target_modules, name) is not None
    return any(name == t or name.endswith("." + t) for t in target_modules or ())


def adapter_parameter_names(model: torch.nn.Module) -> list[str]:
    return [n for n, _ in model.named_parameters() if ".lora_" in "." + n]


def inject_adapter(model: torch.nn.Module, lora_config, adapter_name: str = "default") -> dict[str, list[str]]:
    """Replaces every module of ``model`` that ``lora_config.target_modules`` names and whose class (or a base class) has a
    registered wrapper, then leaves only the adapter factors trainable.  The first registered class that the module is an
    instance of wins, as in the reference's registration order (``GGUFLinear`` before ``torch.nn.Linear``,
    fast_lora.py:193-199).  A targeted module with no registered wrapper is an error, not a silent skip.
    Returns {"wrapped": paths, "trainable": parameter names}."""
    mapping = getattr(lora_config, "_custom_modules", None)
    if not mapping:
        raise RuntimeError("no wrapper classes are registered on this config; call the register_* functions first")
    wrappers = tuple(mapping.values())
    wrapped: list[str] = []
    for name, module in list(model.named_modules()):
        if not name or not _is_target(name, lora_config.target_modules) or isinstance(module, wrappers):
            continue
        parent_name, _, child = name.rpartition(".")
        parent = model.get_submodule(parent_name) if parent_name else model
        if isinstance(parent, wrappers):
            continue  # the base_layer of a wrapper made in an earlier call
        cls = next((wrapper for base, wrapper in mapping.items() if isinstance(module, base)), None)
        if cls is None:
            raise TypeError(f"target module {name!r} ({type(module).__name__}) has no registered LoRA wrapper")
        setattr(parent, child, cls(module, adapter_name, config=lora_config, r=lora_config.r, lora_alpha=lora_config.lora_alpha))
        wrapped.append(name)
    if not wrapped:
        raise ValueError("target_modules matched no module of the model")
    trainable = set(adapter_parameter_names(model))
    for n, p in model.named_parameters():
        p.requires_grad_(n in trainable and not getattr(lora_config, "inference_mode", False))
    return {"wrapped": wrapped, "trainable": sorted(trainable)}


def adapter_options(config, kwargs: dict[str, Any], names: Iterable[str]) -> dict[str, Any]:
    """The adapter options a wrapper honours, from the config PEFT passes (``config=``) or from keyword arguments of a direct
    construction; the keyword wins where both are given."""
    defaults = LoraConfig()
    out = {}
    for n in names:
        if n in kwargs:
            out[n] = kwargs[n]
        elif config is not None and hasattr(config, n):
            out[n] = getattr(config, n)
        else:
            out[n] = getattr(defaults, n)
    return out
