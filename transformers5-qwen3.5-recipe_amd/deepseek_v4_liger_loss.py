"""DeepSeek-V4 twin of the packed lm_head loss (deepseek_v4_liger_loss.py:32, :222-318 of the reference): the same chunked
cross-entropy with DeepSeek's chunk of 512 rows and its Q8_0 head."""

from __future__ import annotations

from typing import Any

import torch

from .fast_lora import GGUFLinear
from .gguf_liger_loss import _packed_for_causal_lm_loss

_PACKED_LM_HEAD_CHUNK_SIZE = 512


def _packed_q8_liger_for_causal_lm_loss(hidden_states: torch.Tensor, lm_head: GGUFLinear, labels: torch.Tensor, hidden_size: int,
                                        num_items_in_batch: int | torch.Tensor | None = None, ignore_index: int = -100,
                                        shift_labels: torch.Tensor | None = None, final_logit_softcapping: float | None = None,
                                        **kwargs: Any) -> torch.Tensor:
    """The optimised DeepSeek causal-LM loss (deepseek_v4_liger_loss.py:222-299): the shared option guards, plus the
    reference's restriction of this entry to Q8_0 heads."""
    quant_type = int(getattr(lm_head.weight, "quant_type", -1))
    if quant_type != 8:
        raise RuntimeError("Packed DeepSeek LM-head loss is validated only for Q8_0 weights.")
    return _packed_for_causal_lm_loss(hidden_states, lm_head, labels, hidden_size, num_items_in_batch=num_items_in_batch, ignore_index=ignore_index,
                                      shift_labels=shift_labels, final_logit_softcapping=final_logit_softcapping,
                                      chunk_size=_PACKED_LM_HEAD_CHUNK_SIZE, **kwargs)


def deepseek_v4_packed_liger_causal_lm_loss(hidden_states: torch.Tensor, lm_head: GGUFLinear, labels: torch.Tensor, *, hidden_size: int,
                                            loss_kwargs: dict[str, Any] | None = None) -> torch.Tensor:
    """Public scoped packed loss (deepseek_v4_liger_loss.py:302-318)."""
    return _packed_q8_liger_for_causal_lm_loss(hidden_states, lm_head, labels, hidden_size=hidden_size, **({} if loss_kwargs is None else loss_kwargs))


def _deepseek_v4_liger_forward(self, input_ids=None, attention_mask=None, position_ids=None, past_key_values=None, inputs_embeds=None,
                               labels=None, use_cache=None, output_router_logits=None, logits_to_keep: int | torch.Tensor = 0, **kwargs: Any):
    """DeepSeek-V4's causal-LM forward over its packed Q8_0 head (deepseek_v4_liger_loss.py:321-392): with labels the scoped
    packed loss and no logits, without labels the head as a layer; the router term as in the stock forward."""
    from .gguf_liger_loss import _output_class, _router_aux_loss

    output_router_logits = output_router_logits if output_router_logits is not None else getattr(self.config, "output_router_logits", False)
    optional = dict(attention_mask=attention_mask, position_ids=position_ids, past_key_values=past_key_values, inputs_embeds=inputs_embeds,
                    use_cache=use_cache)
    outputs = self.model(input_ids=input_ids, output_router_logits=output_router_logits,
                         **{k: v for k, v in optional.items() if v is not None}, **kwargs)
    hidden_states = outputs.last_hidden_state
    loss = logits = None
    if labels is None:
        slice_indices = slice(-logits_to_keep, None) if isinstance(logits_to_keep, int) else logits_to_keep
        logits = self.lm_head(hidden_states[:, slice_indices, :])
    else:
        loss = deepseek_v4_packed_liger_causal_lm_loss(hidden_states, self.lm_head, labels, hidden_size=self.config.hidden_size, loss_kwargs=kwargs)
    aux_loss = None
    if output_router_logits:
        aux_loss = _router_aux_loss(self, outputs, attention_mask)
        if labels is not None:
            loss = loss + self.router_aux_loss_coef * aux_loss.to(loss.device)
    return _output_class()(loss=loss, aux_loss=aux_loss, logits=logits, past_key_values=getattr(outputs, "past_key_values", None),
                           hidden_states=getattr(outputs, "hidden_states", None), attentions=getattr(outputs, "attentions", None),
                           router_logits=getattr(outputs, "router_logits", None))


def apply_deepseek_v4_liger_loss(model: torch.nn.Module) -> torch.nn.Module:
    """Binds that forward to one model instance, once (deepseek_v4_liger_loss.py:395-420)."""
    from types import MethodType

    from .gguf_liger_loss import _unwrapped_causal_lm

    base = _unwrapped_causal_lm(model, "DeepseekV4ForCausalLM", "DeepSeek V4 GGUF loss")
    if getattr(base, "_deepseek_v4_liger_loss_enabled", False):
        return base
    base.forward = MethodType(_deepseek_v4_liger_forward, base)
    base.__dict__["_deepseek_v4_liger_loss_enabled"] = True
    return base
