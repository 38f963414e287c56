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
