"""Chunked cross-entropy through a frozen packed GGUF lm_head.

Host-side mirror of the reference's ``gguf_liger_loss.py``: the same autograd ``Function`` contract
(loss and d(loss)/d(hidden) are both produced in forward, backward only scales by the upstream scalar
and rejects double backward; gguf_liger_loss.py:189-266) and the same causal-LM wrapper guards
(:269-356).  The chunk loop itself (:103-177) runs inside one call into the kernel library, which keeps
nothing wider than an 8192-column slab for chunks below 4096 rows and the chunk's bf16 logits (the reference's
[chunk, vocab] tensor) from there on, and needs no host synchronisation for the non-ignored count.
"""

from __future__ import annotations

from typing import Any

import torch

from . import _lib
from .fast_lora import _NATIVE_MMQ_QUANT_TYPES, GGUFLinear
from .gguf import GGUFQuantizedTensor, row_bytes

_PACKED_LM_HEAD_CHUNK_SIZE = 256


# set to True to wait for the device after every loss call and raise on labels outside [0, vocab) that are not
# ignore_index (the kernels treat such labels as ignored and only count them, so that no call has to synchronise)
VALIDATE_LABELS = False


def _packed_linear_cross_entropy_forward(input: torch.Tensor, packed_weight: torch.Tensor, target: torch.Tensor, quant_type: int,
                                         out_features: int, chunk_size: int, ignore_index: int, reduction: str,
                                         return_token_accuracy: bool = False, return_predicted_tokens: bool = False):
    """Returns (loss, grad_input, loss_1d, lse, status, token_accuracy, predicted_tokens); status is an int32[2] device tensor
    {rows that count, labels out of range}.  token_accuracy = correct argmax rows / rows that count (gguf_liger_loss.py:180-185),
    predicted_tokens int64 [rows] with -1 on ignored rows (:97-101); both None unless asked for."""
    if input.ndim != 2:
        raise ValueError(f"Packed LM-head loss expects two-dimensional hidden states, got {input.shape}.")
    if input.dtype != torch.bfloat16:
        raise TypeError(f"Packed LM-head loss requires BF16 hidden states, got {input.dtype}.")
    if target.ndim != 1 or target.shape[0] != input.shape[0]:
        raise ValueError("Packed LM-head targets must be one-dimensional and match the hidden-state row count.")
    if target.dtype != torch.long:
        raise TypeError(f"Packed LM-head targets require torch.long, got {target.dtype}.")
    if reduction not in {"mean", "sum"}:
        raise ValueError(f"Packed LM-head loss supports only mean or sum reduction, got {reduction!r}.")
    if chunk_size <= 0:
        raise ValueError(f"Packed LM-head chunk_size must be positive, got {chunk_size}.")
    if quant_type not in _NATIVE_MMQ_QUANT_TYPES:
        raise ValueError(f"GGML type id {quant_type} has no native MMQ kernel")
    rows, hidden = input.shape
    _lib.require_device_tensor(input, "hidden states", torch.bfloat16)
    _lib.require_device_tensor(packed_weight, "lm_head payload", torch.uint8)
    _lib.require_device_tensor(target, "targets", torch.long)
    if tuple(packed_weight.shape) != (out_features, row_bytes(quant_type, hidden)):
        raise ValueError(f"lm_head payload shape {tuple(packed_weight.shape)} does not describe [{out_features}, {hidden}] of type {quant_type}")
    dev = input.device
    grad_input = torch.zeros_like(input)
    loss_1d = torch.zeros(rows, dtype=torch.float32, device=dev)
    lse = torch.zeros(rows, dtype=torch.float32, device=dev)
    status = torch.zeros(2, dtype=torch.int32, device=dev)
    correct = torch.zeros(rows, dtype=torch.float32, device=dev) if return_token_accuracy else None
    predicted = torch.full((rows,), -1, dtype=torch.int64, device=dev) if return_predicted_tokens else None
    if rows:
        lib = _lib.load()
        ws = torch.empty(lib.ggq_lmhead_ce_workspace_bytes(rows, out_features, hidden, chunk_size), dtype=torch.uint8, device=dev)
        _lib.check(lib.ggq_lmhead_cross_entropy(quant_type, input.data_ptr(), packed_weight.data_ptr(), target.data_ptr(), rows, out_features,
                                               hidden, chunk_size, ignore_index, int(reduction == "mean"), loss_1d.data_ptr(),
                                               grad_input.data_ptr(), lse.data_ptr(), status.data_ptr(), _lib.ptr(predicted), _lib.ptr(correct),
                                               ws.data_ptr(), ws.numel(), _lib.stream_handle(dev)))
        if VALIDATE_LABELS and int(status[1]):
            raise ValueError(f"{int(status[1])} labels lie outside [0, {out_features}) and are not ignore_index={ignore_index}")
    token_accuracy = None
    if return_token_accuracy:
        # (no rows that count: 0 / 0 in the reference, gguf_liger_loss.py:183; defined as 0 here, like the loss)
        token_accuracy = torch.sum(correct) / torch.clamp(status[0], min=1).to(torch.float32)
    return torch.sum(loss_1d), grad_input, loss_1d, lse, status, token_accuracy, predicted


class _PackedLinearCrossEntropyFunction(torch.autograd.Function):
    """Fused loss over a frozen packed lm_head (counterpart of
    ``_PackedQ8LigerLinearCrossEntropyFunction``, gguf_liger_loss.py:189-266): returns (loss, token_accuracy,
    predicted_tokens), the last two None unless asked for and never differentiable."""

    @staticmethod
    def forward(ctx, input, packed_weight, target, quant_type, out_features, chunk_size, ignore_index, reduction,
                return_token_accuracy=False, return_predicted_tokens=False):
        loss, grad_input, _, _, _, token_accuracy, predicted = _packed_linear_cross_entropy_forward(
            input, packed_weight, target, quant_type, out_features, chunk_size, ignore_index, reduction,
            return_token_accuracy, return_predicted_tokens)
        ctx.save_for_backward(grad_input.detach())
        ctx.mark_non_differentiable(*[t for t in (token_accuracy, predicted) if t is not None])
        return loss, token_accuracy, predicted

    @staticmethod
    def backward(ctx, grad_output, grad_accuracy=None, grad_predicted=None):
        if torch.is_grad_enabled():
            raise RuntimeError("Packed GGUF LM-head loss does not support higher-order gradients")
        (grad_input,) = ctx.saved_tensors
        # the saved gradient assumes an upstream gradient of one; rescale only when it is not
        grad_input = grad_input * grad_output.to(grad_input.dtype)
        return grad_input, None, None, None, None, None, None, None, None, None


def packed_linear_cross_entropy(hidden_states, packed_weight, target, quant_type, out_features, chunk_size=_PACKED_LM_HEAD_CHUNK_SIZE,
                                ignore_index=-100, reduction="mean", return_token_accuracy=False, return_predicted_tokens=False):
    """The loss; with either flag set, the triple (loss, token_accuracy, predicted_tokens)."""
    loss, token_accuracy, predicted = _PackedLinearCrossEntropyFunction.apply(
        hidden_states, packed_weight.as_subclass(torch.Tensor), target, int(quant_type), int(out_features), int(chunk_size),
        int(ignore_index), reduction, bool(return_token_accuracy), bool(return_predicted_tokens))
    if return_token_accuracy or return_predicted_tokens:
        return loss, token_accuracy, predicted
    return loss


def _packed_for_causal_lm_loss(hidden_states: torch.Tensor, lm_head: GGUFLinear, labels: torch.Tensor, hidden_size: int,
                               num_items_in_batch: int | torch.Tensor | None = None, ignore_index: int = -100,
                               shift_labels: torch.Tensor | None = None, final_logit_softcapping: float | None = None,
                               return_token_accuracy: bool = False, return_predicted_tokens: bool = False,
                               chunk_size: int = _PACKED_LM_HEAD_CHUNK_SIZE, **kwargs: Any):
    """Causal-LM loss entry: option guards, label shift, mean vs sum/num_items, optional token accuracy and predicted
    tokens (gguf_liger_loss.py:269-356).  Unlike the reference, any hidden size that is a multiple of 64 and
    any natively supported GGML type is accepted (the reference validates 2048 / Q6_K only, :315-323)."""
    if kwargs.get("return_z_loss", False):
        raise RuntimeError("Packed GGUF LM-head loss does not support z-loss output.")
    if kwargs.get("use_token_scaling", False):
        raise RuntimeError("Packed GGUF LM-head loss does not support token scaling.")
    if kwargs.get("ce_weight") is not None:
        raise RuntimeError("Packed GGUF LM-head loss does not support class weights.")
    if kwargs.get("bias") is not None:
        raise RuntimeError("Packed GGUF LM-head loss does not support a fused bias.")
    if float(kwargs.get("label_smoothing", 0.0)) != 0.0:
        raise RuntimeError("Packed GGUF LM-head loss does not support label smoothing.")
    if float(kwargs.get("lse_square_scale", 0.0)) != 0.0:
        raise RuntimeError("Packed GGUF LM-head loss does not support LSE square scaling.")
    if final_logit_softcapping is not None:
        raise RuntimeError("Packed GGUF LM-head loss does not support logit softcapping.")
    if kwargs.get("accum_dtype") not in {None, torch.float32}:
        raise RuntimeError("Packed GGUF LM-head loss supports only FP32 internal accumulation.")
    if not isinstance(lm_head.weight, GGUFQuantizedTensor):
        raise TypeError("Packed GGUF LM-head loss requires a GGUFQuantizedTensor weight.")
    if lm_head.input_permutation is not None or lm_head.output_permutation is not None:
        raise RuntimeError("Packed GGUF LM-head loss does not support layout permutations.")
    if lm_head.compute_dtype != torch.bfloat16:
        raise RuntimeError("Packed GGUF LM-head loss requires BF16 compute_dtype.")
    if lm_head.in_features != hidden_size or hidden_size % 64:
        raise RuntimeError("Packed GGUF LM-head loss needs hidden_size == lm_head.in_features, a multiple of 64.")
    if lm_head.weight.requires_grad:
        raise RuntimeError("Packed GGUF LM-head weights must remain frozen.")
    if shift_labels is None:
        labels = torch.nn.functional.pad(labels, (0, 1), value=ignore_index)
        shift_labels = labels[..., 1:].contiguous()
    hidden_states = hidden_states.reshape(-1, hidden_size)
    shift_labels = shift_labels.reshape(-1).to(hidden_states.device)
    reduction = "sum" if num_items_in_batch is not None else "mean"
    loss, token_accuracy, predicted_tokens = _PackedLinearCrossEntropyFunction.apply(
        hidden_states, lm_head.weight.as_subclass(torch.Tensor), shift_labels, int(lm_head.weight.quant_type), int(lm_head.out_features),
        int(chunk_size), int(ignore_index), reduction, bool(return_token_accuracy), bool(return_predicted_tokens))
    if num_items_in_batch is not None:
        loss = loss / num_items_in_batch
    if return_token_accuracy or return_predicted_tokens:
        return loss, None, token_accuracy, predicted_tokens  # (loss, z_loss, accuracy, tokens), gguf_liger_loss.py:352-353
    return loss


# ------------------------------------------------------------------------------------------------
# Model-level installation (gguf_liger_loss.py:359-532 of the reference): a replacement forward for the causal-LM class
# that never builds the [tokens, vocab] logits while training, and the function that binds it to one loaded model.
def _causal_lm_output_class():
    """``MoeCausalLMOutputWithPast`` with the two extra fields of Liger's output class (gguf_liger_loss.py:502-512); a plain
    attribute/dict container with the same field names when transformers is not importable."""
    from dataclasses import dataclass, fields

    try:
        from transformers.modeling_outputs import MoeCausalLMOutputWithPast
    except ImportError:
        @dataclass
        class PackedMoeCausalLMOutputWithPast:
            loss: Any = None
            aux_loss: Any = None
            logits: Any = None
            past_key_values: Any = None
            hidden_states: Any = None
            attentions: Any = None
            router_logits: Any = None
            token_accuracy: Any = None
            predicted_tokens: Any = None

            def __getitem__(self, key):
                if isinstance(key, str):
                    return getattr(self, key)
                return tuple(getattr(self, f.name) for f in fields(self) if getattr(self, f.name) is not None)[key]

        return PackedMoeCausalLMOutputWithPast

    @dataclass
    class PackedMoeCausalLMOutputWithPast(MoeCausalLMOutputWithPast):
        token_accuracy: torch.Tensor | None = None
        predicted_tokens: torch.Tensor | None = None

    return PackedMoeCausalLMOutputWithPast


_OUTPUT_CLASS = None


def _output_class():
    global _OUTPUT_CLASS
    if _OUTPUT_CLASS is None:
        _OUTPUT_CLASS = _causal_lm_output_class()
    return _OUTPUT_CLASS


def _router_aux_loss(self, outputs, attention_mask):
    """The load-balancing term of the model family (gguf_liger_loss.py:472-481): transformers' own function, which the
    stock forward of the same class calls."""
    from transformers.models.qwen3_5_moe.modeling_qwen3_5_moe import load_balancing_loss_func

    return load_balancing_loss_func(outputs.router_logits, self.num_experts, self.num_experts_per_tok, attention_mask)


def gguf_liger_lce_forward(self, input_ids=None, attention_mask=None, position_ids=None, past_key_values=None, inputs_embeds=None,
                           labels=None, use_cache=None, output_attentions=None, output_hidden_states=None, output_router_logits=None,
                           mm_token_type_ids=None, cache_position=None, logits_to_keep: int | torch.Tensor = 0, skip_logits: bool | None = None,
                           return_dict: bool | None = None, **kwargs: Any):
    """Causal-LM forward over a packed lm_head (the flow and guards of gguf_liger_loss.py:359-512).  While training with labels
    the loss comes from the chunked packed cross-entropy and ``logits`` stays None; otherwise the head runs as a layer and
    the model's own ``loss_function`` is used.  ``self`` needs ``model``, ``lm_head``, ``config``, ``loss_function``,
    ``vocab_size`` and, for the router term, ``num_experts``, ``num_experts_per_tok`` and ``router_aux_loss_coef``.
    Arguments that are None are not forwarded to ``self.model``, so that model classes without them keep working."""
    config = self.config
    output_router_logits = output_router_logits if output_router_logits is not None else getattr(config, "output_router_logits", False)
    return_dict = return_dict if return_dict is not None else getattr(config, "use_return_dict", True)
    optional = dict(attention_mask=attention_mask, position_ids=position_ids, past_key_values=past_key_values, inputs_embeds=inputs_embeds,
                    use_cache=use_cache, output_attentions=output_attentions, output_hidden_states=output_hidden_states,
                    mm_token_type_ids=mm_token_type_ids, cache_position=cache_position)
    shift_labels = kwargs.pop("shift_labels", None)
    loss_kwargs = dict(kwargs)
    outputs = self.model(input_ids=input_ids, output_router_logits=output_router_logits,
                         **{k: v for k, v in optional.items() if v is not None}, **kwargs)
    hidden_states = outputs.last_hidden_state
    if hidden_states is None:
        raise RuntimeError("Qwen model did not return hidden states")
    slice_indices = slice(-logits_to_keep, None) if isinstance(logits_to_keep, int) else logits_to_keep
    kept_hidden_states = hidden_states[:, slice_indices, :]
    logits = loss = token_accuracy = predicted_tokens = None
    have_labels = labels is not None or shift_labels is not None
    if skip_logits is None:
        skip_logits = self.training and have_labels
    if skip_logits and not (isinstance(logits_to_keep, int) and logits_to_keep == 0):
        raise RuntimeError("Packed GGUF LM-head loss requires logits_to_keep=0 during training.")
    if skip_logits and not have_labels:
        raise RuntimeError("Packed GGUF LM-head loss requires labels or shift_labels.")
    if self.training and not skip_logits and have_labels:
        raise RuntimeError("Packed GGUF training with labels requires the no-full-logits fused loss.")
    if skip_logits:
        if not isinstance(self.lm_head, GGUFLinear):
            raise TypeError(f"GGUF-aware Liger loss requires a GGUFLinear LM head, got {type(self.lm_head).__name__}.")
        if self.lm_head.bias is not None:
            raise RuntimeError("GGUF-aware Liger loss currently requires a bias-free LM head.")
        result = _packed_for_causal_lm_loss(hidden_states=kept_hidden_states, lm_head=self.lm_head, labels=labels, shift_labels=shift_labels,
                                            hidden_size=config.hidden_size, **loss_kwargs)
        if isinstance(result, tuple):
            loss, _, token_accuracy, predicted_tokens = result
        else:
            loss = result
    else:
        logits = self.lm_head(kept_hidden_states)
        if have_labels:
            loss = self.loss_function(logits=logits, labels=labels, shift_labels=shift_labels, vocab_size=self.vocab_size, **loss_kwargs)
    aux_loss = None
    if output_router_logits:
        aux_loss = _router_aux_loss(self, outputs, attention_mask)
        if labels is not None:
            if loss is None:
                raise RuntimeError("router auxiliary loss requires a primary loss")
            loss = loss + self.router_aux_loss_coef * aux_loss.to(loss.device)
    if not return_dict:
        output = (logits,) + tuple(outputs[1:])
        output = ((aux_loss,) + output) if aux_loss is not None else output
        output = ((loss,) + output) if loss is not None else output
        output = output + (token_accuracy,) if token_accuracy is not None else output
        return output + (predicted_tokens,) if predicted_tokens is not None else output
    return _output_class()(loss=loss, aux_loss=aux_loss, logits=logits, past_key_values=getattr(outputs, "past_key_values", None),
                           hidden_states=getattr(outputs, "hidden_states", None), attentions=getattr(outputs, "attentions", None),
                           router_logits=getattr(outputs, "router_logits", None), token_accuracy=token_accuracy,
                           predicted_tokens=predicted_tokens)


def _unwrapped_causal_lm(model: torch.nn.Module, class_name: str, what: str) -> torch.nn.Module:
    get_base_model = getattr(model, "get_base_model", None)
    target = get_base_model() if callable(get_base_model) else model
    if not any(c.__name__ == class_name for c in type(target).__mro__):
        raise TypeError(f"{what} requires {class_name} after unwrapping PEFT, got {type(target).__name__}.")
    if not isinstance(target.lm_head, GGUFLinear):
        raise TypeError(f"{what} requires GGUFLinear, got {type(target.lm_head).__name__}.")
    return target


def apply_gguf_liger_fused_linear_cross_entropy(model: torch.nn.Module) -> torch.nn.Module:
    """Binds ``gguf_liger_lce_forward`` to one loaded text model (gguf_liger_loss.py:515-532): a PEFT wrapper is unwrapped
    through ``get_base_model``, the model must be a ``Qwen3_5MoeForCausalLM`` (by class name anywhere in its MRO, so that
    the fork's and upstream's classes both qualify) whose ``lm_head`` is a packed ``GGUFLinear``.  Returns the patched model."""
    from types import MethodType

    target = _unwrapped_causal_lm(model, "Qwen3_5MoeForCausalLM", "GGUF-aware Liger loss")
    target.forward = MethodType(gguf_liger_lce_forward, target)
    return target
