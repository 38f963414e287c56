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
