"""The reference's operator namespace on this library.

The reference reaches its native kernels through the ``torch_ggml_ops`` wheel: Python functions it imports
(``from torch_ggml_ops import mmq`` fast_lora.py:20, ``grouped_mmq`` / ``grouped_mmq_pair`` fast_moe_lora.py:221-228 and
:339-347, ``fixed_grouped_mmq`` deepseek_v4_lora.py:7) and dispatcher entries it calls directly
(``torch.ops.torch_ggml_ops.mmq`` / ``mmq_grad_input`` gguf_liger_loss.py:109-114 and :172-177,
``grouped_mmq_grad_input`` fast_moe_lora.py:255-262, ``grouped_mmq_pair_grad_input`` fast_moe_lora.py:365-374).
``install()`` registers those seven dispatcher entries under the same names with ``torch.library`` (raw kernels launches, no
autograd, as the reference wraps them in its own ``autograd.Function``s) and, with ``as_module=True``, puts this module into
``sys.modules["torch_ggml_ops"]`` so that the reference's own files import and run unmodified on MI355X.  The Python
functions exported here are differentiable in the activations, like the wheel's.
"""

from __future__ import annotations

import sys

import torch

from . import fast_lora, fast_moe_lora

_NAMESPACE = "torch_ggml_ops"
_installed = False

# differentiable Python entry points, with the wheel's names and argument order
mmq = fast_lora.mmq
mmq_grad_input = fast_lora.mmq_grad_input
grouped_mmq = fast_moe_lora.grouped_mmq
grouped_mmq_pair = fast_moe_lora.grouped_mmq_pair
grouped_mmq_grad_input = fast_moe_lora.grouped_mmq_grad_input
grouped_mmq_pair_grad_input = fast_moe_lora.grouped_mmq_pair_grad_input


def fixed_grouped_mmq(x: torch.Tensor, packed_groups: torch.Tensor) -> torch.Tensor:
    """``[..., groups, k]`` x packed ``[groups, n, bytes]`` (deepseek_v4_lora.py:123); the block format comes from the packed
    tensor's ``quant_type`` (Q8_0 when it carries none)."""
    return fast_lora.fixed_grouped_mmq(x, packed_groups, int(getattr(packed_groups, "quant_type", 8)))


def install(as_module: bool = False) -> None:
    """Registers ``torch.ops.torch_ggml_ops.*`` (once per process); ``as_module`` also makes ``import torch_ggml_ops``
    resolve to this module.  Refuses to shadow a real ``torch_ggml_ops`` that is already imported."""
    global _installed
    if as_module:
        other = sys.modules.get(_NAMESPACE)
        if other is not None and other is not sys.modules[__name__]:
            raise RuntimeError("a different torch_ggml_ops module is already imported")
        sys.modules[_NAMESPACE] = sys.modules[__name__]
    if _installed:
        return
    op = torch.library.custom_op

    @op(f"{_NAMESPACE}::mmq", mutates_args=())
    def _mmq(x: torch.Tensor, packed: torch.Tensor, quant_type: int, out_features: int) -> torch.Tensor:
        return fast_lora._mmq_forward(x, packed, quant_type, out_features)

    @op(f"{_NAMESPACE}::mmq_grad_input", mutates_args=())
    def _mmq_grad_input(grad_output: torch.Tensor, packed: torch.Tensor, quant_type: int, in_features: int) -> torch.Tensor:
        return fast_lora.mmq_grad_input(grad_output, packed, quant_type, in_features)

    @op(f"{_NAMESPACE}::grouped_mmq", mutates_args=())
    def _grouped_mmq(hidden_states: torch.Tensor, payload: torch.Tensor, expert_indices: torch.Tensor, expert_offsets: torch.Tensor,
                     quant_type: int, out_features: int) -> torch.Tensor:
        return fast_moe_lora._grouped_forward(hidden_states, payload, None, expert_indices, expert_offsets, quant_type, out_features, None, None, 0.0)[0]

    @op(f"{_NAMESPACE}::grouped_mmq_grad_input", mutates_args=())
    def _grouped_mmq_grad_input(grad_output: torch.Tensor, payload: torch.Tensor, expert_indices: torch.Tensor, expert_offsets: torch.Tensor,
                                quant_type: int, in_features: int) -> torch.Tensor:
        return fast_moe_lora.grouped_mmq_grad_input(grad_output, payload, expert_indices, expert_offsets, quant_type, in_features)

    @op(f"{_NAMESPACE}::grouped_mmq_pair", mutates_args=())
    def _grouped_mmq_pair(hidden_states: torch.Tensor, first_payload: torch.Tensor, second_payload: torch.Tensor, expert_indices: torch.Tensor,
                          expert_offsets: torch.Tensor, quant_type: int, out_features: int) -> tuple[torch.Tensor, torch.Tensor]:
        y1, y2, _ = fast_moe_lora._grouped_forward(hidden_states, first_payload, second_payload, expert_indices, expert_offsets, quant_type,
                                                   out_features, None, None, 0.0)
        return y1, y2

    @op(f"{_NAMESPACE}::grouped_mmq_pair_grad_input", mutates_args=())
    def _grouped_mmq_pair_grad_input(first_grad: torch.Tensor, second_grad: torch.Tensor, first_payload: torch.Tensor, second_payload: torch.Tensor,
                                     expert_indices: torch.Tensor, expert_offsets: torch.Tensor, quant_type: int, in_features: int) -> torch.Tensor:
        return fast_moe_lora.grouped_mmq_pair_grad_input(first_grad, second_grad, first_payload, second_payload, expert_indices, expert_offsets,
                                                         quant_type, in_features)

    @op(f"{_NAMESPACE}::fixed_grouped_mmq", mutates_args=())
    def _fixed_grouped_mmq(x: torch.Tensor, packed_groups: torch.Tensor, quant_type: int) -> torch.Tensor:
        with torch.no_grad():
            return fast_lora.fixed_grouped_mmq(x, packed_groups, quant_type)

    _installed = True
