"""The reference's operator namespace on this library.

The reference reaches its native kernels through the ``torch_ggml_ops`` wheel: Python functions it imports
(``from torch_ggml_ops import mmq`` fast_lora.py:20, ``grouped_mmq`` / ``grouped_mmq_pair`` fast_moe_lora.py:221-228 and
:339-347, ``fixed_grouped_mmq`` deepseek_v4_lora.py:7) and dispatcher entries it calls directly
(``torch.ops.torch_ggml_ops.mmq`` / ``mmq_grad_input`` gguf_liger_loss.py:109-114 and :172-177,
``grouped_mmq_grad_input`` fast_moe_lora.py:255-262, ``grouped_mmq_pair_grad_input`` fast_moe_lora.py:365-374).
``install()`` registers those seven dispatcher entries under the same names with ``torch.library`` and, with
``as_module=True``, puts this module into ``sys.modules["torch_ggml_ops"]``.  As the wheel's contract has it
(docs/plan_qwen3.5.md:125-150) every entry has a FakeTensor / meta kernel (shapes only, so the call sites trace under
FakeTensorMode and ``torch.compile``), the four forward entries carry registered autograd whose backward is the matching
grad-input entry, and the grad-input entries reject differentiation (higher-order gradients).  The Python functions exported
here are differentiable in the activations, like the wheel's.

What the reference's files need beyond this namespace: ``fast_moe_lora.py`` also imports AITER's ``gmm`` / ``ptgmm``
(fast_moe_lora.py:22), for which ``grouped_mm.install_as_aiter_gmm()`` installs stand-ins on this library, and ``peft`` (:23-24);
``gguf_liger_loss.py`` imports ``liger_kernel`` (:16-25), and all of them the transformers ``gguf`` fork: those stay theirs to
provide.  The package's own modules of the same names replace those files without these imports.
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

    @op(f"{_NAMESPACE}::fixed_grouped_mmq_grad_input", mutates_args=())
    def _fixed_grouped_mmq_grad_input(grad_output: torch.Tensor, packed_groups: torch.Tensor, quant_type: int, in_features: int) -> torch.Tensor:
        return fast_lora.fixed_grouped_mmq_grad_input(grad_output, packed_groups, quant_type, in_features)

    # ---- FakeTensor / meta kernels: output shapes and dtypes only, with the shape checks that need no data
    def _last_dim(t: torch.Tensor, n: int) -> torch.Tensor:
        return t.new_empty((*t.shape[:-1], n))

    def _check_payload(packed: torch.Tensor, dims: int) -> None:
        torch._check(packed.dtype == torch.uint8 and packed.dim() == dims, lambda: f"packed weights must be uint8 with {dims} dimensions")

    @_mmq.register_fake
    def _(x, packed, quant_type, out_features):
        _check_payload(packed, 2)
        torch._check(packed.shape[0] == out_features, lambda: "payload rows do not match out_features")
        return _last_dim(x, out_features)

    @_mmq_grad_input.register_fake
    def _(grad_output, packed, quant_type, in_features):
        _check_payload(packed, 2)
        torch._check(packed.shape[0] == grad_output.shape[-1], lambda: "payload rows do not match the cotangent's last dimension")
        return _last_dim(grad_output, in_features)

    @_grouped_mmq.register_fake
    def _(hidden_states, payload, expert_indices, expert_offsets, quant_type, out_features):
        _check_payload(payload, 3)
        torch._check(hidden_states.dim() == 2 and payload.shape[1] == out_features, lambda: "grouped_mmq: [rows, k] rows against [experts, out_features, bytes]")
        return _last_dim(hidden_states, out_features)

    @_grouped_mmq_grad_input.register_fake
    def _(grad_output, payload, expert_indices, expert_offsets, quant_type, in_features):
        _check_payload(payload, 3)
        torch._check(grad_output.dim() == 2 and payload.shape[1] == grad_output.shape[1], lambda: "grouped_mmq_grad_input: cotangent columns against payload rows")
        return _last_dim(grad_output, in_features)

    @_grouped_mmq_pair.register_fake
    def _(hidden_states, first_payload, second_payload, expert_indices, expert_offsets, quant_type, out_features):
        _check_payload(first_payload, 3)
        torch._check(first_payload.shape == second_payload.shape and first_payload.shape[1] == out_features, lambda: "grouped_mmq_pair: payload shapes")
        return _last_dim(hidden_states, out_features), _last_dim(hidden_states, out_features)

    @_grouped_mmq_pair_grad_input.register_fake
    def _(first_grad, second_grad, first_payload, second_payload, expert_indices, expert_offsets, quant_type, in_features):
        _check_payload(first_payload, 3)
        torch._check(first_grad.shape == second_grad.shape, lambda: "grouped_mmq_pair_grad_input: cotangent shapes differ")
        return _last_dim(first_grad, in_features)

    @_fixed_grouped_mmq.register_fake
    def _(x, packed_groups, quant_type):
        _check_payload(packed_groups, 3)
        torch._check(x.dim() >= 2 and x.shape[-2] == packed_groups.shape[0], lambda: "fixed_grouped_mmq: [..., groups, k] against [groups, n, bytes]")
        return _last_dim(x, packed_groups.shape[1])

    @_fixed_grouped_mmq_grad_input.register_fake
    def _(grad_output, packed_groups, quant_type, in_features):
        _check_payload(packed_groups, 3)
        return _last_dim(grad_output, in_features)

    # ---- registered autograd: the forward entries differentiate in the activations through the grad-input entries
    # (frozen packed weights take no gradient); the grad-input entries have no formula, so differentiating through a
    # backward (a higher-order gradient) fails in the dispatcher
    ops = torch.ops.torch_ggml_ops

    def _save(*names):
        def setup(ctx, inputs, output):
            ctx.saved = {n: inputs[i] for i, n in names}
        return setup

    _mmq.register_autograd(
        lambda ctx, g: (ops.mmq_grad_input(g.contiguous(), ctx.saved["p"], ctx.saved["qt"], ctx.saved["x"].shape[-1]), None, None, None),
        setup_context=_save((0, "x"), (1, "p"), (2, "qt")))
    _grouped_mmq.register_autograd(
        lambda ctx, g: (ops.grouped_mmq_grad_input(g.contiguous(), ctx.saved["p"], ctx.saved["ids"], ctx.saved["off"], ctx.saved["qt"],
                                                   ctx.saved["x"].shape[-1]), None, None, None, None, None),
        setup_context=_save((0, "x"), (1, "p"), (2, "ids"), (3, "off"), (4, "qt")))
    _grouped_mmq_pair.register_autograd(
        lambda ctx, g1, g2: (ops.grouped_mmq_pair_grad_input(g1.contiguous(), g2.contiguous(), ctx.saved["p1"], ctx.saved["p2"], ctx.saved["ids"],
                                                             ctx.saved["off"], ctx.saved["qt"], ctx.saved["x"].shape[-1]), None, None, None, None, None, None),
        setup_context=_save((0, "x"), (1, "p1"), (2, "p2"), (3, "ids"), (4, "off"), (5, "qt")))
    _fixed_grouped_mmq.register_autograd(
        lambda ctx, g: (ops.fixed_grouped_mmq_grad_input(g.contiguous(), ctx.saved["p"], ctx.saved["qt"], ctx.saved["x"].shape[-1]), None, None),
        setup_context=_save((0, "x"), (1, "p"), (2, "qt")))

    _installed = True
