"""Expert-sorted routing layout for the grouped expert matmuls.

Host-side mirror of the reference's ``fast_moe_routing.py``: ``prepare_expert_routing`` sorts the flat
top-k expert ids and gathers the routed rows, ``finalize_expert_routing`` applies the routing weights
and sums every token's routes.  The sort is a stable counting sort on the device (ties keep ascending
route index), the per-expert counts / offsets / active-expert list come out of the same pass, and
gather / combine with their backward passes keep the reference's rounding order
(fast_moe_routing.py:126-226).  Unlike the reference (``_SUPPORTED_ROUTING_GEOMETRIES``, :14-26) any
top-k <= 16 and any hidden size that is a multiple of 8 is accepted.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from . import _lib


# set to True to wait for the device after every plan and raise on expert ids outside [0, num_experts) (the sort clamps such
# ids so that no access leaves its buffers and only flags them in ``status[1]``, so that no call has to synchronise)
VALIDATE_EXPERT_IDS = False


@dataclass(frozen=True)
class ExpertRoutingPlan:
    selected_hidden_states: torch.Tensor | None  # [routes, hidden] bf16, expert-sorted (None: prepared with gather=False)
    expert_indices: torch.Tensor           # [routes] int64, sorted expert id of every row
    routing_weights: torch.Tensor          # [tokens, top_k]
    permutation: torch.Tensor              # [routes] int64: sorted position -> route (token*k + rank)
    inverse_permutation: torch.Tensor      # [routes] int64: route -> sorted position
    num_tokens: int
    num_top_k: int
    hidden_dim: int
    # grouped-execution metadata produced by the same device pass (no host sync):
    expert_counts: torch.Tensor | None = None        # [E] int32 rows per expert
    expert_end_offsets: torch.Tensor | None = None   # [E] int32 cumulative end row per expert
    active_expert_ids: torch.Tensor | None = None    # [E] int64 compact list (first status[0] valid)
    active_end_offsets: torch.Tensor | None = None   # [E] int32 cumulative ends of the active experts
    status: torch.Tensor | None = None               # [2] int32: number of active experts, bad-id flag


def build_route_plan(top_k_index: torch.Tensor, num_experts: int):
    """Device-side stable sort of the routes by expert.  Returns (sorted ids, permutation, inverse,
    counts, end_offsets, active_ids, active_end_offsets, status)."""
    if top_k_index.ndim != 2:
        raise ValueError(f"Expert routing expects a [tokens, top_k] index matrix, got {tuple(top_k_index.shape)}")
    if top_k_index.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("Expert indices must use int32 or int64.")
    _lib.require_device_tensor(top_k_index, "top_k_index")
    tokens, k = top_k_index.shape
    routes = tokens * k
    dev = top_k_index.device
    sorted_ids = torch.empty(routes, dtype=torch.int64, device=dev)
    perm = torch.empty(routes, dtype=torch.int64, device=dev)
    inv = torch.empty(routes, dtype=torch.int64, device=dev)
    counts = torch.empty(num_experts, dtype=torch.int32, device=dev)
    ends = torch.empty(num_experts, dtype=torch.int32, device=dev)
    active_ids = torch.empty(num_experts, dtype=torch.int64, device=dev)
    active_ends = torch.empty(num_experts, dtype=torch.int32, device=dev)
    status = torch.empty(2, dtype=torch.int32, device=dev)
    lib = _lib.load()
    ws = torch.empty(lib.ggq_route_plan_workspace_bytes(tokens, k, num_experts), dtype=torch.uint8, device=dev)
    _lib.check(lib.ggq_route_plan(top_k_index.data_ptr(), int(top_k_index.dtype == torch.int64), tokens, k, num_experts,
                                  sorted_ids.data_ptr(), perm.data_ptr(), inv.data_ptr(), counts.data_ptr(), ends.data_ptr(),
                                  active_ids.data_ptr(), active_ends.data_ptr(), status.data_ptr(), ws.data_ptr(), ws.numel(),
                                  _lib.stream_handle(dev)))
    if VALIDATE_EXPERT_IDS and int(status[1]):
        raise ValueError(f"expert ids outside [0, {num_experts}) in the top-k index matrix")
    return sorted_ids, perm, inv, counts, ends, active_ids, active_ends, status


class _RouteGather(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden_states, permutation, inverse_permutation):
        tokens, hidden = hidden_states.shape
        top_k = permutation.numel() // max(tokens, 1)
        selected = torch.empty(permutation.numel(), hidden, dtype=hidden_states.dtype, device=hidden_states.device)
        _lib.check(_lib.load().ggq_route_gather_forward(hidden_states.data_ptr(), permutation.data_ptr(), selected.data_ptr(),
                                                        tokens, top_k, hidden, _lib.stream_handle(hidden_states.device)))
        ctx.save_for_backward(inverse_permutation)
        ctx.geometry = (tokens, top_k, hidden)
        return selected

    @staticmethod
    def backward(ctx, grad_selected):
        if not ctx.needs_input_grad[0]:
            return None, None, None
        (inverse_permutation,) = ctx.saved_tensors
        tokens, top_k, hidden = ctx.geometry
        grad_selected = grad_selected.contiguous()
        grad_hidden = torch.empty(tokens, hidden, dtype=grad_selected.dtype, device=grad_selected.device)
        _lib.check(_lib.load().ggq_route_gather_backward(grad_selected.data_ptr(), inverse_permutation.data_ptr(), grad_hidden.data_ptr(),
                                                         tokens, top_k, hidden, _lib.stream_handle(grad_selected.device)))
        return grad_hidden, None, None


class _RouteCombine(torch.autograd.Function):
    @staticmethod
    def forward(ctx, expert_output, routing_weights, permutation, inverse_permutation):
        tokens, top_k = routing_weights.shape
        hidden = expert_output.shape[1]
        result = torch.empty(tokens, hidden, dtype=expert_output.dtype, device=expert_output.device)
        _lib.check(_lib.load().ggq_route_combine_forward(expert_output.data_ptr(), routing_weights.data_ptr(),
                                                         int(routing_weights.dtype == torch.bfloat16), inverse_permutation.data_ptr(),
                                                         result.data_ptr(), tokens, top_k, hidden, _lib.stream_handle(expert_output.device)))
        ctx.save_for_backward(expert_output, routing_weights, permutation)
        ctx.geometry = (tokens, top_k, hidden)
        return result

    @staticmethod
    def backward(ctx, grad_final):
        expert_output, routing_weights, permutation = ctx.saved_tensors
        tokens, top_k, hidden = ctx.geometry
        grad_final = grad_final.contiguous()
        d_out = torch.empty_like(expert_output) if ctx.needs_input_grad[0] else None
        d_w = torch.empty_like(routing_weights) if ctx.needs_input_grad[1] else None
        if d_out is not None or d_w is not None:
            _lib.check(_lib.load().ggq_route_combine_backward(expert_output.data_ptr(), routing_weights.data_ptr(),
                                                              int(routing_weights.dtype == torch.bfloat16), permutation.data_ptr(),
                                                              grad_final.data_ptr(), _lib.ptr(d_out), _lib.ptr(d_w), tokens, top_k, hidden,
                                                              _lib.stream_handle(grad_final.device)))
        return d_out, d_w, None, None


def _validate_routing(hidden_states, top_k_index, top_k_weights) -> None:
    if hidden_states.device.type != "cuda":
        raise RuntimeError("Optimized expert routing requires CUDA/ROCm tensors.")
    if hidden_states.dtype != torch.bfloat16 or not hidden_states.is_contiguous():
        raise RuntimeError("Optimized expert routing requires contiguous BF16 hidden states.")
    if top_k_index.device != hidden_states.device:
        raise RuntimeError("Expert indices must be on the hidden-state device.")
    if top_k_weights.device != hidden_states.device:
        raise RuntimeError("Routing weights must be on the hidden-state device.")
    if top_k_index.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("Expert indices must use int32 or int64.")
    if top_k_weights.dtype not in (torch.bfloat16, torch.float32):
        raise RuntimeError("Routing weights must use BF16 or FP32.")
    tokens, hidden = hidden_states.shape
    if tokens <= 0 or hidden % 8 or not 0 < top_k_index.shape[1] <= 16:
        raise RuntimeError("Unsupported expert-routing geometry: needs tokens > 0, hidden % 8 == 0 and top_k <= 16.")


def prepare_expert_routing(hidden_states: torch.Tensor, top_k_index: torch.Tensor, top_k_weights: torch.Tensor,
                           num_experts: int | None = None, gather: bool = True) -> ExpertRoutingPlan:
    """``gather=False`` leaves ``selected_hidden_states`` unset, for a caller whose first grouped launch reads the token
    rows through ``permutation`` itself."""
    if hidden_states.ndim != 2:
        raise ValueError(f"Expert routing expects hidden states [tokens, hidden], got {hidden_states.shape}.")
    if top_k_index.ndim != 2 or top_k_weights.shape != top_k_index.shape:
        raise ValueError("Expert routing expects matching top-k index and weight matrices.")
    if top_k_index.shape[0] != hidden_states.shape[0]:
        raise ValueError("Expert routing token count does not match the hidden-state token count.")
    routing_weights = top_k_weights.contiguous()
    _validate_routing(hidden_states, top_k_index, routing_weights)
    if num_experts is None:
        # the reference's sort needs no expert count; without one, size the histogram from the data
        num_experts = int(top_k_index.max().item()) + 1
    sorted_ids, perm, inv, counts, ends, active_ids, active_ends, status = build_route_plan(top_k_index.contiguous(), num_experts)
    selected = _RouteGather.apply(hidden_states, perm, inv) if gather else None
    return ExpertRoutingPlan(
        selected_hidden_states=selected, expert_indices=sorted_ids, routing_weights=routing_weights,
        permutation=perm, inverse_permutation=inv, num_tokens=hidden_states.shape[0], num_top_k=top_k_index.shape[1],
        hidden_dim=hidden_states.shape[1], expert_counts=counts, expert_end_offsets=ends,
        active_expert_ids=active_ids, active_end_offsets=active_ends, status=status)


def finalize_expert_routing(output: torch.Tensor, hidden_states: torch.Tensor, routing_plan: ExpertRoutingPlan,
                            output_mask: torch.Tensor | None) -> torch.Tensor:
    if output_mask is not None:
        raise RuntimeError("Optimized expert routing does not support output masks.")
    expected = (routing_plan.num_tokens * routing_plan.num_top_k, routing_plan.hidden_dim)
    if output.device.type != "cuda" or output.dtype != torch.bfloat16 or not output.is_contiguous() or tuple(output.shape) != expected:
        raise RuntimeError(f"Optimized expert combine requires contiguous CUDA BF16 output with shape {expected}, got {tuple(output.shape)}.")
    result = _RouteCombine.apply(output, routing_plan.routing_weights, routing_plan.permutation, routing_plan.inverse_permutation)
    return result.to(hidden_states.dtype)
