"""Grouped-expert MoE LoRA over frozen packed GGUF expert weights.

Host-side mirror of the reference's ``fast_moe_lora.py``.  Operator names follow the reference's native
boundary (``grouped_mmq``, ``grouped_mmq_pair`` and their ``_grad_input`` twins, fast_moe_lora.py:221,
255, 339, 364); the expert-layer forward keeps its structure (route -> gate/up pair -> SiLU gate -> down
-> combine, fast_moe_lora.py:685-770).  What differs is the fusion: the per-expert LoRA delta that the
reference computes with separate AITER grouped GEMMs (fast_moe_lora.py:42-151, 675-682) is folded into
the packed-weight kernels, so each projection is one forward call (base + s (x A^T) B^T) and one backward
call (dX plus dA, dB for all expert planes, zeros for experts without rows).

Expert groups are passed as ``expert_indices`` (int64) and cumulative END ``expert_offsets`` (int32), as
in the reference (test_fast_moe_lora.py:136-137).  The layer itself uses the full list of experts with
the device-computed offsets, so no host synchronisation is needed to learn which experts are active.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any

import torch

from . import _lib
from .fast_lora import _NATIVE_MMQ_QUANT_TYPES, supports_native_mmq
from .fast_moe_routing import ExpertRoutingPlan, finalize_expert_routing, prepare_expert_routing
from .gguf import GGUFQuantizedTensor, dequantize_gguf_tensor, row_bytes
from .grouped_mm import aiter_grouped_mm, gmm, lora_grouped_linear

EXPERTS_IMPLEMENTATION = "qwen3_5_moe_gguf_mmq_lora"
# the reference's own structure under the reference's own name (fast_moe_lora.py:38): base projections and LoRA deltas as
# separate grouped products, and expert weights that have no packed kernel served by decode + gmm
SEPARATED_EXPERTS_IMPLEMENTATION = "qwen3_5_moe_gguf_mmq_aiter_lora"

# name -> forward(experts, hidden_states, top_k_index, top_k_weights, lora_weights): the registry packed expert modules look
# their forward up in (stand-in for the fork's ``ALL_GGUF_EXPERTS_FUNCTIONS``, which fast_moe_lora.py:797-799 fills)
ALL_GGUF_EXPERTS_FUNCTIONS: dict[str, Any] = {}


# ------------------------------------------------------------------------------------------------
def _check_grouped(x, payload, expert_indices, expert_offsets, quant_type, n, k, what):
    _lib.require_device_tensor(x, f"{what} rows", torch.bfloat16)
    _lib.require_device_tensor(payload, f"{what} payload", torch.uint8)
    _lib.require_device_tensor(expert_indices, f"{what} expert_indices", torch.int64)
    _lib.require_device_tensor(expert_offsets, f"{what} expert_offsets", torch.int32)
    if quant_type not in _NATIVE_MMQ_QUANT_TYPES:
        raise ValueError(f"{what}: GGML type id {quant_type} has no native grouped MMQ kernel")
    if x.ndim != 2 or payload.ndim != 3 or expert_indices.ndim != 1 or expert_offsets.shape != expert_indices.shape:
        raise ValueError(f"{what}: expects rows [R,K], payload [E,N,bytes], expert_indices [G] and expert_offsets [G]")
    if payload.shape[1] != n or payload.shape[2] != row_bytes(quant_type, k):
        raise ValueError(f"{what}: payload shape {tuple(payload.shape)} does not describe [E,{n},{k}] of type {quant_type}")
    if k % 64:
        raise ValueError(f"{what}: in_features {k} must be a multiple of 64")


def _lora_ws(device, rows, groups, experts, n_total, k, r):
    nbytes = _lib.load().ggq_lora_workspace_bytes(rows, groups, experts, n_total, k, max(r, 1))
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def build_group_tables(expert_indices: torch.Tensor, expert_offsets: torch.Tensor, rows: int, experts: int) -> torch.Tensor:
    """The row-tile tables of one grouping (``ggq_group_tables_build``), for the grouped calls of a step that share it: every
    such call otherwise builds the same tables in a launch of its own."""
    lib = _lib.load()
    groups = expert_indices.numel()
    tables = torch.empty(int(lib.ggq_group_tables_bytes(rows, groups, experts)), dtype=torch.uint8, device=expert_indices.device)
    _lib.check(lib.ggq_group_tables_build(expert_indices.data_ptr(), expert_offsets.data_ptr(), groups, experts, rows, tables.data_ptr(),
                                          tables.numel(), _lib.stream_handle(expert_indices.device)))
    return tables


def _grouped_forward(x, p1, p2, expert_indices, expert_offsets, quant_type, n, lora_a, lora_b, scaling, row_index=None, index_div=1,
                     group_tables=None):
    """``row_index`` (int64, one entry per expert-sorted row) makes row i of the launch row ``row_index[i] // index_div`` of x.
    ``group_tables``: what ``build_group_tables`` returned for these expert_indices / expert_offsets / rows."""
    k = x.shape[1]
    rows = x.shape[0] if row_index is None else row_index.numel()
    experts = p1.shape[0]
    _check_grouped(x, p1, expert_indices, expert_offsets, quant_type, n, k, "grouped_mmq")
    if p2 is not None:
        if p2.shape != p1.shape:
            raise RuntimeError("Paired grouped GGUF MMQ requires matching logical shapes.")
        _lib.require_device_tensor(p2, "grouped_mmq second payload", torch.uint8)
    nseg = 1 if p2 is None else 2
    r = 0
    xa = None
    if lora_a is not None:
        _lib.require_device_tensor(lora_a, "expert lora_A", torch.bfloat16)
        _lib.require_device_tensor(lora_b, "expert lora_B", torch.bfloat16)
        r = lora_a.shape[1]
        if tuple(lora_a.shape) != (experts, r, k) or tuple(lora_b.shape) != (experts, nseg * n, r):
            raise ValueError(f"expert LoRA factors must be A [{experts},r,{k}] and B [{experts},{nseg * n},r], got {tuple(lora_a.shape)}, {tuple(lora_b.shape)}")
        xa = torch.empty(rows, (r + 15) // 16 * 16, dtype=torch.bfloat16, device=x.device)
    y1 = torch.empty(rows, n, dtype=torch.bfloat16, device=x.device)
    y2 = torch.empty(rows, n, dtype=torch.bfloat16, device=x.device) if p2 is not None else None
    if rows:
        ws = _lora_ws(x.device, rows, expert_indices.numel(), experts, nseg * n, k, r)
        tail = (p1.data_ptr(), _lib.ptr(p2), expert_indices.data_ptr(), expert_offsets.data_ptr(), expert_indices.numel(),
                experts, quant_type, rows, n, k, _lib.ptr(lora_a), _lib.ptr(lora_b), r, float(scaling), _lib.ptr(xa), y1.data_ptr(),
                _lib.ptr(y2), _lib.ptr(group_tables), ws.data_ptr(), ws.numel(), _lib.stream_handle(x.device))
        if row_index is None:
            _lib.check(_lib.load().ggq_grouped_lora_mmq_forward(x.data_ptr(), *tail))
        else:
            _lib.check(_lib.load().ggq_grouped_lora_mmq_forward_indexed(x.data_ptr(), x.shape[0], row_index.data_ptr(), int(index_div), *tail))
    return y1, y2, xa


def _grouped_backward(dy1, dy2, p1, p2, expert_indices, expert_offsets, quant_type, k, x, xa, lora_a, lora_b, scaling, want_da, want_db,
                      row_index=None, index_div=1, group_tables=None):
    rows, n = dy1.shape
    experts = p1.shape[0]
    _check_grouped(dy1, p1, expert_indices, expert_offsets, quant_type, n, k, "grouped_mmq_grad_input")
    nseg = 1 if p2 is None else 2
    if p2 is not None:
        _lib.require_device_tensor(dy2, "grouped_mmq_grad_input second cotangent", torch.bfloat16)
    r = 0 if lora_a is None else lora_a.shape[1]
    dx = torch.empty(rows, k, dtype=torch.bfloat16, device=dy1.device)
    da = torch.empty_like(lora_a) if (lora_a is not None and want_da) else None
    db = torch.empty_like(lora_b) if (lora_b is not None and want_db) else None
    ws = _lora_ws(dy1.device, rows, expert_indices.numel(), experts, nseg * n, k, r)
    head = (dy1.data_ptr(), _lib.ptr(dy2), p1.data_ptr(), _lib.ptr(p2), expert_indices.data_ptr(), expert_offsets.data_ptr(),
            expert_indices.numel(), experts, quant_type, rows, n, k, _lib.ptr(x))
    tail = (_lib.ptr(xa), _lib.ptr(lora_a), _lib.ptr(lora_b), r, float(scaling), dx.data_ptr(), _lib.ptr(da), _lib.ptr(db),
            _lib.ptr(group_tables), ws.data_ptr(), ws.numel(), _lib.stream_handle(dy1.device))
    if row_index is None:
        _lib.check(_lib.load().ggq_grouped_lora_mmq_backward(*head, *tail))
    else:
        _lib.check(_lib.load().ggq_grouped_lora_mmq_backward_indexed(*head, x.shape[0], row_index.data_ptr(), int(index_div), *tail))
    return dx, da, db


def grouped_mmq_grad_input(grad_output, payload, expert_indices, expert_offsets, quant_type, in_features):
    """dX[r0:r1] = dY[r0:r1] . W[expert] per group (fast_moe_lora.py:255-262)."""
    payload = payload.as_subclass(torch.Tensor)
    dx, _, _ = _grouped_backward(grad_output, None, payload, None, expert_indices, expert_offsets, int(quant_type), int(in_features),
                                 None, None, None, None, 0.0, False, False)
    return dx


def grouped_mmq_pair_grad_input(first_grad, second_grad, first_payload, second_payload, expert_indices, expert_offsets, quant_type, in_features):
    """dX = dY1 . W1 + dY2 . W2 in one fp32 accumulator, rounded once (fast_moe_lora.py:364-375)."""
    dx, _, _ = _grouped_backward(first_grad, second_grad, first_payload.as_subclass(torch.Tensor), second_payload.as_subclass(torch.Tensor),
                                 expert_indices, expert_offsets, int(quant_type), int(in_features), None, None, None, None, 0.0, False, False)
    return dx


class _GroupedLoraProjection(torch.autograd.Function):
    """One expert projection (or a gate/up pair) with the LoRA delta fused in."""

    @staticmethod
    def forward(ctx, x, p1, p2, expert_indices, expert_offsets, quant_type, n, lora_a, lora_b, scaling, group_tables=None):
        y1, y2, xa = _grouped_forward(x, p1, p2, expert_indices, expert_offsets, quant_type, n, lora_a, lora_b, scaling,
                                      group_tables=group_tables)
        ctx.group_tables = group_tables
        tensors = [x, expert_indices, expert_offsets, p1]
        ctx.has_pair, ctx.has_lora = p2 is not None, lora_a is not None
        if ctx.has_pair:
            tensors.append(p2)
        if ctx.has_lora:
            tensors += [xa, lora_a, lora_b]
        ctx.save_for_backward(*tensors)
        ctx.meta = (quant_type, n, float(scaling))
        if ctx.has_pair:
            return y1, y2
        return y1

    @staticmethod
    def backward(ctx, *grads):
        if torch.is_grad_enabled():
            raise RuntimeError("packed grouped MMQ does not support higher-order gradients")
        saved = list(ctx.saved_tensors)
        x, expert_indices, expert_offsets, p1 = saved[:4]
        rest = saved[4:]
        p2 = rest.pop(0) if ctx.has_pair else None
        xa, lora_a, lora_b = rest if ctx.has_lora else (None, None, None)
        quant_type, n, scaling = ctx.meta
        g1 = grads[0]
        g2 = grads[1] if ctx.has_pair else None
        if ctx.has_pair and (g1 is None or g2 is None):
            if g1 is None and g2 is None:
                return (None,) * 11
            like = g1 if g1 is not None else g2
            g1 = torch.zeros_like(like) if g1 is None else g1
            g2 = torch.zeros_like(like) if g2 is None else g2
        g1 = g1.contiguous()
        g2 = g2.contiguous() if g2 is not None else None
        want_da, want_db = ctx.needs_input_grad[7], ctx.needs_input_grad[8]
        dx, da, db = _grouped_backward(g1, g2, p1, p2, expert_indices, expert_offsets, quant_type, x.shape[1], x, xa, lora_a, lora_b,
                                       scaling, want_da, want_db, group_tables=ctx.group_tables)
        return (dx if ctx.needs_input_grad[0] else None), None, None, None, None, None, None, da, db, None, None


class _RoutedGroupedLoraProjection(torch.autograd.Function):
    """``_GroupedLoraProjection`` applied to ``hidden_states[permutation // top_k]`` without that copy: the launch reads the
    token rows through the permutation, and the backward sums every token's routes (the backward of the reference's
    ``_RouteGather``, fast_moe_routing.py:126-160) after the input-gradient launch.  Bit-identical to gather + projection."""

    @staticmethod
    def forward(ctx, hidden_states, permutation, inverse_permutation, top_k, p1, p2, expert_indices, expert_offsets, quant_type, n,
                lora_a, lora_b, scaling, group_tables=None):
        y1, y2, xa = _grouped_forward(hidden_states, p1, p2, expert_indices, expert_offsets, quant_type, n, lora_a, lora_b, scaling,
                                      row_index=permutation, index_div=top_k, group_tables=group_tables)
        ctx.group_tables = group_tables
        tensors = [hidden_states, permutation, inverse_permutation, expert_indices, expert_offsets, p1]
        ctx.has_pair, ctx.has_lora = p2 is not None, lora_a is not None
        if ctx.has_pair:
            tensors.append(p2)
        if ctx.has_lora:
            tensors += [xa, lora_a, lora_b]
        ctx.save_for_backward(*tensors)
        ctx.meta = (quant_type, n, float(scaling), int(top_k))
        if ctx.has_pair:
            return y1, y2
        return y1

    @staticmethod
    def backward(ctx, *grads):
        if torch.is_grad_enabled():
            raise RuntimeError("packed grouped MMQ does not support higher-order gradients")
        saved = list(ctx.saved_tensors)
        hidden_states, permutation, inverse_permutation, expert_indices, expert_offsets, p1 = saved[:6]
        rest = saved[6:]
        p2 = rest.pop(0) if ctx.has_pair else None
        xa, lora_a, lora_b = rest if ctx.has_lora else (None, None, None)
        quant_type, n, scaling, top_k = ctx.meta
        g1 = grads[0]
        g2 = grads[1] if ctx.has_pair else None
        if ctx.has_pair and (g1 is None or g2 is None):
            if g1 is None and g2 is None:
                return (None,) * 14
            like = g1 if g1 is not None else g2
            g1 = torch.zeros_like(like) if g1 is None else g1
            g2 = torch.zeros_like(like) if g2 is None else g2
        g1 = g1.contiguous()
        g2 = g2.contiguous() if g2 is not None else None
        want_da, want_db = ctx.needs_input_grad[10], ctx.needs_input_grad[11]
        tokens, k = hidden_states.shape
        d_selected, da, db = _grouped_backward(g1, g2, p1, p2, expert_indices, expert_offsets, quant_type, k, hidden_states, xa, lora_a,
                                               lora_b, scaling, want_da, want_db, row_index=permutation, index_div=top_k,
                                               group_tables=ctx.group_tables)
        d_hidden = None
        if ctx.needs_input_grad[0]:
            d_hidden = torch.empty(tokens, k, dtype=d_selected.dtype, device=d_selected.device)
            _lib.check(_lib.load().ggq_route_gather_backward(d_selected.data_ptr(), inverse_permutation.data_ptr(), d_hidden.data_ptr(),
                                                             tokens, top_k, k, _lib.stream_handle(d_selected.device)))
        return (d_hidden,) + (None,) * 9 + (da, db, None, None)


def routed_projection_reads_tokens_in_place(quant_type: int, routes: int, groups: int, tokens: int, in_features: int) -> bool:
    """Whether the first grouped launch of an expert FFN can read the token matrix through the routing permutation
    (host-side answer of the library, no device work)."""
    return bool(_lib.load().ggq_grouped_forward_reads_indexed_rows(int(quant_type), int(routes), int(groups), int(tokens), int(in_features)))


def _as_payload(w):
    return w.as_subclass(torch.Tensor) if w is not None else None


def grouped_mmq(hidden_states, payload, expert_indices, expert_offsets, quant_type, out_features):
    """Y[r0:r1] = X[r0:r1] . W[expert]^T per group (fast_moe_lora.py:221-228); differentiable in X."""
    return _GroupedLoraProjection.apply(hidden_states, _as_payload(payload), None, expert_indices, expert_offsets, int(quant_type),
                                        int(out_features), None, None, 0.0)


def grouped_mmq_pair(hidden_states, first_payload, second_payload, expert_indices, expert_offsets, quant_type, out_features):
    """(gate, up) from one pass over X (fast_moe_lora.py:339-347); differentiable in X."""
    return _GroupedLoraProjection.apply(hidden_states, _as_payload(first_payload), _as_payload(second_payload), expert_indices,
                                        expert_offsets, int(quant_type), int(out_features), None, None, 0.0)


def grouped_lora_mmq(hidden_states, payload, expert_indices, expert_offsets, quant_type, out_features, lora_a, lora_b, scaling):
    return _GroupedLoraProjection.apply(hidden_states, _as_payload(payload), None, expert_indices, expert_offsets, int(quant_type),
                                        int(out_features), lora_a, lora_b, float(scaling))


def grouped_lora_mmq_pair(hidden_states, first_payload, second_payload, expert_indices, expert_offsets, quant_type, out_features,
                          lora_a, lora_b, scaling):
    return _GroupedLoraProjection.apply(hidden_states, _as_payload(first_payload), _as_payload(second_payload), expert_indices,
                                        expert_offsets, int(quant_type), int(out_features), lora_a, lora_b, float(scaling))


class _SwiGLU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate, up, limit):
        _lib.require_device_tensor(gate, "gate", torch.bfloat16)
        _lib.require_device_tensor(up, "up", torch.bfloat16)
        h = torch.empty_like(gate)
        lib, stream = _lib.load(), _lib.stream_handle(gate.device)
        if limit is None:
            _lib.check(lib.ggq_swiglu_forward(gate.data_ptr(), up.data_ptr(), h.data_ptr(), gate.numel(), stream))
        else:
            _lib.check(lib.ggq_swiglu_clamped_forward(gate.data_ptr(), up.data_ptr(), h.data_ptr(), gate.numel(), float(limit), stream))
        ctx.save_for_backward(gate, up)
        ctx.limit = limit
        return h

    @staticmethod
    def backward(ctx, dh):
        gate, up = ctx.saved_tensors
        dh = dh.contiguous()
        dgate, dup = torch.empty_like(gate), torch.empty_like(up)
        lib, stream = _lib.load(), _lib.stream_handle(gate.device)
        if ctx.limit is None:
            _lib.check(lib.ggq_swiglu_backward(gate.data_ptr(), up.data_ptr(), dh.data_ptr(), dgate.data_ptr(), dup.data_ptr(), gate.numel(), stream))
        else:
            _lib.check(lib.ggq_swiglu_clamped_backward(gate.data_ptr(), up.data_ptr(), dh.data_ptr(), dgate.data_ptr(), dup.data_ptr(),
                                                       gate.numel(), float(ctx.limit), stream))
        return dgate, dup, None


def swiglu(gate: torch.Tensor, up: torch.Tensor, limit: float | None = None) -> torch.Tensor:
    """silu(gate) * up (the fork's ``_apply_split_gate`` for ``hidden_act="silu"``, fast_moe_lora.py:747); with
    ``limit`` the DeepSeek form silu(min(gate, limit)) * clamp(up, -limit, limit) (``config.swiglu_limit``,
    test_deepseek_v4_moe_lora.py:184-199)."""
    if limit is not None and not limit > 0:
        raise ValueError(f"swiglu limit must be positive, got {limit}")
    return _SwiGLU.apply(gate, up, limit)


# set to False to run the activation, the down projection and the combine as three autograd nodes (the reference's structure)
FUSE_GATED_DOWN_COMBINE = True
# set to False to let every grouped call of the layer build its own row-tile tables
SHARE_GROUP_TABLES = True


class _RoutedGatedDownProjection(torch.autograd.Function):
    """silu(gate) * up, the down projection with its LoRA delta, and the weighted sum of every token's routes
    (fast_moe_lora.py:747-770 with fast_moe_routing.py:431-459) as ONE autograd node.  The forward runs the same three
    launches as the separate nodes and gives the same bits.  The backward never forms the [routes, hidden] cotangent of the
    expert output: the grad-input launch reads the tokens' cotangent rows through the permutation and leaves the routing
    weight out, the activation's backward applies it and computes the routing weights' gradient as
    <unweighted dH[route], h[route]>, which equals the reference's <dOut[token], expert_out[route]>
    (fast_moe_routing.py:217-224) up to rounding; the factor gradients carry the weight on their rank-r operand."""

    @staticmethod
    def forward(ctx, gate, up, limit, payload, expert_indices, expert_offsets, quant_type, out_features, lora_a, lora_b, scaling,
                routing_weights, permutation, inverse_permutation, group_tables=None):
        _lib.require_device_tensor(gate, "gate", torch.bfloat16)
        _lib.require_device_tensor(up, "up", torch.bfloat16)
        lib, stream = _lib.load(), _lib.stream_handle(gate.device)
        act = torch.empty_like(gate)
        if limit is None:
            _lib.check(lib.ggq_swiglu_forward(gate.data_ptr(), up.data_ptr(), act.data_ptr(), gate.numel(), stream))
        else:
            _lib.check(lib.ggq_swiglu_clamped_forward(gate.data_ptr(), up.data_ptr(), act.data_ptr(), gate.numel(), float(limit), stream))
        y, _, xa = _grouped_forward(act, payload, None, expert_indices, expert_offsets, quant_type, out_features, lora_a, lora_b, scaling,
                                    group_tables=group_tables)
        ctx.group_tables = group_tables
        tokens, top_k = routing_weights.shape
        out = torch.empty(tokens, out_features, dtype=y.dtype, device=y.device)
        _lib.check(lib.ggq_route_combine_forward(y.data_ptr(), routing_weights.data_ptr(), int(routing_weights.dtype == torch.bfloat16),
                                                 inverse_permutation.data_ptr(), out.data_ptr(), tokens, top_k, out_features, stream))
        ctx.has_lora = lora_a is not None
        ctx.save_for_backward(gate, up, act, payload, expert_indices, expert_offsets, routing_weights, permutation,
                              *((xa, lora_a, lora_b) if ctx.has_lora else ()))
        ctx.meta = (float(limit or 0.0), int(quant_type), int(out_features), float(scaling))
        return out

    @staticmethod
    def backward(ctx, grad_out):
        if torch.is_grad_enabled():
            raise RuntimeError("packed grouped MMQ does not support higher-order gradients")
        gate, up, act, payload, expert_indices, expert_offsets, routing_weights, permutation, *rest = ctx.saved_tensors
        xa, lora_a, lora_b = rest if ctx.has_lora else (None, None, None)
        limit, quant_type, n, scaling = ctx.meta
        grad_out = grad_out.contiguous()
        _lib.require_device_tensor(grad_out, "combined output cotangent", torch.bfloat16)
        rows, k = act.shape
        tokens, top_k = routing_weights.shape
        experts = payload.shape[0]
        r = 0 if lora_a is None else lora_a.shape[1]
        dev = act.device
        lib, stream = _lib.load(), _lib.stream_handle(dev)
        d_act = torch.empty(rows, k, dtype=torch.bfloat16, device=dev)
        da = torch.empty_like(lora_a) if (ctx.has_lora and ctx.needs_input_grad[8]) else None
        db = torch.empty_like(lora_b) if (ctx.has_lora and ctx.needs_input_grad[9]) else None
        w_bf16 = int(routing_weights.dtype == torch.bfloat16)
        ws = _lora_ws(dev, rows, expert_indices.numel(), experts, n, k, r)
        _lib.check(lib.ggq_grouped_lora_mmq_backward_routed_output(
            grad_out.data_ptr(), tokens, permutation.data_ptr(), top_k, routing_weights.data_ptr(), w_bf16, payload.data_ptr(),
            expert_indices.data_ptr(), expert_offsets.data_ptr(), expert_indices.numel(), experts, quant_type, rows, n, k, act.data_ptr(),
            _lib.ptr(xa), _lib.ptr(lora_a), _lib.ptr(lora_b), r, scaling, d_act.data_ptr(), _lib.ptr(da), _lib.ptr(db),
            _lib.ptr(ctx.group_tables), ws.data_ptr(), ws.numel(), stream))
        dgate, dup = torch.empty_like(gate), torch.empty_like(up)
        dw = torch.empty_like(routing_weights) if ctx.needs_input_grad[11] else None
        _lib.check(lib.ggq_swiglu_backward_routed(gate.data_ptr(), up.data_ptr(), d_act.data_ptr(), routing_weights.data_ptr(), w_bf16,
                                                  permutation.data_ptr(), dgate.data_ptr(), dup.data_ptr(), _lib.ptr(dw), rows, k, limit, stream))
        return dgate, dup, None, None, None, None, None, None, da, db, None, dw, None, None, None


# ------------------------------------------------------------------------------------------------
def _group_sizes_from_offsets(offsets: torch.Tensor) -> torch.Tensor:
    if offsets.ndim != 1:
        raise ValueError(f"GGUF grouped execution requires one-dimensional offsets, got {offsets.shape}.")
    if offsets.dtype != torch.int32 or offsets.stride() != (1,):
        raise ValueError("GGUF grouped offsets must be contiguous int32.")
    return torch.diff(offsets, prepend=offsets.new_zeros(1))


def _complete_group_sizes(active_group_sizes: torch.Tensor, expert_indices: torch.Tensor, num_experts: int) -> torch.Tensor:
    if expert_indices.numel() == num_experts:
        return active_group_sizes
    return active_group_sizes.new_zeros(num_experts).index_copy(0, expert_indices, active_group_sizes)


@dataclass(frozen=True)
class _ExpertLoraWeights:
    gate_up_a: torch.Tensor  # [experts, rank, hidden]
    gate_up_b: torch.Tensor  # [experts, 2 * intermediate, rank]
    down_a: torch.Tensor     # [experts, rank, intermediate]
    down_b: torch.Tensor     # [experts, hidden, rank]
    scaling: float


@dataclass(frozen=True)
class _ExpertExecutionPlan:
    expert_indices: torch.Tensor
    offsets: torch.Tensor
    output_mask: torch.Tensor | None = None


class GGUFExperts(torch.nn.Module):
    """Packed expert weights of one MoE layer (stand-in for the fork's ``GGUFExperts``; exposes what
    fast_moe_lora.py:541-545, 698-709, 747 reads)."""

    projection_layout = "split_gate_up"
    has_bias = False
    has_gate = True

    def __init__(self, gate_proj: GGUFQuantizedTensor | torch.Tensor, up_proj: GGUFQuantizedTensor | torch.Tensor,
                 down_proj: GGUFQuantizedTensor | torch.Tensor, compute_dtype: torch.dtype = torch.bfloat16, swiglu_limit: float | None = None):
        super().__init__()
        self.swiglu_limit = swiglu_limit  # DeepSeek's config.swiglu_limit; None: plain silu(gate) * up

        def logical(w):  # plain floating-point planes are taken by the separated implementation only
            return tuple(w.logical_shape) if isinstance(w, GGUFQuantizedTensor) else tuple(w.shape)

        e, i, h = logical(gate_proj)
        if logical(up_proj) != (e, i, h) or logical(down_proj) != (e, h, i):
            raise ValueError("expert projections must be gate/up [E,I,H] and down [E,H,I]")
        self.gate_proj, self.up_proj, self.down_proj = gate_proj, up_proj, down_proj
        self.num_experts, self.hidden_dim, self.intermediate_dim = e, h, i
        self.compute_dtype = compute_dtype
        self._all_experts = torch.arange(e, dtype=torch.int64, device=gate_proj.device)

    def _prepare_expert_hidden_states(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return hidden_states.reshape(-1, self.hidden_dim).to(self.compute_dtype).contiguous()

    def _prepare_expert_execution(self, routing_plan: ExpertRoutingPlan, mode: str) -> _ExpertExecutionPlan:
        if mode != "grouped_mm":
            raise RuntimeError(f"unsupported expert execution mode {mode!r}")
        return _ExpertExecutionPlan(self._all_experts, routing_plan.expert_end_offsets, None)

    def _apply_split_gate(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        return swiglu(gate, up, self.swiglu_limit)

    experts_implementation = EXPERTS_IMPLEMENTATION

    def forward(self, hidden_states, top_k_index, top_k_weights, lora_weights: _ExpertLoraWeights | None = None):
        fn = ALL_GGUF_EXPERTS_FUNCTIONS.get(self.experts_implementation)
        if fn is None:
            raise RuntimeError(f"experts implementation {self.experts_implementation!r} is not registered")
        return fn(self, hidden_states, top_k_index, top_k_weights, lora_weights)


def qwen3_5_moe_gguf_mmq_lora_forward(self: GGUFExperts, hidden_states: torch.Tensor, top_k_index: torch.Tensor,
                                      top_k_weights: torch.Tensor, lora_weights: _ExpertLoraWeights | None = None) -> torch.Tensor:
    """Packed expert FFN with LoRA on gate/up and down (orchestration of fast_moe_lora.py:685-770)."""
    if not isinstance(self, GGUFExperts):
        raise TypeError(f"{EXPERTS_IMPLEMENTATION} requires GGUFExperts, got {type(self).__name__}.")
    if self.projection_layout != "split_gate_up" or self.has_bias or not self.has_gate:
        raise RuntimeError("The GGUF LoRA path requires split, bias-free gate/up expert projections.")
    for w in (self.gate_proj, self.up_proj, self.down_proj):
        if w.requires_grad:
            raise RuntimeError("Fast GGUF expert execution requires frozen packed base weights.")
        if not isinstance(w, GGUFQuantizedTensor):
            raise RuntimeError(f"{EXPERTS_IMPLEMENTATION} takes packed expert weights; {SEPARATED_EXPERTS_IMPLEMENTATION} also takes floating-point ones.")
        if not supports_native_mmq(w):
            raise RuntimeError(f"GGML type id {w.quant_type} has no native grouped MMQ kernel.")
    if self.compute_dtype != torch.bfloat16:
        raise RuntimeError("Grouped GGUF MMQ requires BF16 compute dtype.")
    if self.gate_proj.quant_type != self.up_proj.quant_type:
        raise RuntimeError("Paired grouped GGUF MMQ requires one quantization type.")

    compute_hidden_states = self._prepare_expert_hidden_states(hidden_states)
    tokens, top_k = top_k_index.shape[0], top_k_index.shape[1]
    # The gate/up launch reads the token rows in place where it can; the routed copy is made otherwise.
    in_place = (compute_hidden_states.ndim == 2 and compute_hidden_states.is_contiguous()
                and routed_projection_reads_tokens_in_place(self.gate_proj.quant_type, tokens * top_k, self.num_experts, tokens, self.hidden_dim))
    routing_plan = prepare_expert_routing(compute_hidden_states, top_k_index, top_k_weights, self.num_experts, gather=not in_place)
    execution_plan = self._prepare_expert_execution(routing_plan, "grouped_mm")
    if execution_plan.offsets is None:
        raise RuntimeError("GGUF LoRA requires grouped expert offsets.")
    selected = routing_plan.selected_hidden_states
    expert_indices, expert_offsets = execution_plan.expert_indices, execution_plan.offsets
    lw = lora_weights
    s = lw.scaling if lw is not None else 0.0
    # the four packed-weight calls of the step see one grouping: its row-tile tables are built once (the calls whose kernels
    # take another tile shape ignore them and build their own)
    tables = None
    if SHARE_GROUP_TABLES and (int(self.gate_proj.quant_type) == 12 or int(self.down_proj.quant_type) == 12):
        tables = build_group_tables(expert_indices, expert_offsets, tokens * top_k, self.num_experts)

    if in_place:
        gate, up = _RoutedGroupedLoraProjection.apply(
            compute_hidden_states, routing_plan.permutation, routing_plan.inverse_permutation, top_k, _as_payload(self.gate_proj),
            _as_payload(self.up_proj), expert_indices, expert_offsets, int(self.gate_proj.quant_type), self.intermediate_dim,
            lw.gate_up_a if lw else None, lw.gate_up_b if lw else None, s, tables)
    else:
        gate, up = _GroupedLoraProjection.apply(
            selected, _as_payload(self.gate_proj), _as_payload(self.up_proj), expert_indices, expert_offsets,
            int(self.gate_proj.quant_type), self.intermediate_dim, lw.gate_up_a if lw else None, lw.gate_up_b if lw else None, s, tables)
    if (FUSE_GATED_DOWN_COMBINE and execution_plan.output_mask is None and type(self)._apply_split_gate is GGUFExperts._apply_split_gate
            and routing_plan.routing_weights.is_contiguous()):
        combined = _RoutedGatedDownProjection.apply(
            gate, up, self.swiglu_limit, _as_payload(self.down_proj), expert_indices, expert_offsets, int(self.down_proj.quant_type),
            self.hidden_dim, lw.down_a if lw else None, lw.down_b if lw else None, s, routing_plan.routing_weights, routing_plan.permutation,
            routing_plan.inverse_permutation, tables)
        return combined.to(hidden_states.dtype).reshape(hidden_states.shape)
    intermediate = self._apply_split_gate(gate, up)
    output = _GroupedLoraProjection.apply(
        intermediate, _as_payload(self.down_proj), None, expert_indices, expert_offsets, int(self.down_proj.quant_type),
        self.hidden_dim, lw.down_a if lw else None, lw.down_b if lw else None, s, tables)
    return finalize_expert_routing(output, hidden_states, routing_plan, execution_plan.output_mask).reshape(hidden_states.shape)


ALL_GGUF_EXPERTS_FUNCTIONS[EXPERTS_IMPLEMENTATION] = qwen3_5_moe_gguf_mmq_lora_forward


# ------------------------------------------------------------------------------------------------
def _dequantize_selected_experts(weight: Any, expert_indices: torch.Tensor, dtype: torch.dtype, device: torch.device) -> torch.Tensor:
    """Dense [G, N, K] planes of the selected experts (fast_moe_lora.py:154-172): packed planes are decoded, floating-point
    ones copied; anything else is an error."""
    if isinstance(weight, GGUFQuantizedTensor):
        payload = weight.as_subclass(torch.Tensor)
        selected = payload.index_select(0, expert_indices.to(payload.device))
        return dequantize_gguf_tensor(selected, weight.quant_type, dtype=dtype, device=device)
    if not weight.is_floating_point():
        raise RuntimeError("GGUF expert weights must be packed or floating point before grouped execution.")
    return weight.index_select(0, expert_indices.to(weight.device)).to(device=device, dtype=dtype)


class _UnpackedExpertProjection(torch.autograd.Function):
    """The branch of the reference's ``_AiterGGUFExpertProjection`` for weights without a packed kernel
    (fast_moe_lora.py:230-247, 264-287): decode or copy the selected experts' planes, then ``gmm``; the input's gradient is a
    ``gmm`` against the same planes, which are decoded again instead of being kept.  The weights get no gradient."""

    @staticmethod
    def forward(ctx, hidden_states, weight, expert_indices, group_sizes, compute_dtype):
        if weight.requires_grad:
            raise RuntimeError("Fast GGUF expert execution requires frozen packed base weights.")
        if compute_dtype != torch.bfloat16:
            raise RuntimeError("Grouped expert execution requires BF16 compute dtype.")
        ctx.input_dtype = hidden_states.dtype
        ctx.compute_dtype = compute_dtype
        hidden_states = hidden_states.to(compute_dtype).contiguous()
        dense = _dequantize_selected_experts(weight, expert_indices, compute_dtype, hidden_states.device)
        ctx.weight = weight
        ctx.save_for_backward(expert_indices, group_sizes)
        return gmm(hidden_states, dense.transpose(1, 2), group_sizes, preferred_element_type=compute_dtype)

    @staticmethod
    def backward(ctx, grad_output):
        grad_hidden = None
        if ctx.needs_input_grad[0]:
            expert_indices, group_sizes = ctx.saved_tensors
            dense = _dequantize_selected_experts(ctx.weight, expert_indices, ctx.compute_dtype, grad_output.device)
            grad_hidden = gmm(grad_output.contiguous(), dense, group_sizes, preferred_element_type=ctx.compute_dtype).to(ctx.input_dtype)
        return grad_hidden, None, None, None, None


def _base_grouped_linear(hidden_states, weight, expert_indices, expert_offsets, group_sizes, compute_dtype):
    """One frozen expert projection (fast_moe_lora.py:175-288): the packed kernel where the block format has one."""
    if isinstance(weight, GGUFQuantizedTensor) and supports_native_mmq(weight):
        if compute_dtype != torch.bfloat16:
            raise RuntimeError("Grouped GGUF MMQ requires BF16 compute dtype.")
        return grouped_mmq(hidden_states, weight, expert_indices, expert_offsets, int(weight.quant_type), int(weight.logical_shape[-2]))
    return _UnpackedExpertProjection.apply(hidden_states, weight, expert_indices, group_sizes, compute_dtype)


def _base_grouped_pair(hidden_states, first_weight, second_weight, expert_indices, expert_offsets, group_sizes, compute_dtype):
    """The gate/up pair (fast_moe_lora.py:291-395): one paired packed launch where both halves share a native block format,
    two single projections otherwise."""
    packed = [isinstance(w, GGUFQuantizedTensor) and supports_native_mmq(w) for w in (first_weight, second_weight)]
    if all(packed) and first_weight.quant_type == second_weight.quant_type:
        if tuple(first_weight.logical_shape) != tuple(second_weight.logical_shape):
            raise RuntimeError("Paired grouped GGUF MMQ requires matching logical shapes.")
        if compute_dtype != torch.bfloat16:
            raise RuntimeError("Grouped GGUF MMQ requires BF16 compute dtype.")
        return grouped_mmq_pair(hidden_states, first_weight, second_weight, expert_indices, expert_offsets, int(first_weight.quant_type),
                                int(first_weight.logical_shape[-2]))
    return (_base_grouped_linear(hidden_states, first_weight, expert_indices, expert_offsets, group_sizes, compute_dtype),
            _base_grouped_linear(hidden_states, second_weight, expert_indices, expert_offsets, group_sizes, compute_dtype))


def qwen3_5_moe_gguf_mmq_aiter_lora_forward(self: GGUFExperts, hidden_states: torch.Tensor, top_k_index: torch.Tensor,
                                            top_k_weights: torch.Tensor, lora_weights: _ExpertLoraWeights | None = None) -> torch.Tensor:
    """The expert FFN in the reference's own order (fast_moe_lora.py:685-770): base projections, then each LoRA delta as two
    grouped products (``lora_grouped_linear``) added with ``alpha=scaling``; every intermediate is a bf16 tensor of its own.
    Slower than ``qwen3_5_moe_gguf_mmq_lora_forward`` (which folds the deltas into the packed-weight launches), but it also
    takes expert weights that are plain floating-point tensors."""
    if not isinstance(self, GGUFExperts):
        raise TypeError(f"{SEPARATED_EXPERTS_IMPLEMENTATION} requires GGUFExperts, got {type(self).__name__}.")
    if self.projection_layout != "split_gate_up" or self.has_bias or not self.has_gate:
        raise RuntimeError("The GGUF LoRA path requires split, bias-free gate/up expert projections.")
    compute_hidden_states = self._prepare_expert_hidden_states(hidden_states)
    routing_plan = prepare_expert_routing(compute_hidden_states, top_k_index, top_k_weights, self.num_experts)
    execution_plan = self._prepare_expert_execution(routing_plan, "grouped_mm")
    if execution_plan.offsets is None:
        raise RuntimeError("GGUF LoRA requires grouped expert offsets.")
    selected = routing_plan.selected_hidden_states
    expert_indices = execution_plan.expert_indices.to(device=selected.device, dtype=torch.long).contiguous()
    expert_offsets = execution_plan.offsets.to(device=selected.device, dtype=torch.int32).contiguous()
    group_sizes = _group_sizes_from_offsets(expert_offsets)

    gate, up = _base_grouped_pair(selected, self.gate_proj, self.up_proj, expert_indices, expert_offsets, group_sizes, self.compute_dtype)
    lw = lora_weights
    if lw is not None:
        lora_group_sizes = _complete_group_sizes(group_sizes, expert_indices, self.num_experts)
        gate_delta, up_delta = lora_grouped_linear(selected, lw.gate_up_a, lw.gate_up_b, lora_group_sizes).chunk(2, dim=-1)
        gate = torch.add(gate, gate_delta, alpha=lw.scaling)
        up = torch.add(up, up_delta, alpha=lw.scaling)
    intermediate = self._apply_split_gate(gate.contiguous(), up.contiguous())
    output = _base_grouped_linear(intermediate, self.down_proj, expert_indices, expert_offsets, group_sizes, self.compute_dtype)
    if lw is not None:
        output = torch.add(output, lora_grouped_linear(intermediate, lw.down_a, lw.down_b, lora_group_sizes), alpha=lw.scaling)
    return finalize_expert_routing(output, hidden_states, routing_plan, execution_plan.output_mask).reshape(hidden_states.shape)


ALL_GGUF_EXPERTS_FUNCTIONS[SEPARATED_EXPERTS_IMPLEMENTATION] = qwen3_5_moe_gguf_mmq_aiter_lora_forward


def set_gguf_experts_implementation(model: torch.nn.Module, name: str, experts_type: type = GGUFExperts) -> list[str]:
    """Points every packed expert module of ``model`` at a registered forward (what the fork's
    ``model.set_experts_implementation`` does for its GGUF expert modules, fast_moe_lora.py:800).  The model's own method is
    called too when it has one and knows the name; stock transformers knows only its own registry and refuses others, which
    is not an error here.  Returns the module paths."""
    if name not in ALL_GGUF_EXPERTS_FUNCTIONS:
        raise ValueError(f"experts implementation {name!r} is not registered")
    setter = getattr(model, "set_experts_implementation", None)
    if callable(setter):
        try:
            setter(name)
        except ValueError:
            pass
    paths = []
    for path, module in model.named_modules():
        if isinstance(module, experts_type):
            module.experts_implementation = name
            paths.append(path)
    return paths


def _register_expert_wrapper(lora_config, model: torch.nn.Module, name: str, forward, experts_type: type, wrapper: type, what: str,
                             exact_pattern: str | None = None):
    register = getattr(lora_config, "_register_custom_module", None)
    if register is None:
        raise RuntimeError("This PEFT version has no LoraConfig._register_custom_module API. "
                           f"Cannot install {what} without a global PEFT monkey patch.")
    if getattr(lora_config, "target_parameters", None):
        raise ValueError("Persistent GGUF expert LoRA targets the complete 'experts' module, not target_parameters.")
    if isinstance(lora_config.target_modules, str):
        if exact_pattern is None:
            raise TypeError(f"{what} requires an explicit target_modules collection, not a regex string.")
        if lora_config.target_modules != exact_pattern:
            raise ValueError("DeepSeek V4 LoRA uses one exact indexer-excluding target pattern.")
    else:
        target_modules = set(lora_config.target_modules or ())
        target_modules.add("experts")
        lora_config.__dict__["target_modules"] = target_modules
    ALL_GGUF_EXPERTS_FUNCTIONS[name] = forward
    set_gguf_experts_implementation(model, name, experts_type)
    register({experts_type: wrapper})
    return lora_config


def register_fast_moe_lora(lora_config, model: torch.nn.Module):
    """Registers the packed expert forward process-wide and the expert LoRA wrapper on one config
    (fast_moe_lora.py:773-802): "experts" joins ``target_modules``, every ``GGUFExperts`` of ``model`` is pointed at
    ``EXPERTS_IMPLEMENTATION``, and the config maps ``GGUFExperts`` to ``FastGGUFMoeLora``."""
    return _register_expert_wrapper(lora_config, model, EXPERTS_IMPLEMENTATION, qwen3_5_moe_gguf_mmq_lora_forward, GGUFExperts,
                                    FastGGUFMoeLora, "fast GGUF MoE LoRA")


class _ExpertFactor(torch.nn.Module):
    """One expert factor family as a module with a ``weight`` (fast_moe_lora.py:463-470), so adapter checkpoints carry the
    reference's key names (``...lora_A_down.<adapter>.weight``)."""

    def __init__(self, shape: tuple[int, ...], *, device, dtype):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.empty(shape, device=device, dtype=dtype))


class FastGGUFMoeLora(torch.nn.Module):
    """LoRA wrapper owning the four factor families of one packed ``GGUFExperts`` module
    (counterpart of fast_moe_lora.py:482-646; same parameter names and shapes)."""

    adapter_layer_names = ("lora_A", "lora_B", "lora_A_down", "lora_B_down")

    def __init__(self, base_layer: GGUFExperts, adapter_name: str = "default", *, r: int, lora_alpha: float, config: Any = None,
                 **kwargs: Any):
        super().__init__()
        from .peft_compat import adapter_options

        opts = adapter_options(config, kwargs, ("lora_dropout", "use_rslora", "use_dora", "lora_bias", "init_lora_weights",
                                                "alora_invocation_tokens"))
        use_rslora, init_lora_weights = opts["use_rslora"], opts["init_lora_weights"]
        if not isinstance(base_layer, GGUFExperts):
            raise TypeError(f"Fast GGUF MoE LoRA requires GGUFExperts, got {type(base_layer).__name__}.")
        if r <= 0 or r > 64:
            raise ValueError(f"LoRA rank must be in 1..64, got {r}.")
        if float(opts["lora_dropout"]) != 0.0:
            raise ValueError("Fast GGUF MoE LoRA currently requires lora_dropout=0.")
        if opts["lora_bias"]:
            raise ValueError("Fast GGUF MoE LoRA does not support LoRA bias.")
        if opts["use_dora"] or opts["alora_invocation_tokens"] is not None:
            raise ValueError("Fast GGUF MoE LoRA does not support DoRA or aLoRA variants.")
        self.base_layer = base_layer
        e, h, i = base_layer.num_experts, base_layer.hidden_dim, base_layer.intermediate_dim
        dev, dt = base_layer.gate_proj.device, base_layer.compute_dtype

        def factor(shape):
            return _ExpertFactor(shape, device=dev, dtype=dt)

        self.lora_A = torch.nn.ModuleDict({adapter_name: factor((e, r, h))})
        self.lora_B = torch.nn.ModuleDict({adapter_name: factor((e, 2 * i, r))})
        self.lora_A_down = torch.nn.ModuleDict({adapter_name: factor((e, r, i))})
        self.lora_B_down = torch.nn.ModuleDict({adapter_name: factor((e, h, r))})
        self.scaling = {adapter_name: lora_alpha / (math.sqrt(r) if use_rslora else r)}
        self.active_adapter = adapter_name
        self.disable_adapters = False
        if init_lora_weights is True:
            torch.nn.init.kaiming_uniform_(self.lora_A[adapter_name].weight, a=math.sqrt(5))
            torch.nn.init.kaiming_uniform_(self.lora_A_down[adapter_name].weight, a=math.sqrt(5))
        elif init_lora_weights == "gaussian":
            torch.nn.init.normal_(self.lora_A[adapter_name].weight, std=1 / r)
            torch.nn.init.normal_(self.lora_A_down[adapter_name].weight, std=1 / r)
        elif init_lora_weights is not False:
            raise ValueError(f"Fast GGUF MoE LoRA does not support init_lora_weights={init_lora_weights!r}.")
        if init_lora_weights is not False:
            torch.nn.init.zeros_(self.lora_B[adapter_name].weight)
            torch.nn.init.zeros_(self.lora_B_down[adapter_name].weight)

    def get_base_layer(self) -> torch.nn.Module:
        return self.base_layer

    def _active_lora_weights(self) -> _ExpertLoraWeights | None:
        if self.disable_adapters:
            return None
        n = self.active_adapter
        return _ExpertLoraWeights(self.lora_A[n].weight, self.lora_B[n].weight, self.lora_A_down[n].weight, self.lora_B_down[n].weight, float(self.scaling[n]))

    def forward(self, hidden_states: torch.Tensor, top_k_index: torch.Tensor, top_k_weights: torch.Tensor) -> torch.Tensor:
        return self.base_layer(hidden_states, top_k_index, top_k_weights, self._active_lora_weights())

    def merge(self, *args: Any, **kwargs: Any) -> None:
        raise RuntimeError("GGUF expert LoRA adapters cannot be merged into packed base weights.")

    def unmerge(self) -> None:
        raise RuntimeError("GGUF expert LoRA adapters cannot be unmerged because merging is unsupported.")

    def get_delta_weight(self, *args: Any, **kwargs: Any) -> torch.Tensor:
        raise RuntimeError("GGUF expert LoRA does not materialize a full expert delta weight.")
