"""CPU oracle for the dense and grouped LoRA matmul: dequantize, then framework matmul.

TEST INFRASTRUCTURE (see oracle/__init__.py).  Restates the relations the reference's own tests use
as their oracle:

* dense: ``linear(x, dequant_bf16(W))`` + ``matmul(x, A^T)`` + ``addmm(base, xA, B^T, alpha=s)`` and
  autograd through them (test_fast_lora.py:110-128; forward surface fast_lora.py:34-65,134-163);
* grouped: the per-group loop ``dY[r0:r1].float() @ W[g].float()`` (test_fast_moe_lora.py:106-130,
  test_deepseek_v4_moe_lora.py:108-115) and, for a gate/up pair, both products summed in one fp32
  accumulator and rounded once (test_fast_moe_lora.py:199-203);
* the expert layer: fast_moe_lora.py:685-770 (gate/up pair, LoRA delta added with ``alpha=s``,
  SiLU(gate)*up, down projection + LoRA delta).

Arithmetic is float64 on values that are exactly representable (bf16 inputs, bf16-rounded decoded
weights); the only intermediate roundings kept are the ones every implementation of the path shares:
x_A = x A^T and t = dY B are rounded to bf16 before their second product (fast_lora.py:50-61).
Everything is closed-form matrix algebra; the gradient formulas are checked against torch autograd
in tests/test_oracle_matmul.py.
"""

from __future__ import annotations

import numpy as np
import torch

from . import gguf_blocks as gb


def bf16_round(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.float32).to(torch.bfloat16).to(torch.float64)


def weights_bf16(payload: np.ndarray, qt: int) -> torch.Tensor:
    """Packed rows -> float64 tensor holding the bf16-rounded decoded weights [..., N, K]."""
    return torch.from_numpy(gb.dequantize_bf16(payload, qt)).to(torch.float64)


def lora_linear(x, w, a=None, b=None, s=1.0, dy=None, row_weight=None):
    """x [M,K] bf16, w [N,K] float64 (bf16 values), a [r,K], b [N,r] bf16, dy [M,N] bf16.
    Returns dict(y, xa, dx, da, db) in float64 (xa holds bf16 values).
    ``row_weight`` [M] float64: row i's cotangent is row_weight[i] * dy[i] without that product being stored (the order of
    the backward that folds the expert combine into the down projection): dx stays UNWEIGHTED, the factor gradients carry the
    weight on their rank-r operand, which is rounded to bf16 again."""
    x64 = x.to(torch.float64)
    out = {"y": x64 @ w.T}
    if a is not None:
        a64, b64 = a.to(torch.float64), b.to(torch.float64)
        xa = bf16_round(x64 @ a64.T)
        out["xa"] = xa
        out["y"] = out["y"] + s * (xa @ b64.T)
    if dy is not None:
        dy64 = dy.to(torch.float64)
        out["dx"] = dy64 @ w
        if a is not None:
            t = bf16_round(dy64 @ b64)
            out["dx"] = out["dx"] + s * (t @ a64)
            xa_b = out["xa"]
            if row_weight is not None:
                t, xa_b = bf16_round(t * row_weight[:, None]), bf16_round(xa_b * row_weight[:, None])
            out["da"] = s * (t.T @ x64)
            out["db"] = s * (dy64.T @ xa_b)
    return out


def group_bounds(offsets) -> list[tuple[int, int]]:
    """Cumulative END offsets (test_fast_moe_lora.py:136-137: offsets [2,5,6]) -> [(r0, r1), ...]."""
    ends = [int(v) for v in offsets]
    return list(zip([0] + ends[:-1], ends))


def grouped_lora_linear(x, w_all, experts, offsets, a_all=None, b_all=None, s=1.0, dy=None, row_weight=None):
    """Per-group loop of :func:`lora_linear`.  w_all [E,N,K] float64, a_all [E,r,K], b_all [E,N,r].
    experts: active expert ids; offsets: cumulative ends.  Factor gradients cover all E planes and are
    zero for inactive experts (test_fast_moe_lora.py:331-333)."""
    m = x.shape[0]
    n = w_all.shape[1]
    res = {"y": torch.zeros(m, n, dtype=torch.float64)}
    if dy is not None:
        res["dx"] = torch.zeros(m, x.shape[1], dtype=torch.float64)
    if a_all is not None:
        res["xa"] = torch.zeros(m, a_all.shape[1], dtype=torch.float64)
        if dy is not None:
            res["da"] = torch.zeros(a_all.shape, dtype=torch.float64)
            res["db"] = torch.zeros(b_all.shape, dtype=torch.float64)
    for e, (r0, r1) in zip([int(v) for v in experts], group_bounds(offsets)):
        if r1 == r0:
            continue
        part = lora_linear(
            x[r0:r1], w_all[e],
            None if a_all is None else a_all[e], None if b_all is None else b_all[e], s,
            None if dy is None else dy[r0:r1],
            None if row_weight is None else row_weight[r0:r1],
        )
        res["y"][r0:r1] = part["y"]
        if "xa" in part:
            res["xa"][r0:r1] = part["xa"]
        if dy is not None:
            res["dx"][r0:r1] = part["dx"]
            if a_all is not None:
                res["da"][e] = part["da"]
                res["db"][e] = part["db"]
    return res


def silu_mul(gate: torch.Tensor, up: torch.Tensor, limit: float | None = None) -> torch.Tensor:
    """silu(gate) * up; with ``limit`` the DeepSeek form act(gate.clamp(max=limit)) * up.clamp(-limit, limit)
    (the expression test_deepseek_v4_moe_lora.py:194-196 compares the module with)."""
    if limit is not None:
        gate, up = gate.clamp(max=limit), up.clamp(min=-limit, max=limit)
    return gate * torch.sigmoid(gate) * up


def expert_layer(x_sorted, experts, offsets, wg, wu, wd, a_gu, b_gu, a_d, b_d, s, dy=None, row_weight=None, limit=None):
    """Expert-sorted rows through gate/up -> SiLU*up -> down with LoRA on both projections
    (fast_moe_lora.py:722-763).  wg, wu [E,I,H]; wd [E,H,I]; a_gu [E,r,H]; b_gu [E,2I,r];
    a_d [E,r,I]; b_d [E,H,r].  Intermediates are rounded to bf16 where the path stores them
    (gate, up, h).  Returns float64 tensors.
    With ``row_weight`` [rows] (the routing weight of each sorted row) ``dy`` is the UNWEIGHTED cotangent of the down
    projection's rows: its grad-input is rounded to bf16 unweighted ("dh_unweighted"), the activation's backward runs on
    row_weight * that, and "dw" = <dh_unweighted, h> per row is the routing weight's gradient (the same number as
    <dy, out> of the row, by associativity).  ``limit``: the clamped activation (no gradient into a clamped input)."""
    inter = wg.shape[1]
    w_gu = torch.cat([wg, wu], dim=1)
    gu = grouped_lora_linear(x_sorted, w_gu, experts, offsets, a_gu, b_gu, s)
    gate = bf16_round(gu["y"][:, :inter])
    up = bf16_round(gu["y"][:, inter:])
    h = bf16_round(silu_mul(gate, up, limit))
    h_bf = h.to(torch.bfloat16)
    dn = grouped_lora_linear(h_bf, wd, experts, offsets, a_d, b_d, s, dy, row_weight)
    res = {"gate": gate, "up": up, "h": h, "out": dn["y"]}
    if dy is None:
        return res
    dh = bf16_round(dn["dx"])
    if row_weight is not None:
        res["dh_unweighted"], res["dw"] = dh, (dh * h).sum(dim=1)
        dh = dh * row_weight[:, None]
    gc, uc = (gate, up) if limit is None else (gate.clamp(max=limit), up.clamp(min=-limit, max=limit))
    sig = torch.sigmoid(gc)
    dgate = bf16_round(dh * uc * (sig * (1 + gc * (1 - sig))))
    dup = bf16_round(dh * gc * sig)
    if limit is not None:
        dgate = torch.where(gate <= limit, dgate, torch.zeros_like(dgate))
        dup = torch.where((up >= -limit) & (up <= limit), dup, torch.zeros_like(dup))
    dgu = torch.cat([dgate, dup], dim=1).to(torch.bfloat16)
    back = grouped_lora_linear(x_sorted, w_gu, experts, offsets, a_gu, b_gu, s, dgu)
    res.update(dh=dh, dgate=dgate, dup=dup, dx=back["dx"], da_gu=back["da"], db_gu=back["db"],
               da_d=dn["da"], db_d=dn["db"])
    return res


def grouped_mm(lhs, rhs, group_sizes, dy=None):
    """The grouped product the reference takes from AITER (``gmm``, fast_moe_lora.py:42-52) and its two gradients (``gmm``
    against the transposed planes, :55-68; ``ptgmm``, :71-87), as the per-group loop the reference's tests use
    (test_fast_moe_lora.py:106-130).  lhs [M,K], rhs [E,K,N], group_sizes [E] (consecutive row groups; rows no group covers
    give zero rows and take no part in any gradient), dy [M,N].  float64; returns dict(out, dlhs, drhs)."""
    lhs64, rhs64 = lhs.to(torch.float64), rhs.to(torch.float64)
    m, n = lhs64.shape[0], rhs64.shape[2]
    out = {"out": torch.zeros((m, n), dtype=torch.float64)}
    if dy is not None:
        dy64 = dy.to(torch.float64)
        out["dlhs"] = torch.zeros_like(lhs64)
        out["drhs"] = torch.zeros_like(rhs64)
    r0 = 0
    for e, size in enumerate(int(v) for v in group_sizes):
        r1 = min(m, r0 + max(size, 0))
        out["out"][r0:r1] = lhs64[r0:r1] @ rhs64[e]
        if dy is not None:
            out["dlhs"][r0:r1] = dy64[r0:r1] @ rhs64[e].T
            out["drhs"][e] = lhs64[r0:r1].T @ dy64[r0:r1]
        r0 = r1
    return out
