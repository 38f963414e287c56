"""Shared helpers for the parity tests: seeded synthetic operands and error measures."""

from __future__ import annotations

import numpy as np
import torch

from oracle import gguf_blocks as gb

ALL_TYPES = (gb.Q8_0, gb.Q2_K, gb.Q3_K, gb.Q4_K, gb.Q5_K, gb.Q6_K, gb.IQ2_XXS)
TYPE_NAMES = {gb.Q8_0: "Q8_0", gb.Q2_K: "Q2_K", gb.Q3_K: "Q3_K", gb.Q4_K: "Q4_K", gb.Q5_K: "Q5_K", gb.Q6_K: "Q6_K", gb.IQ2_XXS: "IQ2_XXS"}
# bf16 tolerance of the path (BASELINE: max rel err <= 2e-2)
MAX_REL = 2e-2


def make_payload(seed: int, qt: int, rows: int, k: int, kind: str = "quantized", std: float = 0.02) -> np.ndarray:
    """uint8 [rows, row_bytes]: either N(0, std^2) weights through the oracle's quantizer (BASELINE
    configs) or arbitrary bytes with sane scales (exercises every field encoding)."""
    rng = np.random.default_rng(seed)
    if kind == "random":
        return gb.random_payload(rng, qt, rows, k, std)
    w = (rng.standard_normal((rows, k)) * std).astype(np.float32)
    return gb.quantize(w, qt)


def bf16_randn(gen: torch.Generator, *shape, std: float = 1.0) -> torch.Tensor:
    return (torch.randn(*shape, generator=gen) * std).to(torch.bfloat16)


def max_rel(got: torch.Tensor, want: torch.Tensor) -> float:
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    denom = float(want.abs().max())
    if denom == 0.0:
        return float((got - want).abs().max())
    return float((got - want).abs().max()) / denom


def assert_close_bf16(got: torch.Tensor, want: torch.Tensor, what: str, max_rel_err: float = MAX_REL, ulps: float = 2.0) -> None:
    """Two bars: the path's headline tolerance (max |err| / max |ref| <= 2e-2) and, tighter, every
    element within a few bf16 ulps of the reference value plus accumulation noise scaled to the
    tensor's magnitude."""
    got64 = got.detach().double().cpu()
    want64 = want.detach().double().cpu()
    assert got64.shape == want64.shape, f"{what}: shape {tuple(got64.shape)} vs {tuple(want64.shape)}"
    assert torch.isfinite(got64).all(), f"{what}: non-finite values"
    rel = max_rel(got64, want64)
    assert rel <= max_rel_err, f"{what}: max rel err {rel:.3e} > {max_rel_err}"
    scale = float(want64.abs().max())
    tol = ulps * 2.0 ** -8 * want64.abs() + 2.0 ** -9 * scale
    bad = (got64 - want64).abs() > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} elements off by more than {ulps} bf16 ulps (worst {float(((got64 - want64).abs() / tol).max()):.2f}x)"


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
