"""Grouped bf16 matrix products over expert row groups: the two functions the reference imports from AITER
(``from aiter.ops.triton.gmm import gmm, ptgmm``, fast_moe_lora.py:22) and its autograd wrapper around them
(``_AiterGroupedMM`` / ``aiter_grouped_mm``, fast_moe_lora.py:90-151), on ``ggq_gmm`` / ``ggq_ptgmm`` of the HIP library.

The expert layer of this package does not go through these: its LoRA products run inside the fused packed-weight calls.
They exist for code written against the reference's surface (its ``_lora_grouped_linear``, fast_moe_lora.py:674-682, and its
projection of expert weights that have no packed kernel, :230-247, which ``expert_projection_without_packed_kernel`` in
``fast_moe_lora`` restates).  AITER itself is not importable where this package is tested, so ``gmm`` / ``ptgmm`` follow the
reference's call sites (argument order, the ``lhs.T`` convention of ``ptgmm``, ``preferred_element_type`` / ``config``
keywords) and its tests (test_fast_moe_lora.py:280-360), not AITER's source.  bf16 or fp16 (both operands alike), as the
reference's wrapper admits (fast_moe_lora.py:116-119).
"""

from __future__ import annotations

import importlib.util
import sys
import types

import torch

from . import _lib


_DTYPES = (torch.float16, torch.bfloat16)


def _require_device(t: torch.Tensor, name: str) -> None:
    if t.device.type != "cuda":
        raise RuntimeError(f"{name} must live on a ROCm device, got {t.device}")


def _workspace(device: torch.device, experts: int) -> torch.Tensor:
    return torch.empty(int(_lib.load().ggq_gmm_workspace_bytes(experts)), dtype=torch.uint8, device=device)


def _check_group_sizes(group_sizes: torch.Tensor, experts: int, device: torch.device) -> None:
    if group_sizes.ndim != 1 or group_sizes.numel() != experts:
        raise ValueError(f"group_sizes must be [{experts}], got {tuple(group_sizes.shape)}")
    if group_sizes.device != device:
        raise ValueError("group_sizes must share the lhs device.")
    if group_sizes.dtype != torch.int32 or group_sizes.stride() != (1,):
        raise ValueError("group_sizes must be contiguous int32.")


def gmm(lhs: torch.Tensor, rhs: torch.Tensor, group_sizes: torch.Tensor, preferred_element_type: torch.dtype | None = None,
        config=None) -> torch.Tensor:
    """``out[rows of e] = lhs[rows of e] @ rhs[e]``: lhs [M, K] row-major, rhs [E, K, N] with either of its last two
    strides equal to 1 (a contiguous [E, K, N] tensor or the ``.transpose(1, 2)`` of a contiguous [E, N, K] one), group_sizes
    [E] int32 on the device.  ``config`` (AITER's tile choice, moe_gmm_configs.py) is accepted and ignored."""
    _require_device(lhs, "gmm lhs")
    if lhs.dtype not in _DTYPES or rhs.dtype != lhs.dtype or rhs.device != lhs.device:
        raise TypeError(f"gmm requires matching FP16/BF16 inputs on one device, got {lhs.dtype} and {rhs.dtype}.")
    if preferred_element_type not in (None, lhs.dtype):
        raise TypeError(f"gmm writes its inputs' type {lhs.dtype}, got preferred_element_type={preferred_element_type}.")
    if lhs.ndim != 2 or rhs.ndim != 3 or lhs.shape[1] != rhs.shape[1]:
        raise ValueError(f"gmm expects lhs [M,K] and rhs [E,K,N], got {tuple(lhs.shape)} and {tuple(rhs.shape)}.")
    if lhs.stride() != (lhs.shape[1], 1) and lhs.numel() > 0:
        raise ValueError("gmm lhs must be row-major.")
    experts, k, n = rhs.shape
    m = lhs.shape[0]
    _check_group_sizes(group_sizes, experts, lhs.device)
    s0, s1, s2 = rhs.stride()
    planes_dense = experts == 1 or s0 == k * n  # (strides of size-1 dimensions carry no information)
    if rhs.numel() == 0 or planes_dense and (n == 1 or s2 == 1) and (k == 1 or s1 == n):
        k_contiguous = 0
    elif planes_dense and (k == 1 or s1 == 1) and (n == 1 or s2 == k):
        k_contiguous = 1  # [E, N, K] seen through transpose(1, 2)
    else:
        raise ValueError(f"gmm rhs must be a dense [E,K,N] tensor or the transpose(1, 2) of a dense [E,N,K] one, got strides {rhs.stride()}.")
    out = torch.empty((m, n), dtype=lhs.dtype, device=lhs.device)
    ws = _workspace(lhs.device, experts)
    lib, stream = _lib.load(), _lib.stream_handle(lhs.device)
    _lib.check(lib.ggq_gmm(lhs.data_ptr(), rhs.data_ptr(), group_sizes.data_ptr(), out.data_ptr(), m, k, n, experts, k_contiguous,
                           int(lhs.dtype == torch.float16), ws.data_ptr(), ws.numel(), stream))
    return out


def ptgmm(lhs: torch.Tensor, rhs: torch.Tensor, group_sizes: torch.Tensor, preferred_element_type: torch.dtype | None = None,
          config=None) -> torch.Tensor:
    """``out[e] = lhs[:, rows of e] @ rhs[rows of e]``: lhs [K, M] given as the ``.T`` of a row-major [M, K] matrix (the
    reference passes ``lhs.T``, fast_moe_lora.py:76-87), rhs [M, N] row-major.  Returns [E, K, N]; groups without rows get
    zeros."""
    _require_device(rhs, "ptgmm rhs")
    if lhs.dtype not in _DTYPES or rhs.dtype != lhs.dtype or lhs.device != rhs.device:
        raise TypeError(f"ptgmm requires matching FP16/BF16 inputs on one device, got {lhs.dtype} and {rhs.dtype}.")
    if preferred_element_type not in (None, lhs.dtype):
        raise TypeError(f"ptgmm writes its inputs' type {lhs.dtype}, got preferred_element_type={preferred_element_type}.")
    if lhs.ndim != 2 or rhs.ndim != 2 or lhs.shape[1] != rhs.shape[0]:
        raise ValueError(f"ptgmm expects lhs [K,M] and rhs [M,N], got {tuple(lhs.shape)} and {tuple(rhs.shape)}.")
    k, m = lhs.shape
    n = rhs.shape[1]
    if lhs.numel() > 0 and lhs.stride() != (1, k) and not (m == 1 and lhs.stride(0) == 1) and not (k == 1 and lhs.stride(1) == 1):
        raise ValueError("ptgmm lhs must be the transpose of a row-major [M,K] matrix.")
    if rhs.numel() > 0 and rhs.stride() != (n, 1):
        raise ValueError("ptgmm rhs must be row-major.")
    experts = group_sizes.numel()
    _check_group_sizes(group_sizes, experts, rhs.device)
    out = torch.empty((experts, k, n), dtype=rhs.dtype, device=rhs.device)
    ws = _workspace(rhs.device, experts)
    lib, stream = _lib.load(), _lib.stream_handle(rhs.device)
    _lib.check(lib.ggq_ptgmm(lhs.data_ptr(), rhs.data_ptr(), group_sizes.data_ptr(), out.data_ptr(), m, k, n, experts,
                             int(rhs.dtype == torch.float16), ws.data_ptr(), ws.numel(), stream))
    return out


class _AiterGroupedMM(torch.autograd.Function):
    """Autograd-capable ``(M,K) @ (E,K,N)`` grouped matrix multiplication (fast_moe_lora.py:90-141): the gradient of lhs is a
    ``gmm`` against ``rhs.transpose(1, 2)``, the gradient of rhs a ``ptgmm`` whose planes of groups without rows are zero."""

    @staticmethod
    def forward(ctx, lhs, rhs, group_sizes):
        if lhs.ndim != 2 or rhs.ndim != 3 or group_sizes.ndim != 1:
            raise ValueError("AITER grouped MM expects lhs [M,K], rhs [E,K,N], and group_sizes [E].")
        if lhs.shape[1] != rhs.shape[1]:
            raise ValueError(f"Grouped-MM K mismatch: lhs has {lhs.shape[1]}, rhs has {rhs.shape[1]}.")
        if rhs.shape[0] != group_sizes.numel():
            raise ValueError(f"Grouped-MM expert mismatch: rhs has {rhs.shape[0]}, group_sizes has {group_sizes.numel()}.")
        if lhs.dtype not in _DTYPES or rhs.dtype != lhs.dtype:
            raise TypeError(f"AITER grouped MM requires matching FP16/BF16 inputs, got {lhs.dtype} and {rhs.dtype}.")
        if lhs.stride() != (lhs.shape[1], 1):
            raise ValueError("AITER grouped MM lhs must be row-major.")
        if group_sizes.device != lhs.device:
            raise ValueError("AITER grouped MM group_sizes must share the lhs device.")
        if group_sizes.dtype != torch.int32 or group_sizes.stride() != (1,):
            raise ValueError("AITER grouped MM group_sizes must be contiguous int32.")
        ctx.save_for_backward(lhs, rhs, group_sizes)
        return gmm(lhs, rhs, group_sizes, preferred_element_type=lhs.dtype)

    @staticmethod
    def backward(ctx, grad_output):
        lhs, rhs, group_sizes = ctx.saved_tensors
        if grad_output.stride() != (grad_output.shape[1], 1):
            raise ValueError("AITER grouped MM output gradient must be row-major.")
        grad_lhs = gmm(grad_output, rhs.transpose(1, 2), group_sizes, preferred_element_type=grad_output.dtype) if ctx.needs_input_grad[0] else None
        grad_rhs = ptgmm(lhs.T, grad_output, group_sizes, preferred_element_type=lhs.dtype) if ctx.needs_input_grad[1] else None
        return grad_lhs, grad_rhs, None


def aiter_grouped_mm(lhs: torch.Tensor, rhs: torch.Tensor, group_sizes: torch.Tensor) -> torch.Tensor:
    """Apply the autograd-capable grouped matrix multiplication (fast_moe_lora.py:144-151)."""
    return _AiterGroupedMM.apply(lhs, rhs, group_sizes)


def lora_grouped_linear(hidden_states: torch.Tensor, lora_a: torch.Tensor, lora_b: torch.Tensor, group_sizes: torch.Tensor) -> torch.Tensor:
    """``(x @ A[e]^T) @ B[e]^T`` per group, unscaled: the reference's ``_lora_grouped_linear`` (fast_moe_lora.py:674-682) with
    A [E, r, K] and B [E, N, r]."""
    rank_states = aiter_grouped_mm(hidden_states, lora_a.transpose(1, 2), group_sizes)
    return aiter_grouped_mm(rank_states, lora_b.transpose(1, 2), group_sizes)


_AITER_GMM_MODULE = "aiter.ops.triton.gmm"


def install_as_aiter_gmm() -> None:
    """Makes ``from aiter.ops.triton.gmm import gmm, ptgmm`` (fast_moe_lora.py:22) resolve to the two functions above, for a
    process that keeps the reference's ``fast_moe_lora.py`` and has no AITER.  Refuses to shadow an AITER that is installed
    or already imported."""
    present = sys.modules.get(_AITER_GMM_MODULE)
    if present is not None:
        if getattr(present, "gmm", None) is gmm:
            return
        raise RuntimeError("a different aiter.ops.triton.gmm module is already imported")
    if "aiter" not in sys.modules and importlib.util.find_spec("aiter") is not None:
        raise RuntimeError("AITER is installed; its own gmm / ptgmm are not replaced")
    parent = None
    for depth, part in enumerate(_AITER_GMM_MODULE.split(".")):
        name = ".".join(_AITER_GMM_MODULE.split(".")[: depth + 1])
        module = sys.modules.get(name)
        if module is None:
            module = types.ModuleType(name)
            module.__path__ = []  # a package, so that the dotted import walks on
            sys.modules[name] = module
        if parent is not None:
            setattr(parent, part, module)
        parent = module
    parent.gmm, parent.ptgmm = gmm, ptgmm
