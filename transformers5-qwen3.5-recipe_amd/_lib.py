"""ctypes binding of libggml_mmq_gfx950.so (the C ABI declared in include/ggml_mmq_gfx950.h).

The library is the only implementation of the hot path: there is no CPU or framework fallback, and
loading fails loudly when the shared object has not been built (``python -c "import __graft_entry__
as g; g.build()"`` or ``make -C <package>/csrc``).
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from pathlib import Path

import torch

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libggml_mmq_gfx950.so"
_lib: ctypes.CDLL | None = None

_P, _I, _L, _F = c_void_p, c_int, c_int64, c_float

# name -> (restype, argtypes); must list every symbol include/ggml_mmq_gfx950.h declares.
SIGNATURES: dict[str, tuple] = {
    "ggq_last_error": (c_char_p, []),
    "ggq_profile_begin": (_I, []),
    "ggq_profile_end": (_I, [_P, _P, _P, _P, _P, _I]),
    "ggq_set_factor_gradient_overlap": (_I, [_I]),
    "ggq_measure_mfma_ceiling": (_I, [_P, _P, _L, _I, _P, _P, _P]),
    "ggq_debug_force_grouped_shape": (_I, [_I]),
    "ggq_supports_quant_type": (_I, [_I]),
    "ggq_row_bytes": (_L, [_I, _L]),
    "ggq_dequantize": (_I, [_I, _P, _L, _L, _P, _I, _P]),
    "ggq_mmq": (_I, [_P, _P, _I, _L, _L, _L, _P, _P]),
    "ggq_mmq_grad_input": (_I, [_P, _P, _I, _L, _L, _L, _P, _P]),
    "ggq_fixed_grouped_mmq": (_I, [_P, _P, _I, _L, _I, _L, _L, _P, _P]),
    "ggq_fixed_grouped_mmq_grad_input": (_I, [_P, _P, _I, _L, _I, _L, _L, _P, _P]),
    "ggq_lora_workspace_bytes": (_L, [_L, _L, _L, _L, _L, _I]),
    "ggq_lora_mmq_forward": (_I, [_P, _P, _I, _L, _L, _L, _P, _P, _I, _F, _P, _P, _P, _L, _P]),
    "ggq_lora_mmq_backward": (_I, [_P, _P, _I, _L, _L, _L, _P, _P, _P, _P, _I, _F, _P, _P, _P, _P, _L, _P]),
    "ggq_grouped_lora_mmq_forward": (_I, [_P, _P, _P, _P, _P, _L, _L, _I, _L, _L, _L, _P, _P, _I, _F, _P, _P, _P, _P, _P, _L, _P]),
    "ggq_grouped_lora_mmq_backward": (_I, [_P, _P, _P, _P, _P, _P, _L, _L, _I, _L, _L, _L, _P, _P, _P, _P, _I, _F, _P, _P, _P, _P, _P, _L, _P]),
    "ggq_group_tables_bytes": (_L, [_L, _L, _L]),
    "ggq_group_tables_build": (_I, [_P, _P, _L, _L, _L, _P, _L, _P]),
    "ggq_grouped_forward_reads_indexed_rows": (_I, [_I, _L, _L, _L, _L]),
    "ggq_grouped_lora_mmq_forward_indexed": (_I, [_P, _L, _P, _I, _P, _P, _P, _P, _L, _L, _I, _L, _L, _L, _P, _P, _I, _F, _P, _P, _P, _P, _P, _L, _P]),
    "ggq_grouped_lora_mmq_backward_indexed": (_I, [_P, _P, _P, _P, _P, _P, _L, _L, _I, _L, _L, _L, _P, _L, _P, _I, _P, _P, _P, _I, _F, _P, _P, _P, _P, _P, _L, _P]),
    "ggq_route_plan_workspace_bytes": (_L, [_L, _I, _I]),
    "ggq_route_plan": (_I, [_P, _I, _L, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _P]),
    "ggq_route_plan_static": (_I, [_P, _I, _L, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P]),
    "ggq_route_gather_forward": (_I, [_P, _P, _P, _L, _I, _I, _P]),
    "ggq_route_gather_backward": (_I, [_P, _P, _P, _L, _I, _I, _P]),
    "ggq_route_combine_forward": (_I, [_P, _P, _I, _P, _P, _L, _I, _I, _P]),
    "ggq_route_combine_backward": (_I, [_P, _P, _I, _P, _P, _P, _P, _L, _I, _I, _P]),
    "ggq_router_topk": (_I, [_P, _I, _L, _I, _I, _P, _I, _P, _P, _I, _F, _P]),
    "ggq_swiglu_forward": (_I, [_P, _P, _P, _L, _P]),
    "ggq_swiglu_backward": (_I, [_P, _P, _P, _P, _P, _L, _P]),
    "ggq_swiglu_clamped_forward": (_I, [_P, _P, _P, _L, _F, _P]),
    "ggq_swiglu_clamped_backward": (_I, [_P, _P, _P, _P, _P, _L, _F, _P]),
    "ggq_swiglu_backward_routed": (_I, [_P, _P, _P, _P, _I, _P, _P, _P, _P, _L, _I, _F, _P]),
    "ggq_grouped_lora_mmq_backward_routed_output": (_I, [_P, _L, _P, _I, _P, _I, _P, _P, _P, _L, _L, _I, _L, _L, _L, _P, _P, _P, _P, _I, _F, _P, _P, _P,
                                                         _P, _P, _L, _P]),
    "ggq_gmm_workspace_bytes": (_L, [_L]),
    "ggq_gmm": (_I, [_P, _P, _P, _P, _L, _L, _L, _L, _I, _I, _P, _L, _P]),
    "ggq_ptgmm": (_I, [_P, _P, _P, _P, _L, _L, _L, _L, _I, _P, _L, _P]),
    "ggq_lmhead_ce_workspace_bytes": (_L, [_L, _L, _L, _L]),
    "ggq_lmhead_cross_entropy": (_I, [_I, _P, _P, _P, _L, _L, _L, _L, _L, _I, _P, _P, _P, _P, _P, _P, _P, _L, _P]),
}


def load() -> ctypes.CDLL:
    """Load the library once (after torch, so both share one HIP runtime)."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: the gfx950 kernels are not built and there is no fallback path. "
                "Run __graft_entry__.build() (or make -C transformers5-qwen3.5-recipe_amd/csrc)."
            )
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(rc: int, exc: type[Exception] = RuntimeError) -> None:
    if rc != 0:
        msg = load().ggq_last_error().decode(errors="replace")
        kinds = {-1: ValueError, -2: ValueError, -3: RuntimeError, -4: ValueError, -5: RuntimeError, -6: RuntimeError}
        raise kinds.get(rc, exc)(f"ggml_mmq_gfx950 error {rc}: {msg}")


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def stream_handle(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_device_tensor(t: torch.Tensor, name: str, dtype: torch.dtype | tuple | None = None) -> None:
    """Fail closed on operands the kernels cannot take as they are (the reference's ops reject wrong
    dtype / device / contiguity / storage offset instead of repairing them, docs/plan_qwen3.5.md:148)."""
    if t.device.type != "cuda":
        raise RuntimeError(f"{name} must live on a ROCm device, got {t.device}")
    if dtype is not None:
        allowed = dtype if isinstance(dtype, tuple) else (dtype,)
        if t.dtype not in allowed:
            raise TypeError(f"{name} must have dtype {allowed}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous (no hidden operand copies are made)")
    if t.data_ptr() % 16:
        raise ValueError(f"{name} must be 16-byte aligned (storage offset {t.storage_offset()})")
