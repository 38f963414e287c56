"""ctypes binding of oracle/ggml_dequant.c (test infrastructure; see that file's header)."""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

from .gguf_blocks import IQ2_XXS, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, Q8_0, QUANT_SIZES
from .iq2xxs_grid import IQ2XXS_GRID

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "_build" / "libggml_oracle.so"
_lib = None


def build(force: bool = False) -> Path:
    if force or not _LIB_PATH.exists() or _LIB_PATH.stat().st_mtime < (_HERE / "ggml_dequant.c").stat().st_mtime:
        subprocess.run(["make", "-C", str(_HERE), "-B" if force else "-s"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(str(_LIB_PATH))
    return _lib


def dequantize(payload: np.ndarray, qt: int) -> np.ndarray:
    """uint8 [..., row_bytes] -> float32 [..., K] through the scalar C loops."""
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    elems, nbytes = QUANT_SIZES[qt]
    nb = payload.size // nbytes
    out = np.empty(nb * elems, dtype=np.float32)
    src = payload.ctypes.data_as(ctypes.c_void_p)
    dst = out.ctypes.data_as(ctypes.c_void_p)
    L = lib()
    if qt == Q8_0:
        L.oracle_dequant_q8_0(src, ctypes.c_int64(nb), dst)
    elif qt == Q4_K:
        L.oracle_dequant_q4_k(src, ctypes.c_int64(nb), dst)
    elif qt == Q6_K:
        L.oracle_dequant_q6_k(src, ctypes.c_int64(nb), dst)
    elif qt == Q5_K:
        L.oracle_dequant_q5_k(src, ctypes.c_int64(nb), dst)
    elif qt == Q2_K:
        L.oracle_dequant_q2_k(src, ctypes.c_int64(nb), dst)
    elif qt == Q3_K:
        L.oracle_dequant_q3_k(src, ctypes.c_int64(nb), dst)
    elif qt == IQ2_XXS:
        grid = np.array(IQ2XXS_GRID, dtype=np.uint64)
        L.oracle_dequant_iq2_xxs(src, ctypes.c_int64(nb), grid.ctypes.data_as(ctypes.c_void_p), dst)
    else:
        raise ValueError(f"unsupported GGML type {qt}")
    return out.reshape(*payload.shape[:-1], payload.shape[-1] // nbytes * elems)


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().oracle_f32_to_bf16(x.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(x.size), out.ctypes.data_as(ctypes.c_void_p))
    return out
