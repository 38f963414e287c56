"""CPU-side checks of the boundary: the built library exports every symbol the C header declares, the
ctypes signature table covers the same set, the pure host helpers answer correctly, and the Python
mirror fails closed before any launch on operands the reference also rejects
(gguf_liger_loss.py:269-356, fast_moe_routing.py:350-377).  No kernel is launched here."""

import ctypes
import re
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import gguf_blocks as gb

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "ggml_mmq_gfx950.h"


def declared_symbols() -> list[str]:
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(ggq_\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for must in ("ggq_dequantize", "ggq_mmq", "ggq_mmq_grad_input", "ggq_lora_mmq_forward", "ggq_lora_mmq_backward",
                 "ggq_grouped_lora_mmq_forward", "ggq_grouped_lora_mmq_backward", "ggq_route_plan",
                 "ggq_route_gather_forward", "ggq_route_gather_backward", "ggq_route_combine_forward",
                 "ggq_route_combine_backward", "ggq_lmhead_cross_entropy", "ggq_last_error"):
        assert must in names
    assert len(names) >= 20


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg._lib.load()
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in {HEADER.name} but not exported"
    assert set(pkg._lib.SIGNATURES) == set(declared_symbols())


def declared_parameter_counts() -> dict[str, int]:
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    counts = {}
    for name, params in re.findall(r"\b(ggq_\w+)\s*\(([^)]*)\)\s*;", text):
        params = params.strip()
        counts[name] = 0 if params in ("", "void") else params.count(",") + 1
    return counts


def test_signature_table_has_the_arity_and_kinds_the_header_declares(pkg):
    """A ctypes table that is one argument short of the C declaration calls the function with garbage in that slot without
    any error: every entry has as many argument types as the header declares parameters, pointers where it declares pointers."""
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    counts = declared_parameter_counts()
    assert set(counts) == set(pkg._lib.SIGNATURES)
    for name, (restype, argtypes) in pkg._lib.SIGNATURES.items():
        assert len(argtypes) == counts[name], f"{name}: {len(argtypes)} argument types for {counts[name]} declared parameters"
        returns = re.search(r"([\w \*]+?)\s*\b" + name + r"\s*\(", text).group(1).strip()
        want_ret = ctypes.c_char_p if "char" in returns else ctypes.c_int64 if returns.endswith("int64_t") else ctypes.c_int
        assert restype is want_ret, f"{name} returns {returns!r}, the table says {restype}"
        params = re.search(r"\b" + name + r"\s*\(([^)]*)\)\s*;", text).group(1)
        if counts[name] == 0:
            continue
        for i, (decl, ctype) in enumerate(zip([p.strip() for p in params.split(",")], argtypes)):
            is_pointer = "*" in decl
            assert is_pointer == (ctype is ctypes.c_void_p), f"{name} parameter {i} ({decl!r}) against {ctype}"
            if not is_pointer:
                want = ctypes.c_float if decl.startswith("float") else ctypes.c_int64 if decl.startswith("int64_t") else ctypes.c_int
                assert ctype is want, f"{name} parameter {i} ({decl!r}) against {ctype}"


def test_host_only_helpers(pkg):
    lib = pkg._lib.load()
    for qt, (elems, nbytes) in gb.QUANT_SIZES.items():
        assert lib.ggq_supports_quant_type(qt) == 1
        assert lib.ggq_row_bytes(qt, 4 * elems) == 4 * nbytes
        assert lib.ggq_row_bytes(qt, elems + 1) == -1
        assert pkg.gguf.row_bytes(qt, 2 * elems) == 2 * nbytes
    for qt in (0, 2, 15, 99):  # F32, Q4_0, Q8_K: no kernels here
        assert lib.ggq_supports_quant_type(qt) == 0
        assert lib.ggq_row_bytes(qt, 256) == -1
    assert isinstance(lib.ggq_last_error(), bytes)


def test_null_and_shape_errors_come_back_before_any_launch(pkg):
    lib = pkg._lib.load()
    assert lib.ggq_mmq(None, None, 12, 4, 4, 256, None, None) == -4           # null pointers
    assert b"null" in lib.ggq_last_error().lower() or lib.ggq_last_error()
    assert lib.ggq_dequantize(3, ctypes.c_void_p(16), 1, 256, ctypes.c_void_p(16), 0, None) == -1  # unknown type
    assert lib.ggq_dequantize(12, ctypes.c_void_p(16), 1, 100, ctypes.c_void_p(16), 0, None) == -2  # K not whole blocks


def test_python_mirror_guards(pkg):
    loss_mod = pkg.gguf_liger_loss
    h = torch.zeros(4, 64, dtype=torch.bfloat16)
    y = torch.zeros(4, dtype=torch.long)
    p = torch.zeros(8, gb.row_bytes(gb.Q8_0, 64), dtype=torch.uint8)
    fwd = loss_mod._packed_linear_cross_entropy_forward
    with pytest.raises(ValueError):
        fwd(h.reshape(2, 2, 64), p, y, 8, 8, 256, -100, "mean")
    with pytest.raises(TypeError):
        fwd(h.float(), p, y, 8, 8, 256, -100, "mean")
    with pytest.raises(TypeError):
        fwd(h, p, y.int(), 8, 8, 256, -100, "mean")
    with pytest.raises(ValueError):
        fwd(h, p, y, 8, 8, 256, -100, "none")
    with pytest.raises(ValueError):
        fwd(h, p, y, 8, 8, 0, -100, "mean")
    with pytest.raises(ValueError):
        fwd(h, p, y, 2, 8, 256, -100, "mean")  # Q4_0: no native kernel
    with pytest.raises((RuntimeError, ValueError)):
        fwd(h, p, y, 8, 8, 256, -100, "mean")  # host tensors: refused, never copied behind the caller's back
    lm_head = pkg.fast_lora.GGUFLinear(64, 8, pkg.gguf.GGUFQuantizedTensor(p, 8, (8, 64)))
    labels = torch.zeros(1, 4, dtype=torch.long)
    for bad in (dict(return_z_loss=True), dict(label_smoothing=0.1), dict(ce_weight=torch.ones(8)), dict(lse_square_scale=1e-4)):
        with pytest.raises(RuntimeError):
            loss_mod._packed_for_causal_lm_loss(h.reshape(1, 4, 64), lm_head, labels, 64, **bad)
    with pytest.raises(RuntimeError):
        loss_mod._packed_for_causal_lm_loss(h.reshape(1, 4, 64), lm_head, labels, 64, final_logit_softcapping=30.0)
    routing = pkg.fast_moe_routing
    with pytest.raises(ValueError):
        routing.prepare_expert_routing(torch.zeros(2, 3, 8, dtype=torch.bfloat16), torch.zeros(2, 2, dtype=torch.long), torch.zeros(2, 2), 4)
    with pytest.raises(RuntimeError):
        routing.prepare_expert_routing(torch.zeros(2, 8, dtype=torch.bfloat16), torch.zeros(2, 2, dtype=torch.long), torch.zeros(2, 2), 4)
    assert pkg.fast_lora.supports_native_mmq(lm_head.weight)


def test_torch_quantizers_produce_payloads_the_oracle_decodes(pkg):
    """The torch quantizers only manufacture synthetic payloads for the benchmark; what they must
    guarantee is a valid block layout whose decode lands within one quantisation step of the input."""
    gen = torch.Generator().manual_seed(5)
    w = torch.randn(6, 512, generator=gen) * 0.02
    q8 = pkg.gguf.quantize_q8_0(w)
    assert q8.dtype == torch.uint8 and tuple(q8.shape) == (6, gb.row_bytes(gb.Q8_0, 512))
    assert np.array_equal(q8.numpy(), gb.quantize(w.numpy(), gb.Q8_0))  # same rule as gguf-py's quantize
    for fn, qt, step in ((pkg.gguf.quantize_q8_0, gb.Q8_0, 1 / 127), (pkg.gguf.quantize_q4_k, gb.Q4_K, 1 / 15), (pkg.gguf.quantize_q6_k, gb.Q6_K, 1 / 31)):
        payload = fn(w)
        assert tuple(payload.shape) == (6, gb.row_bytes(qt, 512))
        back = gb.dequantize(payload.numpy(), qt)
        blocks = w.numpy().reshape(6, -1, 32)
        span = np.abs(blocks).max(axis=2, keepdims=True) * 2.0
        err = np.abs(back.reshape(6, -1, 32) - blocks)
        assert (err <= span * step * 1.01 + 1e-7).all(), gb.QUANT_SIZES[qt]
    iq = pkg.gguf.random_iq2_xxs((4, 512), generator=gen)
    vals = gb.dequantize(iq.numpy(), gb.IQ2_XXS)
    assert vals.shape == (4, 512) and np.isfinite(vals).all() and np.abs(vals).max() < 1.0
