"""Dense LoRA linear over a frozen packed GGUF weight:  Y = X W^T + s (X A^T) B^T.

Host-side mirror of the reference's ``fast_lora.py``: the same operator names (``mmq``,
``mmq_grad_input``, ``supports_native_mmq``) and module surface (``GGUFLinear`` base layer wrapped by
``FastGGUFLoraLinear`` with ``lora_A`` / ``lora_B`` / ``scaling``), but the base matmul, the LoRA
residual (``_fused_lora_add``, fast_lora.py:34-65) and the whole backward (dX, dA, dB;
test_fast_lora.py:101-134) each run as one call into the gfx950 kernel library.  PEFT is not a
dependency; the wrapper keeps PEFT's attribute names so adapter state dicts line up.
"""

from __future__ import annotations

import math
from typing import Any

import torch

from . import _lib
from .gguf import GGML_QUANT_SIZES, GGUFQuantizedTensor, row_bytes

# GGML type ids with native kernels here: 8, 10, 11, 12, 13, 14, 16.  The reference's wheel also lists 22 (IQ2_S,
# fast_lora.py:24-27), which is not implemented and is rejected, never routed elsewhere.
_NATIVE_MMQ_QUANT_TYPES = frozenset(GGML_QUANT_SIZES)


def supports_native_mmq(weight: Any) -> bool:
    return int(weight.quant_type) in _NATIVE_MMQ_QUANT_TYPES


def _check_packed(payload: torch.Tensor, quant_type: int, rows: int, k: int, what: str) -> None:
    _lib.require_device_tensor(payload, f"{what} payload", torch.uint8)
    if quant_type not in _NATIVE_MMQ_QUANT_TYPES:
        raise ValueError(f"{what}: GGML type id {quant_type} has no native MMQ kernel (supported: {sorted(_NATIVE_MMQ_QUANT_TYPES)})")
    if payload.ndim != 2 or payload.shape[0] != rows or payload.shape[1] != row_bytes(quant_type, k):
        raise ValueError(f"{what}: payload shape {tuple(payload.shape)} does not describe a [{rows}, {k}] weight of type {quant_type}")
    if k % 64:
        raise ValueError(f"{what}: in_features {k} must be a multiple of 64")


def _flat_bf16(x: torch.Tensor, name: str) -> torch.Tensor:
    _lib.require_device_tensor(x, name, torch.bfloat16)
    return x.reshape(-1, x.shape[-1])


def _mmq_forward(x: torch.Tensor, payload: torch.Tensor, quant_type: int, out_features: int) -> torch.Tensor:
    x2 = _flat_bf16(x, "mmq input")
    m, k = x2.shape
    _check_packed(payload, quant_type, out_features, k, "mmq")
    y = torch.empty(m, out_features, dtype=torch.bfloat16, device=x.device)
    if m:
        _lib.check(_lib.load().ggq_mmq(x2.data_ptr(), payload.data_ptr(), quant_type, m, out_features, k, y.data_ptr(), _lib.stream_handle(x.device)))
    return y.reshape(*x.shape[:-1], out_features)


def mmq_grad_input(grad_output: torch.Tensor, payload: torch.Tensor, quant_type: int, in_features: int) -> torch.Tensor:
    """dX = dY . W with W decoded to bf16 and fp32 accumulation (no quantization of the cotangent)."""
    payload = payload.as_subclass(torch.Tensor)
    quant_type = int(quant_type)
    g2 = _flat_bf16(grad_output, "mmq_grad_input cotangent")
    m, n = g2.shape
    _check_packed(payload, quant_type, n, in_features, "mmq_grad_input")
    dx = torch.empty(m, in_features, dtype=torch.bfloat16, device=grad_output.device)
    if m:
        _lib.check(_lib.load().ggq_mmq_grad_input(g2.data_ptr(), payload.data_ptr(), quant_type, m, n, in_features, dx.data_ptr(), _lib.stream_handle(g2.device)))
    return dx.reshape(*grad_output.shape[:-1], in_features)


class _Mmq(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, payload, quant_type, out_features):
        ctx.save_for_backward(payload)
        ctx.quant_type, ctx.in_features = quant_type, x.shape[-1]
        return _mmq_forward(x, payload, quant_type, out_features)

    @staticmethod
    def backward(ctx, grad_output):
        if torch.is_grad_enabled():
            raise RuntimeError("packed MMQ does not support higher-order gradients")
        (payload,) = ctx.saved_tensors
        dx = mmq_grad_input(grad_output.contiguous(), payload, ctx.quant_type, ctx.in_features) if ctx.needs_input_grad[0] else None
        return dx, None, None, None


def mmq(x: torch.Tensor, payload: torch.Tensor, quant_type: int, out_features: int) -> torch.Tensor:
    """Y = X . W^T over packed rows (the reference's ``torch_ggml_ops.mmq``, fast_lora.py:155-160)."""
    payload = payload.as_subclass(torch.Tensor)
    return _Mmq.apply(x, payload, int(quant_type), int(out_features))


class _FixedGroupedMmq(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, packed_groups, quant_type):
        _lib.require_device_tensor(x, "fixed grouped input", torch.bfloat16)
        _lib.require_device_tensor(packed_groups, "packed groups", torch.uint8)
        if x.ndim < 2 or packed_groups.ndim != 3 or x.shape[-2] != packed_groups.shape[0]:
            raise ValueError(f"fixed grouped MMQ takes [..., groups, k] and [groups, n, bytes], got {tuple(x.shape)} and {tuple(packed_groups.shape)}")
        groups, n_group, k = packed_groups.shape[0], packed_groups.shape[1], x.shape[-1]
        _check_packed(packed_groups[0], quant_type, n_group, k, "fixed grouped MMQ")
        rows = x.numel() // (groups * k)
        y = torch.empty(*x.shape[:-1], n_group, dtype=torch.bfloat16, device=x.device)
        _lib.check(_lib.load().ggq_fixed_grouped_mmq(x.data_ptr(), packed_groups.data_ptr(), quant_type, rows, groups, n_group, k, y.data_ptr(),
                                                     _lib.stream_handle(x.device)))
        ctx.save_for_backward(packed_groups)
        ctx.quant_type, ctx.k = quant_type, k
        return y

    @staticmethod
    def backward(ctx, grad_output):
        if torch.is_grad_enabled():
            raise RuntimeError("packed MMQ does not support higher-order gradients")
        if not ctx.needs_input_grad[0]:
            return None, None, None
        (packed_groups,) = ctx.saved_tensors
        g = grad_output.contiguous()
        groups, n_group = packed_groups.shape[0], packed_groups.shape[1]
        rows = g.numel() // (groups * n_group)
        dx = torch.empty(*g.shape[:-1], ctx.k, dtype=torch.bfloat16, device=g.device)
        _lib.check(_lib.load().ggq_fixed_grouped_mmq_grad_input(g.data_ptr(), packed_groups.data_ptr(), ctx.quant_type, rows, groups, n_group, ctx.k,
                                                                dx.data_ptr(), _lib.stream_handle(g.device)))
        return dx, None, None


def fixed_grouped_mmq(x: torch.Tensor, packed_groups: torch.Tensor, quant_type: int = 8) -> torch.Tensor:
    """[..., groups, k] x packed [groups, n, bytes] -> [..., groups, n]: every group its own frozen packed matrix (the
    reference's ``torch_ggml_ops.fixed_grouped_mmq``, deepseek_v4_lora.py:91-124; Q8_0 there, any supported type here)."""
    return _FixedGroupedMmq.apply(x, packed_groups.as_subclass(torch.Tensor), int(quant_type))


def fixed_grouped_mmq_grad_input(grad_output: torch.Tensor, packed_groups: torch.Tensor, quant_type: int, in_features: int) -> torch.Tensor:
    """Input gradient of ``fixed_grouped_mmq``: [..., groups, n] x packed [groups, n, bytes] -> [..., groups, in_features]."""
    packed_groups = packed_groups.as_subclass(torch.Tensor)
    _lib.require_device_tensor(grad_output, "fixed grouped cotangent", torch.bfloat16)
    _lib.require_device_tensor(packed_groups, "fixed grouped payload", torch.uint8)
    groups, n_group = packed_groups.shape[0], packed_groups.shape[1]
    if grad_output.ndim < 2 or tuple(grad_output.shape[-2:]) != (groups, n_group) or packed_groups.shape[2] != row_bytes(quant_type, in_features):
        raise ValueError(f"fixed grouped cotangent {tuple(grad_output.shape)} does not fit packed groups {tuple(packed_groups.shape)} of type {quant_type}")
    rows = grad_output.numel() // (groups * n_group)
    dx = torch.empty(*grad_output.shape[:-1], in_features, dtype=torch.bfloat16, device=grad_output.device)
    _lib.check(_lib.load().ggq_fixed_grouped_mmq_grad_input(grad_output.data_ptr(), packed_groups.data_ptr(), quant_type, rows, groups, n_group, in_features,
                                                            dx.data_ptr(), _lib.stream_handle(grad_output.device)))
    return dx


def _workspace(device, rows: int, groups: int, experts: int, n_total: int, k: int, r: int) -> torch.Tensor:
    nbytes = _lib.load().ggq_lora_workspace_bytes(rows, groups, experts, n_total, k, r)
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


class _LoraMmq(torch.autograd.Function):
    """Base matmul + LoRA residual in one forward call; dX, dA, dB in one backward call."""

    @staticmethod
    def forward(ctx, x, payload, quant_type, out_features, lora_a, lora_b, scaling):
        x2 = _flat_bf16(x, "LoRA linear input")
        m, k = x2.shape
        _check_packed(payload, quant_type, out_features, k, "LoRA linear")
        _lib.require_device_tensor(lora_a, "lora_A", torch.bfloat16)
        _lib.require_device_tensor(lora_b, "lora_B", torch.bfloat16)
        r = lora_a.shape[0]
        if tuple(lora_a.shape) != (r, k) or tuple(lora_b.shape) != (out_features, r):
            raise ValueError(f"LoRA factors must be A [r,{k}] and B [{out_features},r], got {tuple(lora_a.shape)} and {tuple(lora_b.shape)}")
        r_pad = (r + 15) // 16 * 16
        xa = torch.empty(m, r_pad, dtype=torch.bfloat16, device=x.device)
        y = torch.empty(m, out_features, dtype=torch.bfloat16, device=x.device)
        if m:
            ws = _workspace(x.device, m, 0, 1, out_features, k, r)
            _lib.check(_lib.load().ggq_lora_mmq_forward(
                x2.data_ptr(), payload.data_ptr(), quant_type, m, out_features, k, lora_a.data_ptr(), lora_b.data_ptr(), r,
                float(scaling), xa.data_ptr(), y.data_ptr(), ws.data_ptr(), ws.numel(), _lib.stream_handle(x.device)))
        ctx.save_for_backward(x2, xa, payload, lora_a, lora_b)
        ctx.meta = (quant_type, out_features, float(scaling), x.shape)
        return y.reshape(*x.shape[:-1], out_features)

    @staticmethod
    def backward(ctx, grad_output):
        if torch.is_grad_enabled():
            raise RuntimeError("packed MMQ LoRA linear does not support higher-order gradients")
        x2, xa, payload, lora_a, lora_b = ctx.saved_tensors
        quant_type, n, scaling, x_shape = ctx.meta
        g2 = _flat_bf16(grad_output.contiguous(), "LoRA linear cotangent")
        m, k = x2.shape
        r = lora_a.shape[0]
        dx = torch.empty_like(x2)
        da = torch.empty_like(lora_a) if ctx.needs_input_grad[4] else None
        db = torch.empty_like(lora_b) if ctx.needs_input_grad[5] else None
        ws = _workspace(x2.device, m, 0, 1, n, k, r)
        _lib.check(_lib.load().ggq_lora_mmq_backward(
            g2.data_ptr(), payload.data_ptr(), quant_type, m, n, k, x2.data_ptr(), xa.data_ptr(), lora_a.data_ptr(),
            lora_b.data_ptr(), r, scaling, dx.data_ptr(), _lib.ptr(da), _lib.ptr(db), ws.data_ptr(), ws.numel(),
            _lib.stream_handle(x2.device)))
        return (dx.reshape(x_shape) if ctx.needs_input_grad[0] else None), None, None, None, da, db, None


def lora_mmq(x, payload, quant_type, out_features, lora_a, lora_b, scaling) -> torch.Tensor:
    return _LoraMmq.apply(x, payload.as_subclass(torch.Tensor), int(quant_type), int(out_features), lora_a, lora_b, float(scaling))


def _fused_lora_add(result, x, lora_A: torch.nn.Linear, lora_B: torch.nn.Linear, dropout: torch.nn.Module, scaling: float):
    """``result + scaling * lora_B(lora_A(dropout(x)))`` with framework ops, for base layers that are
    not packed (ordinary float linears); same composition as fast_lora.py:34-65."""
    dt = result.dtype
    x_a = torch.matmul(dropout(x).to(dt), lora_A.weight.to(dt).transpose(0, 1))
    shape = result.shape
    out = torch.addmm(result.reshape(-1, shape[-1]), x_a.reshape(-1, x_a.shape[-1]), lora_B.weight.to(dt).transpose(0, 1), beta=1, alpha=scaling).reshape(shape)
    if lora_B.bias is not None:
        out = torch.add(out, lora_B.bias.to(dt), alpha=scaling)
    return out


def _layer_input(x: torch.Tensor) -> torch.Tensor:
    """What a layer hands to the operators, which take only contiguous 16-byte aligned operands and copy nothing themselves:
    callers of a layer (a model's forward) may pass views, so the layer makes the bounded copy."""
    if not x.is_contiguous():
        return x.contiguous()
    return x.clone() if x.data_ptr() % 16 else x


class GGUFLinear(torch.nn.Module):
    """Frozen linear layer whose weight stays packed (stand-in for the fork's ``GGUFLinear``; exposes
    the attributes fast_lora.py:137-162 and gguf_liger_loss.py:305-324 read)."""

    def __init__(self, in_features: int, out_features: int, weight: GGUFQuantizedTensor, bias: torch.Tensor | None = None,
                 compute_dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        if tuple(weight.logical_shape) != (out_features, in_features):
            raise ValueError(f"weight logical shape {weight.logical_shape} != ({out_features}, {in_features})")
        self.in_features, self.out_features = in_features, out_features
        self.weight = weight
        self.bias = bias
        self.compute_dtype = compute_dtype
        self.input_permutation = None
        self.output_permutation = None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.compute_dtype != torch.bfloat16:
            raise RuntimeError("The packed GGUF MMQ linear path requires BF16 compute_dtype.")
        y = mmq(_layer_input(x), self.weight, self.weight.quant_type, self.out_features)
        if self.bias is not None:
            y = y + self.bias.to(device=y.device, dtype=y.dtype)
        return y


_WRAPPER_OPTIONS = ("lora_dropout", "use_rslora", "use_dora", "lora_bias", "init_lora_weights", "alora_invocation_tokens")


def _new_factors(wrapper: torch.nn.Module, adapter_name: str, in_features: int, out_features: int, r: int, lora_alpha: float, opts: dict,
                 device, dtype) -> None:
    """lora_A / lora_B / scaling of one adapter under PEFT's names and shapes.  ``init_lora_weights``: True gives A
    Kaiming-uniform (a = sqrt 5) and B zero, "gaussian" A ~ N(0, 1/r) and B zero, False a non-zero delta for tests
    (A Kaiming-uniform, B ~ N(0, 0.02))."""
    if r <= 0:
        raise ValueError(f"LoRA rank must be positive, got {r}")
    if opts["use_dora"] or opts["alora_invocation_tokens"] is not None:
        raise ValueError("the fast LoRA wrappers do not support DoRA or aLoRA variants")
    if opts["lora_bias"]:
        raise ValueError("the fast LoRA wrappers do not support LoRA bias")
    wrapper.lora_A = torch.nn.ModuleDict({adapter_name: torch.nn.Linear(in_features, r, bias=False, device=device, dtype=dtype)})
    wrapper.lora_B = torch.nn.ModuleDict({adapter_name: torch.nn.Linear(r, out_features, bias=False, device=device, dtype=dtype)})
    init = opts["init_lora_weights"]
    if init is True or init is False:
        torch.nn.init.kaiming_uniform_(wrapper.lora_A[adapter_name].weight, a=math.sqrt(5))
    elif init == "gaussian":
        torch.nn.init.normal_(wrapper.lora_A[adapter_name].weight, std=1 / r)
    else:
        raise ValueError(f"the fast LoRA wrappers do not support init_lora_weights={init!r}")
    if init is False:
        torch.nn.init.normal_(wrapper.lora_B[adapter_name].weight, std=0.02)
    else:
        torch.nn.init.zeros_(wrapper.lora_B[adapter_name].weight)
    wrapper.r = {adapter_name: r}
    wrapper.lora_alpha = {adapter_name: lora_alpha}
    wrapper.scaling = {adapter_name: lora_alpha / (math.sqrt(r) if opts["use_rslora"] else r)}
    wrapper.active_adapter = adapter_name
    wrapper.disable_adapters = False
    wrapper.merged = False


class FastLoraLinear(torch.nn.Module):
    """LoRA wrapper for an ordinary floating ``torch.nn.Linear`` (counterpart of fast_lora.py:68-124): the base layer's own
    forward, then the fused residual ``_fused_lora_add``.  Framework operators only: nothing here is packed.  Constructed the
    way PEFT constructs a registered wrapper: ``(base_layer, adapter_name, config=..., r=..., lora_alpha=..., **kwargs)``."""

    def __init__(self, base_layer: torch.nn.Module, adapter_name: str = "default", *, r: int, lora_alpha: float, config: Any = None,
                 **kwargs: Any):
        super().__init__()
        if not isinstance(adapter_name, str):
            raise TypeError("the second argument is the adapter's name; pass r= and lora_alpha= by keyword")
        from .peft_compat import adapter_options

        opts = adapter_options(config, kwargs, _WRAPPER_OPTIONS)
        self.base_layer = base_layer
        w = base_layer.weight
        _new_factors(self, adapter_name, base_layer.in_features, base_layer.out_features, r, lora_alpha, opts, w.device, w.dtype)
        p = float(opts["lora_dropout"])
        self.lora_dropout = torch.nn.ModuleDict({adapter_name: torch.nn.Dropout(p) if p > 0.0 else torch.nn.Identity()})

    def get_base_layer(self) -> torch.nn.Module:
        return self.base_layer

    def forward(self, x: torch.Tensor, *args: Any, **kwargs: Any) -> torch.Tensor:
        result = self.base_layer(x, *args, **kwargs)
        if self.disable_adapters:
            return result
        name = self.active_adapter
        return _fused_lora_add(result, x, self.lora_A[name], self.lora_B[name], self.lora_dropout[name], self.scaling[name])


class FastGGUFLoraLinear(torch.nn.Module):
    """LoRA wrapper for a frozen packed ``GGUFLinear`` (counterpart of fast_lora.py:127-175), constructed like
    ``FastLoraLinear``.

    One adapter, no dropout, no DoRA: the configurations the reference's fast path accepts
    (fast_lora.py:82-94); anything else is rejected rather than served by a slower route."""

    def __init__(self, base_layer: GGUFLinear, adapter_name: str = "default", *, r: int, lora_alpha: float, config: Any = None,
                 **kwargs: Any):
        super().__init__()
        if not isinstance(adapter_name, str):
            raise TypeError("the second argument is the adapter's name; pass r= and lora_alpha= by keyword")
        from .peft_compat import adapter_options

        opts = adapter_options(config, kwargs, _WRAPPER_OPTIONS)
        if r > 64:
            raise ValueError(f"LoRA rank must be in 1..64, got {r}")
        if float(opts["lora_dropout"]) != 0.0:
            raise ValueError("the packed LoRA linear requires lora_dropout=0")
        if not isinstance(base_layer.weight, GGUFQuantizedTensor) or not supports_native_mmq(base_layer.weight):
            raise TypeError("FastGGUFLoraLinear requires a packed weight of a natively supported GGML type")
        if base_layer.input_permutation is not None or base_layer.output_permutation is not None:
            raise RuntimeError("the packed GGUF MMQ linear path does not support layout permutations")
        self.base_layer = base_layer
        _new_factors(self, adapter_name, base_layer.in_features, base_layer.out_features, r, lora_alpha, opts, base_layer.weight.device,
                     base_layer.compute_dtype)

    def get_base_layer(self) -> torch.nn.Module:
        return self.base_layer

    def forward(self, x: torch.Tensor, *args: Any, **kwargs: Any) -> torch.Tensor:
        if args or kwargs:
            raise TypeError("The packed GGUF MMQ linear path accepts only its input tensor.")
        base = self.base_layer
        if base.compute_dtype != torch.bfloat16:
            raise RuntimeError("The packed GGUF MMQ linear path requires BF16 compute_dtype.")
        if self.disable_adapters:
            return base(x)
        name = self.active_adapter
        y = lora_mmq(_layer_input(x), base.weight, base.weight.quant_type, base.out_features, self.lora_A[name].weight, self.lora_B[name].weight, self.scaling[name])
        if base.bias is not None:
            y = y + base.bias.to(device=y.device, dtype=y.dtype)
        return y

    def merge(self, *args: Any, **kwargs: Any) -> None:
        raise RuntimeError("GGUF LoRA adapters cannot be merged into packed base weights.")

    def unmerge(self) -> None:
        raise RuntimeError("GGUF LoRA adapters cannot be unmerged because merging is unsupported.")


def register_fast_lora(lora_config):
    """Registers the linear wrappers on one LoRA config (fast_lora.py:178-200): config-local, through the config's
    ``_register_custom_module``; nothing is patched process-wide.  ``GGUFLinear`` comes first so that a packed layer never
    falls to the float wrapper."""
    register = getattr(lora_config, "_register_custom_module", None)
    if register is None:
        raise RuntimeError("This PEFT version has no LoraConfig._register_custom_module API. "
                           "Cannot install fast LoRA without a global monkey patch.")
    register({GGUFLinear: FastGGUFLoraLinear, torch.nn.Linear: FastLoraLinear})
    return lora_config


# ------------------------------------------------------------------------------------------------
# Adapter checkpoints with PEFT's key names (what the reference saves and loads through
# get_peft_model_state_dict / set_peft_model_state_dict, test_deepseek_v4_serialization.py:74-101): only the LoRA
# factors, the adapter's name taken out of the keys ("...lora_A_down.default.weight" -> "...lora_A_down.weight").
_ADAPTER_PREFIX = "lora_"


def get_adapter_state_dict(model: torch.nn.Module, adapter_name: str = "default", prefix: str = "") -> dict[str, torch.Tensor]:
    """The adapter's factors under checkpoint names; ``prefix`` (e.g. ``"base_model.model."``) is put in front of every
    key for files that PEFT's own wrapper is to read."""
    out = {}
    for key, value in model.state_dict().items():
        if _ADAPTER_PREFIX not in key:
            continue
        parts = key.split(".")
        if adapter_name not in parts:
            continue  # another adapter's factors
        i = len(parts) - 1 - parts[::-1].index(adapter_name)
        out[prefix + ".".join(parts[:i] + parts[i + 1:])] = value
    return out


def set_adapter_state_dict(model: torch.nn.Module, state: dict[str, torch.Tensor], adapter_name: str = "default", prefix: str = ""):
    """Loads a checkpoint written under those names.  Returns (missing_keys, unexpected_keys): adapter parameters of the
    model the checkpoint lacks, and checkpoint entries no parameter takes.  Shapes must match; dtypes are cast."""
    own = {k: v for k, v in model.state_dict().items() if _ADAPTER_PREFIX in k and adapter_name in k.split(".")}
    renamed = {}
    for key, value in state.items():
        k = key[len(prefix):] if prefix and key.startswith(prefix) else key
        if _ADAPTER_PREFIX in k:
            suffix = k.split(_ADAPTER_PREFIX)[-1]
            if "." in suffix:  # "A_down.weight": the adapter's name goes in front of what follows the factor's name
                rest = ".".join(suffix.split(".")[1:])
                k = k[: len(k) - len(rest)] + f"{adapter_name}." + rest
            else:
                k = f"{k}.{adapter_name}"
        renamed[k] = value
    unexpected = [k for k in renamed if k not in own]
    missing = [k for k in own if k not in renamed]
    with torch.no_grad():
        for k, target in own.items():
            if k in renamed:
                src = renamed[k]
                if tuple(src.shape) != tuple(target.shape):
                    raise ValueError(f"adapter checkpoint entry {k}: shape {tuple(src.shape)} does not fit {tuple(target.shape)}")
                target.copy_(src.to(device=target.device, dtype=target.dtype))
    return missing, unexpected
