"""Packed GGUF weights as the matmul path sees them.

``GGUFQuantizedTensor`` stands in for the class of the same name in the transformers ``gguf`` fork
(imported by the reference at fast_lora.py:22, fast_moe_lora.py:27-30, gguf_liger_loss.py:29): a uint8
payload ``[..., rows, row_bytes]`` carrying ``quant_type`` (GGML type id) and ``logical_shape``.  The
reference only touches ``as_subclass(torch.Tensor)``, ``quant_type``, ``logical_shape`` and
``requires_grad`` (fast_lora.py:139-160, fast_moe_lora.py:206-228).

``dequantize_gguf_tensor`` runs the HIP block decoders.  The ``quantize_*`` functions are torch
restatements of simple min/max block fits that manufacture valid synthetic payloads on any device
(BASELINE configurations: weights drawn from N(0, 0.02^2), then quantized); they are not ggml's
search-based quantizers and are not on the hot path.
"""

from __future__ import annotations

import torch

from . import _lib

Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, IQ2_XXS = 8, 10, 11, 12, 13, 14, 16
# type id -> (elements per block, bytes per block)
GGML_QUANT_SIZES = {Q8_0: (32, 34), Q2_K: (256, 84), Q3_K: (256, 110), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210), IQ2_XXS: (256, 66)}
QUANT_NAMES = {Q8_0: "Q8_0", Q2_K: "Q2_K", Q3_K: "Q3_K", Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", IQ2_XXS: "IQ2_XXS"}


def row_bytes(quant_type: int, k: int) -> int:
    if quant_type not in GGML_QUANT_SIZES:
        raise ValueError(f"GGML type id {quant_type} has no native kernels (supported: {sorted(GGML_QUANT_SIZES)})")
    elems, nbytes = GGML_QUANT_SIZES[quant_type]
    if k % elems:
        raise ValueError(f"K={k} is not a multiple of the {elems}-element block of {QUANT_NAMES[quant_type]}")
    return k // elems * nbytes


class GGUFQuantizedTensor(torch.Tensor):
    """uint8 payload + (quant_type, logical_shape).  Never differentiable."""

    quant_type: int
    logical_shape: tuple[int, ...]

    @staticmethod
    def __new__(cls, payload: torch.Tensor, quant_type: int, logical_shape):
        if payload.dtype != torch.uint8:
            raise TypeError(f"packed payload must be uint8, got {payload.dtype}")
        logical_shape = tuple(int(v) for v in logical_shape)
        expected = logical_shape[:-1] + (row_bytes(int(quant_type), logical_shape[-1]),)
        if tuple(payload.shape) != expected:
            raise ValueError(f"payload shape {tuple(payload.shape)} does not match logical shape {logical_shape}: expected {expected}")
        t = torch.Tensor._make_subclass(cls, payload, False)
        t.quant_type = int(quant_type)
        t.logical_shape = logical_shape
        return t

    def __repr__(self) -> str:  # pragma: no cover - cosmetic
        return f"GGUFQuantizedTensor({QUANT_NAMES.get(self.quant_type, self.quant_type)}, logical_shape={self.logical_shape}, device={self.device})"

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        # operations on the payload yield plain tensors (the metadata no longer describes them)
        with torch._C.DisableTorchFunctionSubclass():
            return func(*args, **(kwargs or {}))


def dequantize_gguf_tensor(payload: torch.Tensor, quant_type: int, dtype: torch.dtype = torch.bfloat16, device=None) -> torch.Tensor:
    """Packed ``[..., rows, row_bytes]`` -> logical ``[..., rows, K]`` in bf16 or fp32, bit-exact with
    ggml's decoders (fp32 arithmetic, then round-to-nearest-even for bf16)."""
    payload = payload.as_subclass(torch.Tensor)
    if device is not None and torch.device(device) != payload.device:
        payload = payload.to(device)
    quant_type = int(quant_type)
    if quant_type not in GGML_QUANT_SIZES:
        raise ValueError(f"GGML type id {quant_type} has no native decoder (supported: {sorted(GGML_QUANT_SIZES)})")
    if dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"dequantize_gguf_tensor produces bfloat16 or float32, got {dtype}")
    _lib.require_device_tensor(payload, "payload", torch.uint8)
    elems, nbytes = GGML_QUANT_SIZES[quant_type]
    if payload.shape[-1] % nbytes:
        raise ValueError("payload rows are not a whole number of blocks")
    k = payload.shape[-1] // nbytes * elems
    rows = payload.numel() // payload.shape[-1] if payload.numel() else 0
    out = torch.empty(payload.shape[:-1] + (k,), dtype=dtype, device=payload.device)
    if rows:
        _lib.check(_lib.load().ggq_dequantize(quant_type, payload.data_ptr(), rows, k, out.data_ptr(), int(dtype == torch.float32), _lib.stream_handle(payload.device)))
    return out


# ------------------------------------------------------------------------------------------------
# synthetic payload factories (torch, any device)
def _roundf(x: torch.Tensor) -> torch.Tensor:
    return torch.sign(x) * torch.floor(x.abs() + 0.5)


def _f16_bytes(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.float16).contiguous().view(torch.uint8)


def quantize_q8_0(w: torch.Tensor) -> torch.Tensor:
    lead, k = w.shape[:-1], w.shape[-1]
    x = w.float().reshape(-1, 32)
    d = x.abs().amax(dim=1, keepdim=True) / 127.0
    inv = torch.where(d == 0, torch.zeros_like(d), 1.0 / d)
    q = _roundf(x * inv).to(torch.int8)
    out = torch.empty(x.shape[0], 34, dtype=torch.uint8, device=w.device)
    out[:, 0:2] = _f16_bytes(d).reshape(-1, 2)
    out[:, 2:] = q.view(torch.uint8)
    return out.reshape(*lead, k // 32 * 34)


def quantize_q4_k(w: torch.Tensor) -> torch.Tensor:
    lead, k = w.shape[:-1], w.shape[-1]
    sub = w.float().reshape(-1, 8, 32)
    nb = sub.shape[0]
    lo = sub.amin(dim=2).clamp(max=0)
    hi = sub.amax(dim=2)
    scale = (hi - lo) / 15.0
    off = -lo
    d = (scale.amax(dim=1, keepdim=True) / 63.0).to(torch.float16).float()
    dmin = (off.amax(dim=1, keepdim=True) / 63.0).to(torch.float16).float()
    sc = torch.where(d > 0, _roundf(scale / d.clamp(min=1e-30)).clamp(0, 63), torch.zeros_like(scale)).to(torch.uint8)
    m = torch.where(dmin > 0, _roundf(off / dmin.clamp(min=1e-30)).clamp(0, 63), torch.zeros_like(off)).to(torch.uint8)
    dl = (d * sc.float()).unsqueeze(2)
    ml = (dmin * m.float()).unsqueeze(2)
    q = torch.where(dl > 0, _roundf((sub + ml) / dl.clamp(min=1e-30)), torch.zeros_like(sub)).clamp(0, 15).to(torch.uint8)
    q = q.reshape(nb, 4, 2, 32)
    out = torch.empty(nb, 144, dtype=torch.uint8, device=w.device)
    out[:, 0:2] = _f16_bytes(d).reshape(-1, 2)
    out[:, 2:4] = _f16_bytes(dmin).reshape(-1, 2)
    out[:, 4:8] = sc[:, 0:4] | ((sc[:, 4:8] >> 4) << 6)
    out[:, 8:12] = m[:, 0:4] | ((m[:, 4:8] >> 4) << 6)
    out[:, 12:16] = (sc[:, 4:8] & 0x0F) | ((m[:, 4:8] & 0x0F) << 4)
    out[:, 16:] = (q[:, :, 0, :] | (q[:, :, 1, :] << 4)).reshape(nb, 128)
    return out.reshape(*lead, k // 256 * 144)


def quantize_q6_k(w: torch.Tensor) -> torch.Tensor:
    lead, k = w.shape[:-1], w.shape[-1]
    sub = w.float().reshape(-1, 16, 16)
    nb = sub.shape[0]
    scale = sub.abs().amax(dim=2) / 31.0
    d = (scale.amax(dim=1, keepdim=True) / 127.0).to(torch.float16).float()
    sc = torch.where(d > 0, _roundf(scale / d.clamp(min=1e-30)).clamp(0, 127), torch.zeros_like(scale)).to(torch.int8)
    dl = (d * sc.float()).unsqueeze(2)
    q = torch.where(dl != 0, _roundf(sub / torch.where(dl != 0, dl, torch.ones_like(dl))), torch.zeros_like(sub))
    q = (q.clamp(-32, 31) + 32).to(torch.uint8).reshape(nb, 2, 4, 32)
    ql = torch.empty(nb, 2, 64, dtype=torch.uint8, device=w.device)
    ql[:, :, 0:32] = (q[:, :, 0] & 0x0F) | ((q[:, :, 2] & 0x0F) << 4)
    ql[:, :, 32:64] = (q[:, :, 1] & 0x0F) | ((q[:, :, 3] & 0x0F) << 4)
    qh = (q[:, :, 0] >> 4) | ((q[:, :, 1] >> 4) << 2) | ((q[:, :, 2] >> 4) << 4) | ((q[:, :, 3] >> 4) << 6)
    out = torch.empty(nb, 210, dtype=torch.uint8, device=w.device)
    out[:, 0:128] = ql.reshape(nb, 128)
    out[:, 128:192] = qh.reshape(nb, 64)
    out[:, 192:208] = sc.view(torch.uint8)
    out[:, 208:210] = _f16_bytes(d).reshape(-1, 2)
    return out.reshape(*lead, k // 256 * 210)


_IQ2XXS_GRID: dict = {}


def _iq2xxs_grid(device) -> torch.Tensor:
    """The 256 codebook points of IQ2_XXS as ``[256, 8]`` float64 magnitudes, read back through the library's own decoder
    (eight crafted blocks: block scale 1, group scale code 1, all signs plus, codebook indices 0..255), so that the
    quantizer below and the kernels cannot disagree about the table."""
    key = str(device)
    if key not in _IQ2XXS_GRID:
        blocks = torch.zeros(8, 66, dtype=torch.uint8)
        blocks[:, 0:2] = torch.tensor([0x00, 0x3C], dtype=torch.uint8)  # d = 1.0 in half precision
        body = blocks[:, 2:].reshape(8, 8, 8)
        body[:, :, 0:4] = torch.arange(256, dtype=torch.int64).reshape(8, 8, 4).to(torch.uint8)
        body[:, :, 7] = 1 << 4  # bits 28..31 of the second word: scale code 1 -> db = 1 * (0.5 + 1) * 0.25
        decoded = dequantize_gguf_tensor(blocks.to(device), IQ2_XXS, torch.float32)  # [8, 256]
        _IQ2XXS_GRID[key] = (decoded.double() / 0.375).reshape(256, 8)
    return _IQ2XXS_GRID[key]


def quantize_iq2_xxs(w: torch.Tensor, chunk_groups: int = 1 << 20) -> torch.Tensor:
    """IQ2_XXS payload of ``w [..., K]`` on the device the library runs on: per 32 weights a 4-bit scale code against the
    block's half-precision scale, per 8 weights the nearest codebook point of the magnitudes and seven sign bits (the
    weakest weight changes sign where the number of minus signs would be odd).  A nearest-point fit, not ggml's
    importance-weighted search; it manufactures BASELINE's "drawn from N(0, 0.02^2) and quantized" weights."""
    lead, k = w.shape[:-1], w.shape[-1]
    if k % 256:
        raise ValueError(f"last dimension {k} is not a multiple of 256")
    grid = _iq2xxs_grid(w.device)
    x = w.float().reshape(-1, 8, 32)
    nb = x.shape[0]
    # (divided by a device tensor: a division by a host scalar is carried out as a multiplication by its reciprocal on the
    # device, which is not the correctly rounded quotient the format's reference arithmetic takes)
    db_want = x.abs().amax(dim=2) / torch.full((), 33.0, dtype=torch.float32, device=w.device)
    d = (db_want.amax(dim=1, keepdim=True) * (4.0 / 15.5)).to(torch.float16).float()
    ls = torch.where(d > 0, (_roundf(db_want * 4 / torch.where(d > 0, d, torch.ones_like(d)) - 0.5)).clamp(0, 15), torch.zeros_like(db_want))
    db = d * (0.5 + ls) * 0.25
    v = x.reshape(nb, 8, 4, 8)
    neg = v < 0
    mag = v.abs()
    odd = (neg.sum(dim=3) & 1).bool()
    flip = torch.zeros_like(neg).scatter_(3, mag.argmin(dim=3, keepdim=True), odd.unsqueeze(3))
    neg = neg ^ flip
    dbx = db[:, :, None, None]
    t = torch.where(dbx > 0, mag / torch.where(dbx > 0, dbx, torch.ones_like(dbx)), torch.zeros_like(mag)).reshape(-1, 8)
    norms = (grid * grid).sum(dim=1)[None, :]
    idx = torch.empty(t.shape[0], dtype=torch.int64, device=w.device)
    for lo in range(0, t.shape[0], chunk_groups):  # the nearest codebook point: argmin |g|^2 - 2 t.g, in double precision
        idx[lo:lo + chunk_groups] = (norms - 2.0 * (t[lo:lo + chunk_groups].double() @ grid.T)).argmin(dim=1)
    sign7 = (neg[..., 0:7].to(torch.int64) << torch.arange(7, device=w.device)).sum(dim=3)  # [nb, 8, 4]
    aux = (ls.to(torch.int64) << 28) | (sign7 << (7 * torch.arange(4, device=w.device))).sum(dim=2)  # [nb, 8]
    out = torch.empty(nb, 66, dtype=torch.uint8, device=w.device)
    out[:, 0:2] = _f16_bytes(d).reshape(-1, 2)
    body = out[:, 2:].reshape(nb, 8, 8)
    body[:, :, 0:4] = idx.reshape(nb, 8, 4).to(torch.uint8)
    for byte in range(4):
        body[:, :, 4 + byte] = ((aux >> (8 * byte)) & 0xFF).to(torch.uint8)
    return out.reshape(*lead, k // 256 * 66)


def random_iq2_xxs(shape, generator: torch.Generator | None = None, device="cpu", std: float = 0.02) -> torch.Tensor:
    """Random IQ2_XXS payload for a logical ``[..., K]`` tensor: every byte pattern is a valid block
    (any codebook index, sign pattern and 4-bit scale); the half-precision block scale is set so that
    the decoded weights have roughly the requested spread."""
    *lead, k = shape
    nb = 1
    for v in lead:
        nb *= v
    nb *= k // 256
    b = torch.randint(0, 256, (nb, 66), dtype=torch.uint8, device=device, generator=generator)
    d = (std / 60.0) * (0.5 + torch.rand(nb, 1, device=device, generator=generator))
    b[:, 0:2] = _f16_bytes(d).reshape(-1, 2)
    return b.reshape(*lead, k // 256 * 66)


def quantize(w: torch.Tensor, quant_type: int) -> torch.Tensor:
    fn = {Q8_0: quantize_q8_0, Q4_K: quantize_q4_k, Q6_K: quantize_q6_k, IQ2_XXS: quantize_iq2_xxs}.get(int(quant_type))
    if fn is None:
        raise ValueError(f"no synthetic quantizer for GGML type id {quant_type}")
    elems = GGML_QUANT_SIZES[int(quant_type)][0]
    if w.shape[-1] % elems:
        raise ValueError(f"last dimension {w.shape[-1]} is not a multiple of {elems}")
    return fn(w)
