"""CPU oracle for the GGUF block formats on the quantized-weight matmul path.

TEST INFRASTRUCTURE.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import this module; the product (the HIP library and the host package) never does.

The reference never decodes blocks itself: it calls ``dequantize_gguf_tensor`` of the transformers
``gguf`` fork (fast_moe_lora.py:163-165, 235-240; test_fast_lora.py:110-115) and hands packed bytes
to ``torch_ggml_ops`` (fast_lora.py:154-160).  Neither dependency is vendored or pinned, so the
decoders below restate the published ggml block layouts (ggml-common.h / ggml-quants.c
``dequantize_row_*``; the same arithmetic as gguf-py ``gguf/quants.py``):

  type      id  block bytes  elements  layout
  Q8_0       8      34          32     f16 d; i8 qs[32]
  Q2_K      10      84         256     u8 scales[16]; u8 qs[64]; f16 d; f16 dmin
  Q3_K      11     110         256     u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d
  Q4_K      12     144         256     f16 d; f16 dmin; u8 scales[12]; u8 qs[128]
  Q5_K      13     176         256     f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]
  Q6_K      14     210         256     u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d
  IQ2_XXS   16      66         256     f16 d; u16 qs[32]

All decoders return float32 values that are *exact* products (Q3_K included) except Q2_K, Q4_K and Q5_K, whose
``d*sc*q - dmin*m`` rounds once to float32 (d*sc, dmin*m and (d*sc)*q are exact: 11+6+4 significand bits).  The bf16
weights the matmul oracles use are ``round-to-nearest-even(float32 value)``.

Pinned by: hand-computed known-answer blocks and format invariants in tests/test_oracle_blocks.py and
the independent C restatement oracle/ggml_dequant.c.  parity unpinned: no file in the build
environment holds upstream decoder output (the reference stores no golden vectors, .gitignore:11),
and the IQ2_XXS codebook values are restated from memory of the public table (see iq2xxs_grid.py).

The quantizers here only manufacture valid synthetic payloads from float weights (BASELINE configs:
"drawn from N(0, 0.02^2) and quantized to ..."); they are simple min/max fits, not ggml's search.
Q8_0 follows gguf-py ``quantize`` exactly (used by test_deepseek_v4_lora.py:36-40).
"""

from __future__ import annotations

import numpy as np

from .iq2xxs_grid import IQ2XXS_GRID

Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, IQ2_XXS = 8, 10, 11, 12, 13, 14, 16
# (elements per block, bytes per block); matches gguf.GGML_QUANT_SIZES used at
# test_deepseek_v4_moe_lora.py:58.
QUANT_SIZES = {Q8_0: (32, 34), Q2_K: (256, 84), Q3_K: (256, 110), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210), IQ2_XXS: (256, 66)}

_GRID_BYTES = np.array(IQ2XXS_GRID, dtype=np.uint64).view(np.uint8).reshape(256, 8)  # little endian
# ksigns_iq2xs[i] = i | (parity(i) << 7): the eighth sign makes the number of minus signs even.
_KSIGNS = np.array([i | ((bin(i).count("1") & 1) << 7) for i in range(128)], dtype=np.uint8)


def row_bytes(qt: int, k: int) -> int:
    elems, nbytes = QUANT_SIZES[qt]
    if k % elems:
        raise ValueError(f"K={k} is not a multiple of the {elems}-element block of type {qt}")
    return k // elems * nbytes


def _f16(raw: np.ndarray) -> np.ndarray:
    """Two bytes (little endian) -> float32 value of the IEEE half."""
    return np.ascontiguousarray(raw).view(np.float16).astype(np.float32)


# --------------------------------------------------------------------------------------------
# decoders: payload uint8 [..., row_bytes] -> float32 [..., K]
# --------------------------------------------------------------------------------------------
def dequantize(payload: np.ndarray, qt: int) -> np.ndarray:
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    elems, nbytes = QUANT_SIZES[qt]
    if payload.shape[-1] % nbytes:
        raise ValueError("payload row is not a whole number of blocks")
    lead = payload.shape[:-1]
    blocks = payload.reshape(-1, nbytes)
    out = {Q8_0: _deq_q8_0, Q2_K: _deq_q2_k, Q3_K: _deq_q3_k, Q4_K: _deq_q4_k, Q5_K: _deq_q5_k, Q6_K: _deq_q6_k, IQ2_XXS: _deq_iq2_xxs}[qt](blocks)
    return out.reshape(*lead, payload.shape[-1] // nbytes * elems)


def _deq_q8_0(b: np.ndarray) -> np.ndarray:
    d = _f16(b[:, 0:2])                                    # [nb,1]
    q = b[:, 2:34].view(np.int8).astype(np.float32)
    return d * q


def unpack_q4_k_scales(s: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """12 packed bytes -> (sc[8], m[8]) 6-bit values (ggml get_scale_min_k4)."""
    s = s.astype(np.uint8)
    sc = np.empty(s.shape[:-1] + (8,), dtype=np.uint8)
    m = np.empty_like(sc)
    sc[..., 0:4] = s[..., 0:4] & 63
    m[..., 0:4] = s[..., 4:8] & 63
    sc[..., 4:8] = (s[..., 8:12] & 0x0F) | ((s[..., 0:4] >> 6) << 4)
    m[..., 4:8] = (s[..., 8:12] >> 4) | ((s[..., 4:8] >> 6) << 4)
    return sc, m


def _deq_q4_k(b: np.ndarray) -> np.ndarray:
    nb = b.shape[0]
    d = _f16(b[:, 0:2])
    dmin = _f16(b[:, 2:4])
    sc, m = unpack_q4_k_scales(b[:, 4:16])
    dl = d * sc.astype(np.float32)                         # [nb,8] exact
    ml = dmin * m.astype(np.float32)
    qs = b[:, 16:144].reshape(nb, 4, 32)
    q = np.empty((nb, 4, 2, 32), dtype=np.float32)
    q[:, :, 0, :] = (qs & 0x0F)                            # first 32 of each 64: low nibbles
    q[:, :, 1, :] = (qs >> 4)                              # next 32: high nibbles
    q = q.reshape(nb, 8, 32)
    y = dl[:, :, None] * q                                 # exact in float32
    y = y - ml[:, :, None]                                 # one float32 rounding
    return y.reshape(nb, 256)


def _deq_q5_k(b: np.ndarray) -> np.ndarray:
    """Q4_K's layout with a fifth bit per element: bit 2c (+1 for the high nibbles) of qh[l] belongs to element l of
    the c-th 64-element chunk (ggml dequantize_row_q5_K)."""
    nb = b.shape[0]
    d = _f16(b[:, 0:2])
    dmin = _f16(b[:, 2:4])
    sc, m = unpack_q4_k_scales(b[:, 4:16])
    dl = d * sc.astype(np.float32)
    ml = dmin * m.astype(np.float32)
    qh = b[:, 16:48]                                        # [nb,32]
    qs = b[:, 48:176].reshape(nb, 4, 32)
    q = np.empty((nb, 4, 2, 32), dtype=np.float32)
    for c in range(4):
        q[:, c, 0, :] = (qs[:, c, :] & 0x0F) + (((qh >> (2 * c)) & 1) << 4)
        q[:, c, 1, :] = (qs[:, c, :] >> 4) + (((qh >> (2 * c + 1)) & 1) << 4)
    q = q.reshape(nb, 8, 32)
    y = dl[:, :, None] * q                                 # exact in float32 (11 + 6 + 5 bits)
    y = y - ml[:, :, None]                                 # one float32 rounding
    return y.reshape(nb, 256)


def unpack_q3_k_scales(s: np.ndarray) -> np.ndarray:
    """12 packed bytes -> sixteen signed scales (6-bit value - 32): scale k keeps its low four bits in nibble k // 8 of
    byte (k // 4 % 2) * 4 + k % 4 and its high two bits at position 2 (k // 4) of byte 8 + k % 4."""
    s = s.astype(np.int32)
    out = np.empty(s.shape[:-1] + (16,), dtype=np.int32)
    for k in range(16):
        low = (s[..., (k // 4 % 2) * 4 + k % 4] >> (4 * (k // 8))) & 0xF
        high = (s[..., 8 + k % 4] >> (2 * (k // 4))) & 3
        out[..., k] = (low | (high << 4)) - 32
    return out


def _deq_q3_k(b: np.ndarray) -> np.ndarray:
    """Sixteen 16-element sub-blocks with signed 6-bit scales; element 128 n + 32 j + l is bits 2j..2j+1 of
    qs[32 n + l], minus 4 unless bit 4 n + j of hmask[l] is set (ggml dequantize_row_q3_K)."""
    nb = b.shape[0]
    hm = b[:, 0:32]
    qs = b[:, 32:96].reshape(nb, 2, 32)
    d = _f16(b[:, 108:110])
    dl = d * unpack_q3_k_scales(b[:, 96:108]).astype(np.float32)     # [nb,16] exact
    q = np.empty((nb, 2, 4, 32), dtype=np.float32)
    for n in range(2):
        for j in range(4):
            low = ((qs[:, n, :] >> (2 * j)) & 3).astype(np.int32)
            high = ((hm >> (4 * n + j)) & 1).astype(np.int32)
            q[:, n, j, :] = low - 4 * (1 - high)
    return (dl[:, :, None] * q.reshape(nb, 16, 16)).reshape(nb, 256)


def _deq_q2_k(b: np.ndarray) -> np.ndarray:
    """Sixteen 16-element sub-blocks, each with a 4-bit scale (low nibble) and a 4-bit min (high nibble); element
    128 n + 32 j + l is bits 2j..2j+1 of qs[32 n + l] (ggml dequantize_row_q2_K)."""
    nb = b.shape[0]
    scales = b[:, 0:16]
    qs = b[:, 16:80].reshape(nb, 2, 32)
    d = _f16(b[:, 80:82])
    dmin = _f16(b[:, 82:84])
    dl = d * (scales & 0x0F).astype(np.float32)            # [nb,16] exact
    ml = dmin * (scales >> 4).astype(np.float32)
    q = np.empty((nb, 2, 4, 32), dtype=np.float32)
    for j in range(4):
        q[:, :, j, :] = (qs >> (2 * j)) & 3
    q = q.reshape(nb, 16, 16)                              # sub-block 8 n + 2 j + (l >= 16)
    y = dl[:, :, None] * q - ml[:, :, None]
    return y.reshape(nb, 256)


def _deq_q6_k(b: np.ndarray) -> np.ndarray:
    nb = b.shape[0]
    ql = b[:, 0:128].reshape(nb, 2, 64)
    qh = b[:, 128:192].reshape(nb, 2, 32)
    sc = b[:, 192:208].view(np.int8).astype(np.float32)    # [nb,16]
    d = _f16(b[:, 208:210])
    q = np.empty((nb, 2, 4, 32), dtype=np.int32)
    q[:, :, 0, :] = (ql[:, :, 0:32] & 0x0F) | (((qh >> 0) & 3) << 4)
    q[:, :, 1, :] = (ql[:, :, 32:64] & 0x0F) | (((qh >> 2) & 3) << 4)
    q[:, :, 2, :] = (ql[:, :, 0:32] >> 4) | (((qh >> 4) & 3) << 4)
    q[:, :, 3, :] = (ql[:, :, 32:64] >> 4) | (((qh >> 6) & 3) << 4)
    q = (q - 32).astype(np.float32).reshape(nb, 16, 16)    # element e -> sub-scale e // 16
    y = (d * sc)[:, :, None] * q
    return y.reshape(nb, 256)


def _deq_iq2_xxs(b: np.ndarray) -> np.ndarray:
    nb = b.shape[0]
    d = _f16(b[:, 0:2])                                    # [nb,1]
    g = b[:, 2:66].reshape(nb, 8, 8)                       # eight 8-byte groups of 32 elements
    idx = g[:, :, 0:4]                                     # four codebook indices
    aux = np.ascontiguousarray(g[:, :, 4:8]).view(np.uint32).reshape(nb, 8)
    db = d * (0.5 + (aux >> 28).astype(np.float32)) * 0.25  # [nb,8]
    sign_idx = (aux[:, :, None] >> (7 * np.arange(4, dtype=np.uint32))) & 127    # [nb,8,4]
    signs = _KSIGNS[sign_idx]                              # [nb,8,4] eight sign bits each
    neg = (signs[..., None] >> np.arange(8, dtype=np.uint8)) & 1                 # [nb,8,4,8]
    mag = _GRID_BYTES[idx].astype(np.float32)              # [nb,8,4,8]
    y = db[:, :, None, None] * mag * np.where(neg == 1, np.float32(-1), np.float32(1))
    return y.reshape(nb, 256).astype(np.float32)


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit pattern (uint16), round to nearest even (torch ``.to(bfloat16)``)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = (u + (np.uint32(0x7FFF) + ((u >> 16) & 1))) >> 16
    return rounded.astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def dequantize_bf16(payload: np.ndarray, qt: int) -> np.ndarray:
    """Decoded weights rounded to bf16, returned as float32 values."""
    return bf16_bits_to_f32(to_bf16_bits(dequantize(payload, qt)))


# --------------------------------------------------------------------------------------------
# quantizers (synthetic payload factories): float32 [..., K] -> uint8 [..., row_bytes]
# --------------------------------------------------------------------------------------------
def _roundf(x: np.ndarray) -> np.ndarray:
    """C roundf: half away from zero (gguf-py ``np_roundf``)."""
    a = np.abs(x)
    return np.sign(x) * np.floor(a + np.float32(0.5))


def _f16_bytes(x: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(x.astype(np.float16)).view(np.uint8)


def quantize(w: np.ndarray, qt: int) -> np.ndarray:
    w = np.ascontiguousarray(w, dtype=np.float32)
    elems, nbytes = QUANT_SIZES[qt]
    if w.shape[-1] % elems:
        raise ValueError(f"last dim {w.shape[-1]} is not a multiple of {elems}")
    lead = w.shape[:-1]
    blocks = w.reshape(-1, elems)
    out = {Q8_0: _q_q8_0, Q2_K: _q_q2_k, Q3_K: _q_q3_k, Q4_K: _q_q4_k, Q5_K: _q_q5_k, Q6_K: _q_q6_k, IQ2_XXS: _q_iq2_xxs}[qt](blocks)
    return out.reshape(*lead, w.shape[-1] // elems * nbytes)


def _q_q8_0(x: np.ndarray) -> np.ndarray:
    d = np.abs(x).max(axis=1, keepdims=True) / np.float32(127)
    with np.errstate(divide="ignore"):
        inv = np.where(d == 0, np.float32(0), np.float32(1) / d).astype(np.float32)
    q = _roundf(x * inv).astype(np.int8)
    out = np.empty((x.shape[0], 34), dtype=np.uint8)
    out[:, 0:2] = _f16_bytes(d).reshape(-1, 2)
    out[:, 2:] = q.view(np.uint8)
    return out


def pack_q4_k_scales(sc: np.ndarray, m: np.ndarray) -> np.ndarray:
    sc = sc.astype(np.uint8)
    m = m.astype(np.uint8)
    s = np.empty(sc.shape[:-1] + (12,), dtype=np.uint8)
    s[..., 0:4] = sc[..., 0:4] | ((sc[..., 4:8] >> 4) << 6)
    s[..., 4:8] = m[..., 0:4] | ((m[..., 4:8] >> 4) << 6)
    s[..., 8:12] = (sc[..., 4:8] & 0x0F) | ((m[..., 4:8] & 0x0F) << 4)
    return s


def _q_q4_k(x: np.ndarray) -> np.ndarray:
    nb = x.shape[0]
    sub = x.reshape(nb, 8, 32)
    lo = np.minimum(sub.min(axis=2), 0)
    hi = sub.max(axis=2)
    scale = (hi - lo) / np.float32(15)
    off = -lo
    d = (scale.max(axis=1, keepdims=True) / np.float32(63)).astype(np.float16).astype(np.float32)
    dmin = (off.max(axis=1, keepdims=True) / np.float32(63)).astype(np.float16).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(d > 0, np.clip(_roundf(scale / d), 0, 63), 0).astype(np.uint8)
        m = np.where(dmin > 0, np.clip(_roundf(off / dmin), 0, 63), 0).astype(np.uint8)
        dl = d * sc.astype(np.float32)
        ml = dmin * m.astype(np.float32)
        q = np.where(dl[:, :, None] > 0, _roundf((sub + ml[:, :, None]) / dl[:, :, None]), 0)
    q = np.clip(q, 0, 15).astype(np.uint8).reshape(nb, 4, 2, 32)
    out = np.empty((nb, 144), dtype=np.uint8)
    out[:, 0:2] = _f16_bytes(d).reshape(-1, 2)
    out[:, 2:4] = _f16_bytes(dmin).reshape(-1, 2)
    out[:, 4:16] = pack_q4_k_scales(sc, m)
    out[:, 16:] = (q[:, :, 0, :] | (q[:, :, 1, :] << 4)).reshape(nb, 128)
    return out


def _q_q5_k(x: np.ndarray) -> np.ndarray:
    nb = x.shape[0]
    sub = x.reshape(nb, 8, 32)
    lo = np.minimum(sub.min(axis=2), 0)
    hi = sub.max(axis=2)
    scale = (hi - lo) / np.float32(31)
    off = -lo
    d = (scale.max(axis=1, keepdims=True) / np.float32(63)).astype(np.float16).astype(np.float32)
    dmin = (off.max(axis=1, keepdims=True) / np.float32(63)).astype(np.float16).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(d > 0, np.clip(_roundf(scale / d), 0, 63), 0).astype(np.uint8)
        m = np.where(dmin > 0, np.clip(_roundf(off / dmin), 0, 63), 0).astype(np.uint8)
        dl = d * sc.astype(np.float32)
        ml = dmin * m.astype(np.float32)
        q = np.where(dl[:, :, None] > 0, _roundf((sub + ml[:, :, None]) / dl[:, :, None]), 0)
    q = np.clip(q, 0, 31).astype(np.uint8).reshape(nb, 4, 2, 32)
    out = np.empty((nb, 176), dtype=np.uint8)
    out[:, 0:2] = _f16_bytes(d).reshape(-1, 2)
    out[:, 2:4] = _f16_bytes(dmin).reshape(-1, 2)
    out[:, 4:16] = pack_q4_k_scales(sc, m)
    qh = np.zeros((nb, 32), dtype=np.uint8)
    for c in range(4):
        qh |= ((q[:, c, 0, :] >> 4) << (2 * c)) | ((q[:, c, 1, :] >> 4) << (2 * c + 1))
    out[:, 16:48] = qh
    out[:, 48:] = ((q[:, :, 0, :] & 0x0F) | ((q[:, :, 1, :] & 0x0F) << 4)).reshape(nb, 128)
    return out


def _q_q2_k(x: np.ndarray) -> np.ndarray:
    nb = x.shape[0]
    sub = x.reshape(nb, 16, 16)
    lo = np.minimum(sub.min(axis=2), 0)
    hi = sub.max(axis=2)
    scale = (hi - lo) / np.float32(3)
    off = -lo
    d = (scale.max(axis=1, keepdims=True) / np.float32(15)).astype(np.float16).astype(np.float32)
    dmin = (off.max(axis=1, keepdims=True) / np.float32(15)).astype(np.float16).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(d > 0, np.clip(_roundf(scale / d), 0, 15), 0).astype(np.uint8)
        m = np.where(dmin > 0, np.clip(_roundf(off / dmin), 0, 15), 0).astype(np.uint8)
        dl = d * sc.astype(np.float32)
        ml = dmin * m.astype(np.float32)
        q = np.where(dl[:, :, None] > 0, _roundf((sub + ml[:, :, None]) / dl[:, :, None]), 0)
    q = np.clip(q, 0, 3).astype(np.uint8).reshape(nb, 2, 4, 32)   # [n, j, l]: element 128 n + 32 j + l
    out = np.empty((nb, 84), dtype=np.uint8)
    out[:, 0:16] = sc | (m << 4)
    qs = np.zeros((nb, 2, 32), dtype=np.uint8)
    for j in range(4):
        qs |= q[:, :, j, :] << (2 * j)
    out[:, 16:80] = qs.reshape(nb, 64)
    out[:, 80:82] = _f16_bytes(d).reshape(-1, 2)
    out[:, 82:84] = _f16_bytes(dmin).reshape(-1, 2)
    return out


def _q_q3_k(x: np.ndarray) -> np.ndarray:
    nb = x.shape[0]
    sub = x.reshape(nb, 16, 16)
    scale = np.abs(sub).max(axis=2) / np.float32(4)
    d = (scale.max(axis=1, keepdims=True) / np.float32(31)).astype(np.float16).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(d > 0, np.clip(_roundf(scale / d), 0, 31), 0).astype(np.int32)
        dl = d * sc.astype(np.float32)
        q = np.where(dl[:, :, None] > 0, _roundf(sub / dl[:, :, None]), 0)
    v = (np.clip(q, -4, 3).astype(np.int32) + 4).astype(np.uint8).reshape(nb, 2, 4, 32)   # [n, j, l]: element 128 n + 32 j + l
    out = np.zeros((nb, 110), dtype=np.uint8)
    hm = np.zeros((nb, 32), dtype=np.uint8)
    qs = np.zeros((nb, 2, 32), dtype=np.uint8)
    for n in range(2):
        for j in range(4):
            qs[:, n, :] |= (v[:, n, j, :] & 3) << (2 * j)
            hm |= (v[:, n, j, :] >> 2) << (4 * n + j)
    out[:, 0:32] = hm
    out[:, 32:96] = qs.reshape(nb, 64)
    s6 = (sc + 32).astype(np.uint8)
    for k in range(16):
        out[:, 96 + (k // 4 % 2) * 4 + k % 4] |= (s6[:, k] & 0xF) << (4 * (k // 8))
        out[:, 104 + k % 4] |= (s6[:, k] >> 4) << (2 * (k // 4))
    out[:, 108:110] = _f16_bytes(d).reshape(-1, 2)
    return out


def _q_q6_k(x: np.ndarray) -> np.ndarray:
    nb = x.shape[0]
    sub = x.reshape(nb, 16, 16)
    scale = np.abs(sub).max(axis=2) / np.float32(31)
    d = (scale.max(axis=1, keepdims=True) / np.float32(127)).astype(np.float16).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(d > 0, np.clip(_roundf(scale / d), 0, 127), 0).astype(np.int8)
        dl = d * sc.astype(np.float32)
        q = np.where(dl[:, :, None] != 0, _roundf(sub / dl[:, :, None]), 0)
    q = (np.clip(q, -32, 31) + 32).astype(np.uint8).reshape(nb, 2, 4, 32)
    ql = np.empty((nb, 2, 64), dtype=np.uint8)
    ql[:, :, 0:32] = (q[:, :, 0] & 0x0F) | ((q[:, :, 2] & 0x0F) << 4)
    ql[:, :, 32:64] = (q[:, :, 1] & 0x0F) | ((q[:, :, 3] & 0x0F) << 4)
    qh = (q[:, :, 0] >> 4) | ((q[:, :, 1] >> 4) << 2) | ((q[:, :, 2] >> 4) << 4) | ((q[:, :, 3] >> 4) << 6)
    out = np.empty((nb, 210), dtype=np.uint8)
    out[:, 0:128] = ql.reshape(nb, 128)
    out[:, 128:192] = qh.reshape(nb, 64)
    out[:, 192:208] = sc.view(np.uint8)
    out[:, 208:210] = _f16_bytes(d).reshape(-1, 2)
    return out


def _q_iq2_xxs(x: np.ndarray) -> np.ndarray:
    nb = x.shape[0]
    grp = x.reshape(nb, 8, 32)
    amax = np.abs(grp).max(axis=2)                          # [nb,8]
    db_want = amax / np.float32(33)
    d = (db_want.max(axis=1, keepdims=True) * np.float32(4.0 / 15.5)).astype(np.float16).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        ls = np.where(d > 0, np.clip(_roundf(db_want * 4 / d - np.float32(0.5)), 0, 15), 0).astype(np.uint32)
    db = d * (np.float32(0.5) + ls.astype(np.float32)) * np.float32(0.25)
    v = grp.reshape(nb, 8, 4, 8)
    neg = v < 0
    mag = np.abs(v)
    odd = (neg.sum(axis=3) & 1).astype(bool)                # need an even number of minus signs
    weakest = mag.argmin(axis=3)
    flip = np.zeros_like(neg)
    np.put_along_axis(flip, weakest[..., None], odd[..., None], axis=3)
    neg = neg ^ flip
    with np.errstate(divide="ignore", invalid="ignore"):
        t = np.where(db[:, :, None, None] > 0, mag / db[:, :, None, None], 0).astype(np.float32)
    grid = _GRID_BYTES.astype(np.float64)                   # [256,8]
    # nearest codebook point: argmin |t|^2 - 2 t.g + |g|^2, in double precision (so that a restatement whose products are
    # summed in another order picks the same point), a million groups at a time
    norms = (grid * grid).sum(axis=1)[None, :]
    tt = t.reshape(-1, 8)
    idx = np.empty(tt.shape[0], dtype=np.uint8)
    for lo in range(0, tt.shape[0], 1 << 20):
        idx[lo:lo + (1 << 20)] = (norms - 2.0 * (tt[lo:lo + (1 << 20)].astype(np.float64) @ grid.T)).argmin(axis=1)
    idx = idx.reshape(nb, 8, 4)
    sign7 = (neg[..., 0:7].astype(np.uint32) << np.arange(7, dtype=np.uint32)).sum(axis=3)   # [nb,8,4]
    aux1 = (ls << 28) | (sign7 << (7 * np.arange(4, dtype=np.uint32))).sum(axis=2).astype(np.uint32)
    out = np.empty((nb, 66), dtype=np.uint8)
    out[:, 0:2] = _f16_bytes(d).reshape(-1, 2)
    body = np.empty((nb, 8, 8), dtype=np.uint8)
    body[:, :, 0:4] = idx
    body[:, :, 4:8] = np.ascontiguousarray(aux1.astype(np.uint32)).view(np.uint8).reshape(nb, 8, 4)
    out[:, 2:] = body.reshape(nb, 64)
    return out


def random_payload(rng: np.random.Generator, qt: int, rows: int, k: int, std: float = 0.02) -> np.ndarray:
    """Arbitrary-byte payload with sane half-precision scales: every byte pattern is a valid block,
    so this exercises all scale/min/sign/index encodings (negative Q6_K sub-scales, all 6-bit Q4_K
    scale splits) that the min/max quantizers never emit."""
    elems, nbytes = QUANT_SIZES[qt]
    nb = rows * (k // elems)
    b = rng.integers(0, 256, size=(nb, nbytes), dtype=np.uint8)
    mag = {Q8_0: std / 64, Q2_K: std / 25, Q3_K: std / 60, Q4_K: std / 250, Q5_K: std / 800, Q6_K: std / 1500, IQ2_XXS: std / 60}[qt]
    d = (mag * (0.5 + rng.random(nb))).astype(np.float32)
    if qt == Q6_K:
        b[:, 208:210] = _f16_bytes(d).reshape(-1, 2)
    elif qt == Q3_K:
        b[:, 108:110] = _f16_bytes(d).reshape(-1, 2)
    elif qt == Q2_K:
        b[:, 80:82] = _f16_bytes(d).reshape(-1, 2)
        b[:, 82:84] = _f16_bytes(d * np.float32(0.7)).reshape(-1, 2)
    else:
        b[:, 0:2] = _f16_bytes(d).reshape(-1, 2)
    if qt in (Q4_K, Q5_K):
        b[:, 2:4] = _f16_bytes(d * np.float32(0.7)).reshape(-1, 2)
    return b.reshape(rows, k // elems * nbytes)
