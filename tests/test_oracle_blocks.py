"""Pins for the block-decoder oracle: hand-computed known-answer blocks (derived on paper from the
published ggml block layouts, not by re-running the decoder's formula), the independent scalar C
restatement, format invariants and structural checks of the IQ2_XXS codebook."""

import numpy as np
import pytest

from oracle import c_oracle
from oracle import gguf_blocks as gb
from oracle.iq2xxs_grid import IQ2XXS_GRID

F16 = {1.0: (0x00, 0x3C), 0.5: (0x00, 0x38), 0.25: (0x00, 0x34)}


def both(payload, qt):
    a = gb.dequantize(payload, qt)
    b = c_oracle.dequantize(payload, qt)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), "numpy and C restatements disagree"
    return a


def test_q8_0_known_answer():
    blk = np.zeros(34, dtype=np.uint8)
    blk[0:2] = F16[0.5]
    q = np.zeros(32, dtype=np.int8)
    q[:5] = [-128, -1, 0, 1, 127]
    q[31] = 64
    blk[2:] = q.view(np.uint8)
    y = both(blk[None, :], gb.Q8_0)[0]
    assert y[:5].tolist() == [-64.0, -0.5, 0.0, 0.5, 63.5]
    assert y[31] == 32.0 and np.all(y[5:31] == 0)


def test_q4_k_known_answer():
    # d = 1, dmin = 0.5; sub-block scales sc = 1,2,3,4,33,34,35,36 and mins m = 5,6,7,8,37,38,39,40
    # packed by hand into the 12 scale bytes (6-bit fields, upper two bits of sc[4..7] / m[4..7] in the
    # tops of bytes 0..7); qs[i] = (i % 16) | ((15 - i % 16) << 4).
    blk = np.zeros(144, dtype=np.uint8)
    blk[0:2] = F16[1.0]
    blk[2:4] = F16[0.5]
    blk[4:16] = [129, 130, 131, 132, 133, 134, 135, 136, 81, 98, 115, 132]
    i = np.arange(128)
    blk[16:] = (i % 16) | ((15 - i % 16) << 4)
    y = both(blk[None, :], gb.Q4_K)[0]
    want = {0: -2.5, 5: 2.5, 32: 27.0, 47: -3.0, 64: -3.5, 79: 41.5, 128: -18.5, 131: 80.5, 224: 520.0, 255: -20.0}
    for e, v in want.items():
        assert y[e] == v, (e, y[e], v)


def test_q5_k_known_answer():
    # Same d, dmin and scale bytes as the Q4_K block above (sc = 1,2,3,4,33,34,35,36, m = 5..8,37..40) and
    # the same nibbles; qh[l] = 0xA5 for even l and 0x5A for odd l.  Sub-block s takes its fifth bit from
    # bit s of qh[l], so even l sees bits {0,2,5,7} set and odd l bits {1,3,4,6}.
    blk = np.zeros(176, dtype=np.uint8)
    blk[0:2] = F16[1.0]
    blk[2:4] = F16[0.5]
    blk[4:16] = [129, 130, 131, 132, 133, 134, 135, 136, 81, 98, 115, 132]
    blk[16:48] = [0xA5, 0x5A] * 16
    i = np.arange(128)
    blk[48:] = (i % 16) | ((15 - i % 16) << 4)
    y = both(blk[None, :], gb.Q5_K)[0]
    want = {0: 13.5, 1: -1.5, 32: 27.0, 33: 57.0, 64: 44.5, 111: 60.0, 128: -18.5, 131: 608.5,
            192: -19.5, 193: 575.5, 224: 1096.0, 255: -20.0}
    for e, v in want.items():
        assert y[e] == v, (e, y[e], v)


def test_q3_k_known_answer():
    # d = 0.5; 6-bit scales 24..39 (signed -8..7), packed by hand: low nibbles 8..15 in the low halves of bytes 0..7,
    # 0..7 in their high halves, the upper two bits (1,1,2,2 per group of four) as 0xA5 in bytes 8..11; qs as in the
    # Q2_K block; hmask[l] = 0xA5 for even l, 0x5A for odd l (a clear bit subtracts 4).
    blk = np.zeros(110, dtype=np.uint8)
    blk[0:32] = [0xA5, 0x5A] * 16
    blk[32:96] = [0xE4, 0x1B] * 32
    blk[96:108] = [0x08, 0x19, 0x2A, 0x3B, 0x4C, 0x5D, 0x6E, 0x7F, 0xA5, 0xA5, 0xA5, 0xA5]
    blk[108:110] = F16[0.5]
    assert gb.unpack_q3_k_scales(blk[96:108]).tolist() == list(range(-8, 8))
    y = both(blk[None, :], gb.Q3_K)[0]
    want = {0: 0.0, 1: 4.0, 17: 3.5, 32: 9.0, 33: -6.0, 96: 1.0, 127: 0.0, 128: 0.0, 160: 1.0, 177: -3.0,
            254: 10.5, 255: -14.0}
    for e, v in want.items():
        assert y[e] == v, (e, y[e], v)


def test_q2_k_known_answer():
    # d = 0.5, dmin = 0.25; scales[k] = k | (15-k) << 4 (scale k, min 15-k); qs = 0xE4 at even bytes
    # (bit pairs 0,1,2,3 from the bottom) and 0x1B at odd bytes (3,2,1,0).
    blk = np.zeros(84, dtype=np.uint8)
    k = np.arange(16)
    blk[0:16] = k | ((15 - k) << 4)
    blk[16:80] = [0xE4, 0x1B] * 32
    blk[80:82] = F16[0.5]
    blk[82:84] = F16[0.25]
    y = both(blk[None, :], gb.Q2_K)[0]
    want = {0: -3.75, 17: -2.0, 32: -2.25, 49: 0.0, 96: 6.75, 127: -2.0, 128: -1.75, 145: 12.0,
            254: 22.5, 255: 0.0}
    for e, v in want.items():
        assert y[e] == v, (e, y[e], v)


def test_q6_k_known_answer():
    # d = 0.25; int8 sub-scales 1,-2,3,-4,...,15,-16; ql = 0x21 for l < 32 and 0x43 for l >= 32 of each
    # 64-byte half; qh = 0xE4 (bit pairs 0,1,2,3 from the bottom).
    blk = np.zeros(210, dtype=np.uint8)
    ql = np.empty(128, dtype=np.uint8)
    ql[0:32] = 0x21
    ql[32:64] = 0x43
    ql[64:96] = 0x21
    ql[96:128] = 0x43
    blk[0:128] = ql
    blk[128:192] = 0xE4
    sc = np.array([(j + 1) * (1 if j % 2 == 0 else -1) for j in range(16)], dtype=np.int8)
    blk[192:208] = sc.view(np.uint8)
    blk[208:210] = F16[0.25]
    y = both(blk[None, :], gb.Q6_K)[0]
    want = {0: -7.75, 16: 15.5, 32: -9.75, 64: 2.5, 96: 35.0, 127: -40.0, 128: -69.75, 255: -80.0}
    for e, v in want.items():
        assert y[e] == v, (e, y[e], v)


def test_iq2_xxs_constant_byte_payload_known_answer():
    # every byte 32: the synthetic expert payload of test_deepseek_v4_moe_lora.py:55-64.
    # d = half(0x2020) = 2^-7 * (1 + 32/1024); scale nibble 2 -> db = d * 2.5 / 4; all four codebook
    # indices are 32 -> bytes 25,8,8,8,8,25,8,8; sign indices 32, 64, 0, 1 (+ parity bit 7).
    payload = np.full((1, 66), 32, dtype=np.uint8)
    y = both(payload, gb.IQ2_XXS)[0]
    a, b = 0.125885009765625, 0.040283203125  # db * 25, db * 8
    run0 = [a, b, b, b, b, -a, b, -b]
    run1 = [a, b, b, b, b, a, -b, -b]
    run2 = [a, b, b, b, b, a, b, b]
    run3 = [-a, b, b, b, b, a, b, -b]
    assert y[:32].tolist() == run0 + run1 + run2 + run3
    assert np.array_equal(y[:32], y[224:256])  # all eight groups are identical


def test_iq2xxs_grid_structure():
    g = np.array(IQ2XXS_GRID, dtype=np.uint64)
    assert g.shape == (256,) and np.all(g[1:] > g[:-1]) and int(g[0]) == 0x0808080808080808
    b = g.view(np.uint8).reshape(256, 8)
    assert set(np.unique(b).tolist()) == {0x08, 0x19, 0x2B}
    assert np.all((b == 0x19).sum(axis=1) % 2 == 0)  # E8 lattice points (half-integer coset)
    n19, n2b = (b == 0x19).sum(axis=1), (b == 0x2B).sum(axis=1)
    assert int(((n19 == 2) & (n2b == 0)).sum()) == 28 and int(((n19 == 0) & (n2b == 1)).sum()) == 8


# The same 256 points in a second encoding, typed separately from the byte table: eight 2-bit digits per point, least
# significant first, digit 0 / 1 / 2 = magnitude 0x08 / 0x19 / 0x2b (the form in which the public ggml quantizer source lists
# its IQ2_XXS lattice points).  It pins nothing against upstream, but a typing slip in one entry of either table fails here.
_IQ2XXS_GRID_DIGITS = (
    0, 2, 5, 8, 10, 17, 20, 32, 34, 40, 42, 65, 68, 80, 88, 97,
    100, 128, 130, 138, 162, 257, 260, 272, 277, 320, 388, 408, 512, 514, 546, 642,
    1025, 1028, 1040, 1057, 1060, 1088, 1090, 1096, 1120, 1153, 1156, 1168, 1188, 1280, 1282, 1288,
    1312, 1350, 1385, 1408, 1425, 1545, 1552, 1600, 1668, 1700, 2048, 2053, 2056, 2068, 2088, 2113,
    2116, 2128, 2130, 2184, 2308, 2368, 2562, 2580, 4097, 4100, 4112, 4129, 4160, 4192, 4228, 4240,
    4245, 4352, 4360, 4384, 4432, 4442, 4480, 4644, 4677, 5120, 5128, 5152, 5157, 5193, 5248, 5400,
    5474, 5632, 5654, 6145, 6148, 6160, 6208, 6273, 6400, 6405, 6560, 6737, 8192, 8194, 8202, 8260,
    8289, 8320, 8322, 8489, 8520, 8704, 8706, 9217, 9220, 9232, 9280, 9302, 9472, 9537, 9572, 9872,
    10248, 10272, 10388, 10820, 16385, 16388, 16400, 16408, 16417, 16420, 16448, 16456, 16470, 16480, 16513, 16516,
    16528, 16640, 16672, 16737, 16768, 16773, 16897, 16912, 16968, 16982, 17000, 17408, 17416, 17440, 17536, 17561,
    17682, 17700, 17920, 18433, 18436, 18448, 18496, 18501, 18688, 18776, 18785, 18818, 19013, 19088, 20480, 20488,
    20497, 20505, 20512, 20608, 20616, 20740, 20802, 20900, 21137, 21648, 21650, 21770, 22017, 22100, 22528, 22545,
    22553, 22628, 22848, 23048, 24580, 24592, 24640, 24680, 24832, 24917, 25112, 25184, 25600, 25605, 25872, 25874,
    25988, 26690, 32768, 32770, 32778, 32833, 32898, 33028, 33048, 33088, 33297, 33793, 33796, 33808, 33813, 33856,
    33888, 34048, 34118, 34196, 34313, 34368, 34400, 34818, 35076, 35345, 36868, 36880, 36900, 36928, 37025, 37142,
    37248, 37445, 37888, 37922, 37956, 38225, 39041, 39200, 40962, 41040, 41093, 41225, 41472, 42008, 43088, 43268,
)


def test_iq2xxs_grid_agrees_with_its_digit_encoding():
    assert len(_IQ2XXS_GRID_DIGITS) == 256
    magnitude = {0: 0x08, 1: 0x19, 2: 0x2B}
    for i, (digits, point) in enumerate(zip(_IQ2XXS_GRID_DIGITS, IQ2XXS_GRID)):
        expanded = sum(magnitude[(digits >> (2 * j)) & 3] << (8 * j) for j in range(8))  # digit 3 does not occur: KeyError
        assert expanded == point, (i, digits, hex(point))


@pytest.mark.parametrize("qt", [gb.Q8_0, gb.Q2_K, gb.Q3_K, gb.Q4_K, gb.Q5_K, gb.Q6_K, gb.IQ2_XXS])
def test_numpy_and_c_agree_on_arbitrary_bytes(qt):
    payload = gb.random_payload(np.random.default_rng(qt), qt, 23, 1024)
    y = both(payload, qt)
    assert np.isfinite(y).all()
    assert np.array_equal(gb.to_bf16_bits(y), c_oracle.to_bf16_bits(y))


def test_format_invariants():
    rng = np.random.default_rng(3)
    # Q4_K with all-zero quants decodes to -dmin*m per sub-block, whatever d is
    p = gb.random_payload(rng, gb.Q4_K, 1, 256)
    p[0, 16:] = 0
    y = gb.dequantize(p, gb.Q4_K)[0].reshape(8, 32)
    _, m = gb.unpack_q4_k_scales(p[0, 4:16])
    dmin = p[0, 2:4].copy().view(np.float16).astype(np.float32)[0]
    assert np.array_equal(y, np.repeat((-(dmin * m.astype(np.float32)))[:, None], 32, axis=1))
    # Q5_K: clearing qh removes exactly 16*d*sc from the values whose fifth bit was set, and a block with
    # qh = 0 decodes like the Q4_K block made of the same header, scales and nibbles
    p = gb.random_payload(rng, gb.Q5_K, 1, 256)
    q4 = np.concatenate([p[:, :16], p[:, 48:]], axis=1)
    p0 = p.copy()
    p0[0, 16:48] = 0
    assert np.array_equal(gb.dequantize(p0, gb.Q5_K), gb.dequantize(q4, gb.Q4_K))
    sc, _ = gb.unpack_q4_k_scales(p[0, 4:16])
    d = p[0, 0:2].copy().view(np.float16).astype(np.float32)[0]
    bits = ((p[0, 16:48][None, :] >> np.arange(8)[:, None]) & 1).astype(np.float32)  # [sub-block, l]
    step = (d * sc.astype(np.float32))[:, None] * 16.0 * bits
    got = (gb.dequantize(p, gb.Q5_K) - gb.dequantize(p0, gb.Q5_K))[0].reshape(8, 32)
    assert np.allclose(got, step, rtol=1e-6, atol=0)
    # Q2_K with all-zero quants decodes to -dmin*(scales >> 4) per run of sixteen
    p = gb.random_payload(rng, gb.Q2_K, 1, 256)
    p[0, 16:80] = 0
    dmin = p[0, 82:84].copy().view(np.float16).astype(np.float32)[0]
    y = gb.dequantize(p, gb.Q2_K)[0].reshape(16, 16)
    assert np.array_equal(y, np.repeat((-(dmin * (p[0, :16] >> 4).astype(np.float32)))[:, None], 16, axis=1))
    # Q3_K: setting every hmask bit adds exactly 4*d*scale to the values whose bit was clear; negating d negates all
    p = gb.random_payload(rng, gb.Q3_K, 1, 256)
    p1 = p.copy()
    p1[0, 0:32] = 0xFF
    d = p[0, 108:110].copy().view(np.float16).astype(np.float32)[0]
    sc = gb.unpack_q3_k_scales(p[0, 96:108]).astype(np.float32)
    clear = 1.0 - ((p[0, 0:32][None, :] >> np.arange(8)[:, None]) & 1).astype(np.float32)     # [run u, l]
    step = (d * sc).reshape(8, 2)[:, :, None] * 4.0 * clear.reshape(8, 2, 16)
    got = (gb.dequantize(p1, gb.Q3_K) - gb.dequantize(p, gb.Q3_K))[0].reshape(8, 2, 16)
    assert np.array_equal(got, step)
    pn = p.copy()
    pn[0, 109] ^= 0x80
    assert np.array_equal(gb.dequantize(pn, gb.Q3_K), -gb.dequantize(p, gb.Q3_K))
    # negating an IQ2_XXS block scale negates every weight; Q8_0 is linear in d
    p = gb.random_payload(rng, gb.IQ2_XXS, 1, 256)
    q = p.copy()
    q[0, 1] ^= 0x80
    assert np.array_equal(gb.dequantize(q, gb.IQ2_XXS), -gb.dequantize(p, gb.IQ2_XXS))
    # each IQ2_XXS run of eight has an even number of minus signs relative to |w|
    w = gb.dequantize(p, gb.IQ2_XXS)[0].reshape(32, 8)
    assert np.all((w < 0).sum(axis=1) % 2 == 0)


def test_bf16_rounding_is_nearest_even():
    x = np.array([1.0, 1.00390625, 1.005859375, 1.01171875, -1.00390625, 3.0e38], dtype=np.float32)
    # 1 + 2^-8 is a tie -> even (1.0); 1 + 1.5*2^-8 rounds up; 1 + 3*2^-8 is a tie -> even (1.015625)
    want = np.array([0x3F80, 0x3F80, 0x3F81, 0x3F82, 0xBF80, 0x7F62], dtype=np.uint16)
    assert np.array_equal(gb.to_bf16_bits(x), want)


@pytest.mark.parametrize("qt,bound", [(gb.Q8_0, 0.01), (gb.Q2_K, 0.35), (gb.Q3_K, 0.25), (gb.Q4_K, 0.12), (gb.Q5_K, 0.06), (gb.Q6_K, 0.03),
                                      (gb.IQ2_XXS, 0.6)])
def test_quantizer_round_trip_error(qt, bound):
    rng = np.random.default_rng(11)
    w = (rng.standard_normal((16, 1024)) * 0.02).astype(np.float32)
    p = gb.quantize(w, qt)
    assert p.shape == (16, gb.row_bytes(qt, 1024))
    err = np.sqrt(((gb.dequantize(p, qt) - w) ** 2).mean()) / 0.02
    assert err < bound
