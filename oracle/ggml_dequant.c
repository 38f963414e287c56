/* CPU oracle, C restatement of the GGUF block decoders on the quantized-weight matmul path.
 *
 * TEST INFRASTRUCTURE: only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * load this library.  It is the checker, never the product.
 *
 * The reference reaches these decoders through un-vendored dependencies
 * (dequantize_gguf_tensor: fast_moe_lora.py:163-165, test_fast_lora.py:110-115; packed payloads
 * handed to torch_ggml_ops: fast_lora.py:154-160).  The loops below restate the published ggml
 * algorithm (ggml-quants.c dequantize_row_q8_0 / _q2_K / _q4_K / _q5_K / _q6_K / _iq2_xxs) one scalar at a time,
 * independently of the vectorised numpy restatement in gguf_blocks.py; the two are checked against
 * each other and against hand-computed blocks in tests/test_oracle_blocks.py.
 * parity unpinned: no upstream decoder output exists in the build environment; the IQ2_XXS codebook
 * is passed in by the caller (oracle/iq2xxs_grid.py).
 *
 * Build: make -C oracle   (gcc -O2 -shared -fPIC; -ffp-contract=off keeps mul and sub separate).
 */
#include <stdint.h>
#include <string.h>

static float half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal half: renormalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static uint32_t rd32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

/* y[32*nb] from nb blocks of {f16 d; i8 qs[32]} */
void oracle_dequant_q8_0(const uint8_t *x, int64_t nb, float *y) {
    for (int64_t i = 0; i < nb; i++, x += 34, y += 32) {
        float d = half_to_float(rd16(x));
        for (int j = 0; j < 32; j++) y[j] = d * (float)(int8_t)x[2 + j];
    }
}

static void scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* y[256*nb] from nb blocks of {f16 d; f16 dmin; u8 scales[12]; u8 qs[128]} */
void oracle_dequant_q4_k(const uint8_t *x, int64_t nb, float *y) {
    for (int64_t i = 0; i < nb; i++, x += 144) {
        float d = half_to_float(rd16(x));
        float dmin = half_to_float(rd16(x + 2));
        const uint8_t *scales = x + 4;
        const uint8_t *q = x + 16;
        int is = 0;
        for (int j = 0; j < 256; j += 64) {
            uint8_t sc, m;
            scale_min_k4(is + 0, scales, &sc, &m);
            float d1 = d * sc, m1 = dmin * m;
            scale_min_k4(is + 1, scales, &sc, &m);
            float d2 = d * sc, m2 = dmin * m;
            for (int l = 0; l < 32; l++) *y++ = d1 * (float)(q[l] & 0x0F) - m1;
            for (int l = 0; l < 32; l++) *y++ = d2 * (float)(q[l] >> 4) - m2;
            q += 32;
            is += 2;
        }
    }
}

/* y[256*nb] from nb blocks of {f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]} (dequantize_row_q5_K) */
void oracle_dequant_q5_k(const uint8_t *x, int64_t nb, float *y) {
    for (int64_t i = 0; i < nb; i++, x += 176) {
        float d = half_to_float(rd16(x));
        float dmin = half_to_float(rd16(x + 2));
        const uint8_t *scales = x + 4;
        const uint8_t *qh = x + 16;
        const uint8_t *ql = x + 48;
        int is = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int j = 0; j < 256; j += 64) {
            uint8_t sc, m;
            scale_min_k4(is + 0, scales, &sc, &m);
            float d1 = d * sc, m1 = dmin * m;
            scale_min_k4(is + 1, scales, &sc, &m);
            float d2 = d * sc, m2 = dmin * m;
            for (int l = 0; l < 32; l++) *y++ = d1 * (float)((ql[l] & 0x0F) + ((qh[l] & u1) ? 16 : 0)) - m1;
            for (int l = 0; l < 32; l++) *y++ = d2 * (float)((ql[l] >> 4) + ((qh[l] & u2) ? 16 : 0)) - m2;
            ql += 32;
            is += 2;
            u1 <<= 2;
            u2 <<= 2;
        }
    }
}

/* y[256*nb] from nb blocks of {u8 scales[16]; u8 qs[64]; f16 d; f16 dmin} (dequantize_row_q2_K) */
void oracle_dequant_q2_k(const uint8_t *x, int64_t nb, float *y) {
    for (int64_t i = 0; i < nb; i++, x += 84) {
        const uint8_t *scales = x;
        const uint8_t *q = x + 16;
        float d = half_to_float(rd16(x + 80));
        float dmin = half_to_float(rd16(x + 82));
        int is = 0;
        for (int n = 0; n < 256; n += 128) {
            int shift = 0;
            for (int j = 0; j < 4; j++) {
                uint8_t sc = scales[is++];
                float dl = d * (sc & 0xF), ml = dmin * (sc >> 4);
                for (int l = 0; l < 16; l++) *y++ = dl * (float)((q[l] >> shift) & 3) - ml;
                sc = scales[is++];
                dl = d * (sc & 0xF), ml = dmin * (sc >> 4);
                for (int l = 0; l < 16; l++) *y++ = dl * (float)((q[l + 16] >> shift) & 3) - ml;
                shift += 2;
            }
            q += 32;
        }
    }
}

/* y[256*nb] from nb blocks of {u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d} (dequantize_row_q3_K): the twelve
 * scale bytes unpack to sixteen 6-bit values through the word-wise mask shuffle of the format's reference code. */
void oracle_dequant_q3_k(const uint8_t *x, int64_t nb, float *y) {
    const uint32_t kmask1 = 0x03030303u, kmask2 = 0x0f0f0f0fu;
    for (int64_t i = 0; i < nb; i++, x += 110) {
        const uint8_t *hm = x;
        const uint8_t *q = x + 32;
        float d_all = half_to_float(rd16(x + 108));
        uint32_t aux[4];
        for (int w = 0; w < 3; w++)
            aux[w] = (uint32_t)x[96 + 4 * w] | ((uint32_t)x[97 + 4 * w] << 8) | ((uint32_t)x[98 + 4 * w] << 16) | ((uint32_t)x[99 + 4 * w] << 24);
        uint32_t tmp = aux[2];
        aux[2] = ((aux[0] >> 4) & kmask2) | (((tmp >> 4) & kmask1) << 4);
        aux[3] = ((aux[1] >> 4) & kmask2) | (((tmp >> 6) & kmask1) << 4);
        aux[0] = (aux[0] & kmask2) | (((tmp >> 0) & kmask1) << 4);
        aux[1] = (aux[1] & kmask2) | (((tmp >> 2) & kmask1) << 4);
        int8_t scales[16];
        for (int k = 0; k < 16; k++) scales[k] = (int8_t)((aux[k / 4] >> (8 * (k % 4))) & 0xFF);
        int is = 0;
        uint8_t m = 1;
        for (int n = 0; n < 256; n += 128) {
            int shift = 0;
            for (int j = 0; j < 4; j++) {
                float dl = d_all * (float)(scales[is++] - 32);
                for (int l = 0; l < 16; l++) *y++ = dl * (float)((int)((q[l] >> shift) & 3) - ((hm[l] & m) ? 0 : 4));
                dl = d_all * (float)(scales[is++] - 32);
                for (int l = 0; l < 16; l++) *y++ = dl * (float)((int)((q[l + 16] >> shift) & 3) - ((hm[l + 16] & m) ? 0 : 4));
                shift += 2;
                m <<= 1;
            }
            q += 32;
        }
    }
}

/* y[256*nb] from nb blocks of {u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d} */
void oracle_dequant_q6_k(const uint8_t *x, int64_t nb, float *y) {
    for (int64_t i = 0; i < nb; i++, x += 210) {
        const uint8_t *ql = x;
        const uint8_t *qh = x + 128;
        const int8_t *sc = (const int8_t *)(x + 192);
        float d = half_to_float(rd16(x + 208));
        for (int n = 0; n < 256; n += 128) {
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int q1 = (int)((ql[l + 0] & 0x0F) | (((qh[l] >> 0) & 3) << 4)) - 32;
                int q2 = (int)((ql[l + 32] & 0x0F) | (((qh[l] >> 2) & 3) << 4)) - 32;
                int q3 = (int)((ql[l + 0] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                y[l + 0] = d * sc[is + 0] * q1;
                y[l + 32] = d * sc[is + 2] * q2;
                y[l + 64] = d * sc[is + 4] * q3;
                y[l + 96] = d * sc[is + 6] * q4;
            }
            y += 128;
            ql += 64;
            qh += 32;
            sc += 8;
        }
    }
}

/* y[256*nb] from nb blocks of {f16 d; u16 qs[32]}; grid = 256 codebook entries of 8 bytes */
void oracle_dequant_iq2_xxs(const uint8_t *x, int64_t nb, const uint64_t *grid, float *y) {
    for (int64_t i = 0; i < nb; i++, x += 66) {
        float d = half_to_float(rd16(x));
        const uint8_t *qs = x + 2;
        for (int ib32 = 0; ib32 < 8; ib32++) {
            const uint8_t *aux8 = qs + 8 * ib32;
            uint32_t aux1 = rd32(aux8 + 4);
            float db = d * (0.5f + (float)(aux1 >> 28)) * 0.25f;
            for (int l = 0; l < 4; l++) {
                uint64_t g = grid[aux8[l]];
                uint32_t s7 = (aux1 >> (7 * l)) & 127;
                uint32_t signs = s7 | ((uint32_t)(__builtin_popcount(s7) & 1) << 7);
                for (int j = 0; j < 8; j++) {
                    float mag = (float)((g >> (8 * j)) & 0xFF);
                    y[j] = db * mag * ((signs >> j) & 1 ? -1.0f : 1.0f);
                }
                y += 8;
            }
        }
    }
}

/* float32 -> bf16 bits, round to nearest even (finite inputs) */
void oracle_f32_to_bf16(const float *x, int64_t n, uint16_t *out) {
    for (int64_t i = 0; i < n; i++) {
        uint32_t u;
        memcpy(&u, x + i, 4);
        u += 0x7FFFu + ((u >> 16) & 1u);
        out[i] = (uint16_t)(u >> 16);
    }
}
