// In-register GGUF block decoders used by the matmul kernels.
//
// Unit of work: one 64-element segment (k = 64*kseg .. 64*kseg+63) of one weight row.  load() pulls the
// segment's packed bytes from global memory into registers (it can be issued a whole K-step ahead),
// decode() unpacks scales / mins / codebook entries in registers and returns the 64 weights as 32
// packed bf16 pairs (element e in bits 16*(e&1) of out[e>>1]).
//
// Every product below is exact in fp32 (half-precision scale x small integers), Q4_K adds one
// fp32 rounding at the subtraction; the bf16 value is round-to-nearest-even of that fp32 value, which
// is what ggml's dequantize_row_* followed by a float->bf16 cast produces.
#pragma once
#include "common.h"

namespace ggq {

template <int QT>
struct Fmt;

// ------------------------------------------------------------------------------------------------
// Q8_0: 34-byte block = f16 d; i8 q[32].  A 64-element segment is two blocks = 68 bytes (4-aligned).
template <>
struct Fmt<kQ8_0> {
    static constexpr int kBlockElems = 32, kBlockBytes = 34;
    struct Raw {
        uint32_t w[17];
    };
    static GGQ_HD int64_t row_bytes(int k) { return (int64_t)(k / 32) * 34; }
    static GGQ_HD void load(Raw& r, const uint8_t* row, int kseg) {
        const uint8_t* p = row + (int64_t)kseg * 68;
        uint4 a = ld_u128(p), b = ld_u128(p + 16), c = ld_u128(p + 32), d = ld_u128(p + 48);
        r.w[0] = a.x, r.w[1] = a.y, r.w[2] = a.z, r.w[3] = a.w;
        r.w[4] = b.x, r.w[5] = b.y, r.w[6] = b.z, r.w[7] = b.w;
        r.w[8] = c.x, r.w[9] = c.y, r.w[10] = c.z, r.w[11] = c.w;
        r.w[12] = d.x, r.w[13] = d.y, r.w[14] = d.z, r.w[15] = d.w;
        r.w[16] = ld_u32(p + 64);
    }
    // q (signed byte) = (q ^ 0x80) - 128 as unsigned byte u: d*q = fma(d, u, -128 d), exact.
    static GGQ_HD void four(uint32_t q, float d, float c, uint32_t* out) {
        uint32_t u = opaque(q ^ 0x80808080u);
        out[0] = pack_bf16(fmaf(d, ubyte0(u), c), fmaf(d, ubyte1(u), c));
        out[1] = pack_bf16(fmaf(d, ubyte2(u), c), fmaf(d, ubyte3(u), c));
    }
    static GGQ_HD void decode(const Raw& r, int, uint32_t* out, const uint2*) {
        float d0 = half_bits_to_f32(r.w[0] & 0xFFFFu);
        float d1 = half_bits_to_f32(r.w[8] >> 16);
        float c0 = -128.0f * d0, c1 = -128.0f * d1;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            uint32_t q = (r.w[j] >> 16) | (r.w[j + 1] << 16);  // block 0 quants start at byte 2
            four(q, d0, c0, out + 2 * j);
        }
#pragma unroll
        for (int j = 0; j < 8; j++) four(r.w[9 + j], d1, c1, out + 16 + 2 * j);
    }
};

// ------------------------------------------------------------------------------------------------
// Q4_K: 144-byte block = f16 d; f16 dmin; u8 scales[12]; u8 qs[128].  Segment c of a block is
// qs[32c..32c+31]: low nibbles are elements 64c..64c+31 (sub-block 2c), high nibbles the next 32.
template <>
struct Fmt<kQ4_K> {
    static constexpr int kBlockElems = 256, kBlockBytes = 144;
    struct Raw {
        uint4 hdr, q0, q1;
    };
    static GGQ_HD int64_t row_bytes(int k) { return (int64_t)(k / 256) * 144; }
    static GGQ_HD void load(Raw& r, const uint8_t* row, int kseg) {
        const uint8_t* blk = row + (int64_t)(kseg >> 2) * 144;
        r.hdr = *(const uint4*)blk;
        const uint8_t* q = blk + 16 + 32 * (kseg & 3);
        r.q0 = *(const uint4*)q;
        r.q1 = *(const uint4*)(q + 16);
    }
    static GGQ_HD void eight(uint32_t q, float dl1, float nm1, float dl2, float nm2,
                                                 uint32_t* lo_out, uint32_t* hi_out) {
        uint32_t lo = opaque(q & 0x0F0F0F0Fu);
        uint32_t hi = opaque((q >> 4) & 0x0F0F0F0Fu);
        lo_out[0] = pack_bf16(fmaf(dl1, ubyte0(lo), nm1), fmaf(dl1, ubyte1(lo), nm1));
        lo_out[1] = pack_bf16(fmaf(dl1, ubyte2(lo), nm1), fmaf(dl1, ubyte3(lo), nm1));
        hi_out[0] = pack_bf16(fmaf(dl2, ubyte0(hi), nm2), fmaf(dl2, ubyte1(hi), nm2));
        hi_out[1] = pack_bf16(fmaf(dl2, ubyte2(hi), nm2), fmaf(dl2, ubyte3(hi), nm2));
    }
    static GGQ_HD void decode(const Raw& r, int kseg, uint32_t* out, const uint2*) {
        const int c = kseg & 3;
        const float d = half_bits_to_f32(r.hdr.x & 0xFFFFu);
        const float dmin = half_bits_to_f32(r.hdr.x >> 16);
        const uint32_t s0 = r.hdr.y, s1 = r.hdr.z, s2 = r.hdr.w;
        uint32_t sc1, m1, sc2, m2;
        if (c < 2) {  // sub-blocks 0..3: plain 6-bit fields
            const int sh = 16 * c;
            sc1 = (s0 >> sh) & 63u;
            m1 = (s1 >> sh) & 63u;
            sc2 = (s0 >> (sh + 8)) & 63u;
            m2 = (s1 >> (sh + 8)) & 63u;
        } else {  // sub-blocks 4..7: low 4 bits in scales[8..11], high 2 bits in the tops of [0..7]
            const int sh = 16 * (c - 2);
            sc1 = ((s2 >> sh) & 0xFu) | (((s0 >> (sh + 6)) & 3u) << 4);
            m1 = ((s2 >> (sh + 4)) & 0xFu) | (((s1 >> (sh + 6)) & 3u) << 4);
            sc2 = ((s2 >> (sh + 8)) & 0xFu) | (((s0 >> (sh + 14)) & 3u) << 4);
            m2 = ((s2 >> (sh + 12)) & 0xFu) | (((s1 >> (sh + 14)) & 3u) << 4);
        }
        const float dl1 = d * (float)sc1, nm1 = -(dmin * (float)m1);
        const float dl2 = d * (float)sc2, nm2 = -(dmin * (float)m2);
        const uint32_t q[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
        for (int i = 0; i < 8; i++) eight(q[i], dl1, nm1, dl2, nm2, out + 2 * i, out + 16 + 2 * i);
    }
};

// ------------------------------------------------------------------------------------------------
// Q6_K: 210-byte block = u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d.  Blocks are only 2-byte
// aligned.  Segment s of a block lives in half h = s/2: its 64 elements use the low (s even) or high
// (s odd) nibbles of ql[64h..64h+63] and bit pairs 4*(s&1), 4*(s&1)+2 of qh[32h..32h+31].
template <>
struct Fmt<kQ6_K> {
    static constexpr int kBlockElems = 256, kBlockBytes = 210;
    struct Raw {
        uint4 ql[4];
        uint4 qh[2];
        uint32_t sc4, d16;
    };
    static GGQ_HD int64_t row_bytes(int k) { return (int64_t)(k / 256) * 210; }
    static GGQ_HD void load(Raw& r, const uint8_t* row, int kseg) {
        const uint8_t* blk = row + (int64_t)(kseg >> 2) * 210;
        const int s = kseg & 3, h = s >> 1;
        const uint8_t* ql = blk + 64 * h;
        r.ql[0] = ld_u128(ql), r.ql[1] = ld_u128(ql + 16), r.ql[2] = ld_u128(ql + 32), r.ql[3] = ld_u128(ql + 48);
        const uint8_t* qh = blk + 128 + 32 * h;
        r.qh[0] = ld_u128(qh), r.qh[1] = ld_u128(qh + 16);
        r.sc4 = ld_u32(blk + 192 + 8 * h + 4 * (s & 1));
        r.d16 = ld_u16(blk + 208);
    }
    static GGQ_HD void decode(const Raw& r, int kseg, uint32_t* out, const uint2*) {
        const int odd = kseg & 1;
        const float d = half_bits_to_f32(r.d16);
        float dl[4], c[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int sc = (int)(int8_t)((r.sc4 >> (8 * j)) & 0xFFu);
            dl[j] = d * (float)sc;
            c[j] = -32.0f * dl[j];
        }
        const uint32_t qlw[16] = {r.ql[0].x, r.ql[0].y, r.ql[0].z, r.ql[0].w, r.ql[1].x, r.ql[1].y,
                                  r.ql[1].z, r.ql[1].w, r.ql[2].x, r.ql[2].y, r.ql[2].z, r.ql[2].w,
                                  r.ql[3].x, r.ql[3].y, r.ql[3].z, r.ql[3].w};
        const uint32_t qhw[8] = {r.qh[0].x, r.qh[0].y, r.qh[0].z, r.qh[0].w,
                                 r.qh[1].x, r.qh[1].y, r.qh[1].z, r.qh[1].w};
        const int nib_shift = 4 * odd;
#pragma unroll
        for (int p = 0; p < 2; p++) {
            const int two_shift = 4 * odd + 2 * p;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                uint32_t nib = (qlw[8 * p + i] >> nib_shift) & 0x0F0F0F0Fu;
                uint32_t two = (qhw[i] >> two_shift) & 0x03030303u;
                uint32_t q = opaque(nib | (two << 4));  // four 6-bit values, each q+32 of the format
                const float s = dl[2 * p + (i >> 2)], cc = c[2 * p + (i >> 2)];
                out[16 * p + 2 * i] = pack_bf16(fmaf(s, ubyte0(q), cc), fmaf(s, ubyte1(q), cc));
                out[16 * p + 2 * i + 1] = pack_bf16(fmaf(s, ubyte2(q), cc), fmaf(s, ubyte3(q), cc));
            }
        }
    }
};

// ------------------------------------------------------------------------------------------------
// IQ2_XXS: 66-byte block = f16 d; u16 qs[32].  Each 32-element group is 8 bytes: four codebook
// indices, then a u32 with four 7-bit sign indices and a 4-bit scale in bits 28..31.  The eighth sign
// of each 8-element run is the parity of the other seven.  A segment is two groups (16 bytes).
template <>
struct Fmt<kIQ2_XXS> {
    static constexpr int kBlockElems = 256, kBlockBytes = 66;
    struct Raw {
        uint4 g;
        uint32_t d16;
    };
    static GGQ_HD int64_t row_bytes(int k) { return (int64_t)(k / 256) * 66; }
    static GGQ_HD void load(Raw& r, const uint8_t* row, int kseg) {
        const uint8_t* blk = row + (int64_t)(kseg >> 2) * 66;
        r.d16 = ld_u16(blk);
        r.g = ld_u128(blk + 2 + 16 * (kseg & 3));
    }
    static GGQ_HD uint32_t signed_pair(float db, float m0, float m1, uint32_t signs, int j) {
        float v0 = db * m0, v1 = db * m1;
        uint32_t b0 = __builtin_bit_cast(uint32_t, v0) ^ ((signs << (31 - j)) & 0x80000000u);
        uint32_t b1 = __builtin_bit_cast(uint32_t, v1) ^ ((signs << (30 - j)) & 0x80000000u);
        return pack_bf16(__builtin_bit_cast(float, b0), __builtin_bit_cast(float, b1));
    }
    static GGQ_HD void group(uint32_t idx4, uint32_t aux, float d, uint32_t* out,
                                                 const uint2* grid) {
        const float db = d * (0.5f + (float)(aux >> 28)) * 0.25f;
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint2 g = grid[(idx4 >> (8 * l)) & 0xFFu];
            const uint32_t s7 = (aux >> (7 * l)) & 127u;
            const uint32_t signs = s7 | ((__builtin_popcount(s7) & 1u) << 7);
            const uint32_t glo = opaque(g.x), ghi = opaque(g.y);
            out[4 * l + 0] = signed_pair(db, ubyte0(glo), ubyte1(glo), signs, 0);
            out[4 * l + 1] = signed_pair(db, ubyte2(glo), ubyte3(glo), signs, 2);
            out[4 * l + 2] = signed_pair(db, ubyte0(ghi), ubyte1(ghi), signs, 4);
            out[4 * l + 3] = signed_pair(db, ubyte2(ghi), ubyte3(ghi), signs, 6);
        }
    }
    static GGQ_HD void decode(const Raw& r, int, uint32_t* out, const uint2* grid) {
        const float d = half_bits_to_f32(r.d16);
        group(r.g.x, r.g.y, d, out, grid);
        group(r.g.z, r.g.w, d, out + 16, grid);
    }
};

}  // namespace ggq
