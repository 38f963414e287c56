// In-register GGUF block decoders used by the matmul kernels.
//
// Unit of work: one 32-element run (k = 32*ksub .. 32*ksub+31) of one weight row; every format has a
// natural 32-element grain (a Q8_0 block, a Q4_K sub-block, a quarter of a Q6_K half, an IQ2_XXS
// group).  load() pulls the run's packed bytes from global memory into registers (it can be issued a
// whole K-step ahead), decode() unpacks scales / mins / codebook entries in registers and returns the
// 32 weights as 16 packed bf16 pairs (element e in bits 16*(e&1) of out[e>>1]).
//
// Every product below is exact in fp32 (half-precision scale x small integers), Q4_K adds one
// fp32 rounding at the subtraction; the bf16 value is round-to-nearest-even of that fp32 value, which
// is what ggml's dequantize_row_* followed by a float->bf16 cast produces.
#pragma once
#include "common.h"

namespace ggq {

template <int QT>
struct Fmt;

// pin(): a compiler-level fence on the registers of a Raw: every later use stays behind this point in
// program order (nothing is emitted).  The matmul kernel puts it behind a barrier so that the wait for
// a prefetched run is not pulled in front of that barrier.
#if defined(__HIP_DEVICE_COMPILE__)
#define GGQ_PIN1(a) asm volatile("" : "+v"(a))
#else
#define GGQ_PIN1(a) (void)(a)
#endif
#define GGQ_PIN4(q) GGQ_PIN1((q).x); GGQ_PIN1((q).y); GGQ_PIN1((q).z); GGQ_PIN1((q).w)

// ------------------------------------------------------------------------------------------------
// Q8_0: 34-byte block = f16 d; i8 q[32]; one block per run.  Blocks are 2-byte aligned.
template <>
struct Fmt<kQ8_0> {
    static constexpr int kBlockElems = 32, kBlockBytes = 34;
    struct Raw {
        uint4 q0, q1;
        uint32_t d16;
    };
    static GGQ_HD void pin(Raw& r) { GGQ_PIN4(r.q0); GGQ_PIN4(r.q1); GGQ_PIN1(r.d16); }
    static GGQ_HD void load(Raw& r, const uint8_t* row, int ksub) {
        const uint8_t* p = row + (int64_t)ksub * 34;
        r.d16 = ld_u16(p);
        r.q0 = ld_u128(p + 2);
        r.q1 = ld_u128(p + 18);
    }
    // q (signed byte) = (q ^ 0x80) - 128 as unsigned byte u: d*q = fma(d, u, -128 d), exact.
    static GGQ_HD void four(uint32_t q, float d, float c, uint32_t* out) {
        uint32_t u = opaque(q ^ 0x80808080u);
        out[0] = pack_bf16(fmaf(d, ubyte0(u), c), fmaf(d, ubyte1(u), c));
        out[1] = pack_bf16(fmaf(d, ubyte2(u), c), fmaf(d, ubyte3(u), c));
    }
    static GGQ_HD void decode(const Raw& r, int, uint32_t* out, const uint2*) {
        const float d = half_bits_to_f32(r.d16), c = -128.0f * d;
        const uint32_t q[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
        for (int i = 0; i < 8; i++) four(q[i], d, c, out + 2 * i);
    }
};

// ------------------------------------------------------------------------------------------------
// Q4_K: 144-byte block = f16 d; f16 dmin; u8 scales[12]; u8 qs[128].  Sub-block j (run ksub & 7) uses
// qs[32*(j/2) .. +31]: low nibbles for even j, high nibbles for odd j, with its own 6-bit (sc, m).
template <>
struct Fmt<kQ4_K> {
    static constexpr int kBlockElems = 256, kBlockBytes = 144;
    struct Raw {
        uint4 hdr, q0, q1;
    };
    static GGQ_HD void pin(Raw& r) { GGQ_PIN4(r.hdr); GGQ_PIN4(r.q0); GGQ_PIN4(r.q1); }
    static GGQ_HD void load(Raw& r, const uint8_t* row, int ksub) {
        const uint8_t* blk = row + (int64_t)(ksub >> 3) * 144;
        r.hdr = *(const uint4*)blk;
        const uint8_t* q = blk + 16 + 32 * ((ksub & 7) >> 1);
        r.q0 = *(const uint4*)q;
        r.q1 = *(const uint4*)(q + 16);
    }
    static GGQ_HD void decode(const Raw& r, int ksub, uint32_t* out, const uint2*) {
        const int j = ksub & 7;
        const float d = half_bits_to_f32(r.hdr.x & 0xFFFFu);
        const float dmin = half_bits_to_f32(r.hdr.x >> 16);
        const uint32_t s0 = r.hdr.y, s1 = r.hdr.z, s2 = r.hdr.w;
        uint32_t sc, m;
        if (j < 4) {  // plain 6-bit fields
            const int sh = 8 * j;
            sc = (s0 >> sh) & 63u;
            m = (s1 >> sh) & 63u;
        } else {  // low 4 bits in scales[8..11], high 2 bits in the tops of scales[0..7]
            const int sh = 8 * (j - 4);
            sc = ((s2 >> sh) & 0xFu) | (((s0 >> (sh + 6)) & 3u) << 4);
            m = ((s2 >> (sh + 4)) & 0xFu) | (((s1 >> (sh + 6)) & 3u) << 4);
        }
        const float dl = d * (float)sc * kMixScale, nm = -(dmin * (float)m);
        const int shift = 4 * (j & 1);
        const uint32_t q[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            // nibbles of bytes 0, 2 and of bytes 1, 3, each in its own 16-bit half
            const uint32_t e02 = (q[i] >> shift) & 0x000F000Fu, e13 = (q[i] >> (shift + 8)) & 0x000F000Fu;
            out[2 * i] = pack_bf16(mix_lo(e02, dl, nm), mix_lo(e13, dl, nm));
            out[2 * i + 1] = pack_bf16(mix_hi(e02, dl, nm), mix_hi(e13, dl, nm));
        }
    }
};

// ------------------------------------------------------------------------------------------------
// Q5_K: 176-byte block = f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]: Q4_K with a fifth bit per
// element.  Sub-block j (run ksub & 7) uses qs[32*(j/2) .. +31] (low nibbles for even j, high for odd j) and bit j
// of qh[l] for its element l, with Q4_K's 6-bit (sc, m).
template <>
struct Fmt<kQ5_K> {
    static constexpr int kBlockElems = 256, kBlockBytes = 176;
    struct Raw {
        uint4 hdr, h0, h1, q0, q1;
    };
    static GGQ_HD void pin(Raw& r) { GGQ_PIN4(r.hdr); GGQ_PIN4(r.h0); GGQ_PIN4(r.h1); GGQ_PIN4(r.q0); GGQ_PIN4(r.q1); }
    static GGQ_HD void load(Raw& r, const uint8_t* row, int ksub) {
        const uint8_t* blk = row + (int64_t)(ksub >> 3) * 176;
        r.hdr = *(const uint4*)blk;
        r.h0 = *(const uint4*)(blk + 16);
        r.h1 = *(const uint4*)(blk + 32);
        const uint8_t* q = blk + 48 + 32 * ((ksub & 7) >> 1);
        r.q0 = *(const uint4*)q;
        r.q1 = *(const uint4*)(q + 16);
    }
    static GGQ_HD void decode(const Raw& r, int ksub, uint32_t* out, const uint2*) {
        const int j = ksub & 7;
        const float d = half_bits_to_f32(r.hdr.x & 0xFFFFu);
        const float dmin = half_bits_to_f32(r.hdr.x >> 16);
        const uint32_t s0 = r.hdr.y, s1 = r.hdr.z, s2 = r.hdr.w;
        uint32_t sc, m;
        if (j < 4) {
            const int sh = 8 * j;
            sc = (s0 >> sh) & 63u;
            m = (s1 >> sh) & 63u;
        } else {
            const int sh = 8 * (j - 4);
            sc = ((s2 >> sh) & 0xFu) | (((s0 >> (sh + 6)) & 3u) << 4);
            m = ((s2 >> (sh + 4)) & 0xFu) | (((s1 >> (sh + 6)) & 3u) << 4);
        }
        const float dl = d * (float)sc * kMixScale, nm = -(dmin * (float)m);
        const int shift = 4 * (j & 1);
        const uint32_t q[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
        const uint32_t h[8] = {r.h0.x, r.h0.y, r.h0.z, r.h0.w, r.h1.x, r.h1.y, r.h1.z, r.h1.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            // five-bit values of bytes 0, 2 and of bytes 1, 3, each in its own 16-bit half (a half-precision denormal)
            const uint32_t hb = (h[i] >> j) & 0x01010101u;  // the element's fifth bit, one per byte
            const uint32_t v = ((q[i] >> shift) & 0x0F0F0F0Fu) | (hb << 4);
            const uint32_t e02 = v & 0x001F001Fu, e13 = (v >> 8) & 0x001F001Fu;
            out[2 * i] = pack_bf16(mix_lo(e02, dl, nm), mix_lo(e13, dl, nm));
            out[2 * i + 1] = pack_bf16(mix_hi(e02, dl, nm), mix_hi(e13, dl, nm));
        }
    }
};

// ------------------------------------------------------------------------------------------------
// Q2_K: 84-byte block = u8 scales[16]; u8 qs[64]; f16 d; f16 dmin (4-byte aligned).  Run u = ksub & 7 lives in
// half n = u / 4 with bit pair s = u % 4 of qs[32 n .. +31]; its elements 0..15 use scales[8 n + 2 s], elements
// 16..31 scales[8 n + 2 s + 1] (low nibble: scale, high nibble: min).
template <>
struct Fmt<kQ2_K> {
    static constexpr int kBlockElems = 256, kBlockBytes = 84;
    struct Raw {
        uint4 q0, q1;
        uint32_t sc2, dd;
    };
    static GGQ_HD void pin(Raw& r) { GGQ_PIN4(r.q0); GGQ_PIN4(r.q1); GGQ_PIN1(r.sc2); GGQ_PIN1(r.dd); }
    static GGQ_HD void load(Raw& r, const uint8_t* row, int ksub) {
        const uint8_t* blk = row + (int64_t)(ksub >> 3) * 84;
        const int u = ksub & 7, n = u >> 2, s = u & 3;
        r.q0 = ld_u128(blk + 16 + 32 * n);
        r.q1 = ld_u128(blk + 32 + 32 * n);
        r.sc2 = ld_u16(blk + 8 * n + 2 * s);
        r.dd = ld_u32(blk + 80);
    }
    static GGQ_HD void decode(const Raw& r, int ksub, uint32_t* out, const uint2*) {
        const int shift = 2 * (ksub & 3);
        const float d = half_bits_to_f32(r.dd & 0xFFFFu), dmin = half_bits_to_f32(r.dd >> 16);
        const uint32_t q[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const uint32_t sb = (r.sc2 >> (8 * half)) & 0xFFu;
            const float dl = d * (float)(sb & 0xFu) * kMixScale, nm = -(dmin * (float)(sb >> 4));
#pragma unroll
            for (int i = 4 * half; i < 4 * half + 4; i++) {
                const uint32_t e02 = (q[i] >> shift) & 0x00030003u, e13 = (q[i] >> (shift + 8)) & 0x00030003u;
                out[2 * i] = pack_bf16(mix_lo(e02, dl, nm), mix_lo(e13, dl, nm));
                out[2 * i + 1] = pack_bf16(mix_hi(e02, dl, nm), mix_hi(e13, dl, nm));
            }
        }
    }
};

// ------------------------------------------------------------------------------------------------
// Q3_K: 110-byte block = u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d (2-byte aligned).  Run u = ksub & 7 takes
// bit pair u % 4 of qs[32 (u / 4) .. +31] and bit u of hmask[l] for its element l: value (pair | bit << 2) - 4 in
// [-4, 3].  Sixteen 6-bit scales (stored + 32): scale k has its low four bits in the nibble k / 8 of byte
// (k / 4 % 2) * 4 + k % 4 and its high two bits at position 2 (k / 4) of byte 8 + k % 4; elements 0..15 of the run use
// scale 2 u, elements 16..31 scale 2 u + 1.
template <>
struct Fmt<kQ3_K> {
    static constexpr int kBlockElems = 256, kBlockBytes = 110;
    struct Raw {
        uint4 h0, h1, q0, q1;
        uint32_t sl, sh, d16;
    };
    static GGQ_HD void pin(Raw& r) { GGQ_PIN4(r.h0); GGQ_PIN4(r.h1); GGQ_PIN4(r.q0); GGQ_PIN4(r.q1); GGQ_PIN1(r.sl); GGQ_PIN1(r.sh); GGQ_PIN1(r.d16); }
    static GGQ_HD void load(Raw& r, const uint8_t* row, int ksub) {
        const uint8_t* blk = row + (int64_t)(ksub >> 3) * 110;
        const int u = ksub & 7, n = u >> 2, g = u >> 1, b = 2 * (u & 1);
        r.h0 = ld_u128(blk), r.h1 = ld_u128(blk + 16);
        r.q0 = ld_u128(blk + 32 + 32 * n), r.q1 = ld_u128(blk + 48 + 32 * n);
        r.sl = ld_u16(blk + 96 + 4 * (g & 1) + b);
        r.sh = ld_u16(blk + 104 + b);
        r.d16 = ld_u16(blk + 108);
    }
    static GGQ_HD void decode(const Raw& r, int ksub, uint32_t* out, const uint2*) {
        const int u = ksub & 7, g = u >> 1, shift = 2 * (u & 3);
        const float d = half_bits_to_f32(r.d16);
        const uint32_t q[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
        const uint32_t h[8] = {r.h0.x, r.h0.y, r.h0.z, r.h0.w, r.h1.x, r.h1.y, r.h1.z, r.h1.w};
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const uint32_t lo = (r.sl >> (8 * half)) & 0xFFu, hi = (r.sh >> (8 * half)) & 0xFFu;
            const int sc = (int)(((lo >> (4 * (g >> 1))) & 0xFu) | (((hi >> (2 * g)) & 3u) << 4)) - 32;
            const float ds = d * (float)sc;
            const float dl = ds * kMixScale, nm = -4.0f * ds;
#pragma unroll
            for (int i = 4 * half; i < 4 * half + 4; i++) {
                const uint32_t v = ((q[i] >> shift) & 0x03030303u) | (((h[i] >> u) & 0x01010101u) << 2);
                const uint32_t e02 = v & 0x00070007u, e13 = (v >> 8) & 0x00070007u;
                out[2 * i] = pack_bf16(mix_lo(e02, dl, nm), mix_lo(e13, dl, nm));
                out[2 * i + 1] = pack_bf16(mix_hi(e02, dl, nm), mix_hi(e13, dl, nm));
            }
        }
    }
};

// ------------------------------------------------------------------------------------------------
// Q6_K: 210-byte block = u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d.  Blocks are only 2-byte
// aligned.  Run u = ksub & 7 lives in half h = u/4 as part p = u%4: low (p < 2) or high nibbles of
// ql[64h + 32(p&1) .. +31], bit pair 2p of qh[32h .. +31], int8 scales[8h + 2p], [8h + 2p + 1].
template <>
struct Fmt<kQ6_K> {
    static constexpr int kBlockElems = 256, kBlockBytes = 210;
    struct Raw {
        uint4 ql[2];
        uint4 qh[2];
        uint32_t sc2, d16;
    };
    static GGQ_HD void pin(Raw& r) { GGQ_PIN4(r.ql[0]); GGQ_PIN4(r.ql[1]); GGQ_PIN4(r.qh[0]); GGQ_PIN4(r.qh[1]); GGQ_PIN1(r.sc2); GGQ_PIN1(r.d16); }
    static GGQ_HD void load(Raw& r, const uint8_t* row, int ksub) {
        const uint8_t* blk = row + (int64_t)(ksub >> 3) * 210;
        const int u = ksub & 7, h = u >> 2, p = u & 3;
        const uint8_t* ql = blk + 64 * h + 32 * (p & 1);
        r.ql[0] = ld_u128(ql), r.ql[1] = ld_u128(ql + 16);
        const uint8_t* qh = blk + 128 + 32 * h;
        r.qh[0] = ld_u128(qh), r.qh[1] = ld_u128(qh + 16);
        r.sc2 = ld_u16(blk + 192 + 8 * h + 2 * p);
        r.d16 = ld_u16(blk + 208);
    }
    static GGQ_HD void decode(const Raw& r, int ksub, uint32_t* out, const uint2*) {
        const int p = ksub & 3;
        const float d = half_bits_to_f32(r.d16);
        const float dl0 = d * (float)(int)(int8_t)(r.sc2 & 0xFFu), dl1 = d * (float)(int)(int8_t)(r.sc2 >> 8);
        const float c0 = -32.0f * dl0, c1 = -32.0f * dl1;
        const int nshift = 4 * (p >> 1), hshift = 2 * p;
        const uint32_t qlw[8] = {r.ql[0].x, r.ql[0].y, r.ql[0].z, r.ql[0].w, r.ql[1].x, r.ql[1].y, r.ql[1].z, r.ql[1].w};
        const uint32_t qhw[8] = {r.qh[0].x, r.qh[0].y, r.qh[0].z, r.qh[0].w, r.qh[1].x, r.qh[1].y, r.qh[1].z, r.qh[1].w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t nib = (qlw[i] >> nshift) & 0x0F0F0F0Fu;
            const uint32_t two = (qhw[i] >> hshift) & 0x03030303u;
            const uint32_t q = opaque(nib | (two << 4));  // four 6-bit values, each (weight level + 32)
            const float s = i < 4 ? dl0 : dl1, cc = i < 4 ? c0 : c1;
            out[2 * i] = pack_bf16(fmaf(s, ubyte0(q), cc), fmaf(s, ubyte1(q), cc));
            out[2 * i + 1] = pack_bf16(fmaf(s, ubyte2(q), cc), fmaf(s, ubyte3(q), cc));
        }
    }
};

// ------------------------------------------------------------------------------------------------
// IQ2_XXS: 66-byte block = f16 d; u16 qs[32].  Each 32-element group (one run) is 8 bytes: four codebook
// indices, then a u32 with four 7-bit sign indices and a 4-bit scale in bits 28..31.  The eighth sign
// of each 8-element stretch is the parity of the other seven.
template <>
struct Fmt<kIQ2_XXS> {
    static constexpr int kBlockElems = 256, kBlockBytes = 66;
    struct Raw {
        uint32_t idx4, aux, d16;
    };
    static GGQ_HD void pin(Raw& r) { GGQ_PIN1(r.idx4); GGQ_PIN1(r.aux); GGQ_PIN1(r.d16); }
    static GGQ_HD void load(Raw& r, const uint8_t* row, int ksub) {
        const uint8_t* blk = row + (int64_t)(ksub >> 3) * 66;
        r.d16 = ld_u16(blk);
        const uint8_t* g = blk + 2 + 8 * (ksub & 7);
        r.idx4 = ld_u32(g);
        r.aux = ld_u32(g + 4);
    }
    // Tables the tile kernel stages in LDS once per workgroup (built by table_entry below): for every codebook entry the
    // four byte selectors that pick its eight magnitudes, two per word, out of a 3-entry bf16 table, and for every 7-bit
    // sign index the four words that flip the signs of the eight values (bit 15 / bit 31 of a pair; the eighth sign is
    // the parity of the other seven).  A run then costs one selection and one exclusive-or per pair of weights.
    static constexpr int kTableWords = 256 * 4 + 128 * 4;  // uint32 words: selectors [256][4], then sign masks [128][4]
    // Word `i` of the tables (i < kTableWords); `grid_entry` is the codebook entry i / 4 for i < 1024.
    static GGQ_HD uint32_t table_word(int i, uint64_t grid_entry) {
        if (i < 1024) {
            const int p = i & 3;  // pair of the entry: magnitudes 2p, 2p + 1; codebook bytes are 0x08, 0x19, 0x2b: index = byte >> 4
            const uint32_t t0 = (uint32_t)(grid_entry >> (16 * p + 4)) & 3u, t1 = (uint32_t)(grid_entry >> (16 * p + 12)) & 3u;
            return (2 * t0) | ((2 * t0 + 1) << 8) | ((2 * t1) << 16) | ((2 * t1 + 1) << 24);
        }
        const uint32_t s7 = (uint32_t)(i - 1024) >> 2, p = (uint32_t)i & 3u;
        const uint32_t signs = s7 | ((__builtin_popcount(s7) & 1u) << 7);
        return (((signs >> (2 * p)) & 1u) << 15) | (((signs >> (2 * p + 1)) & 1u) << 31);
    }
    static __device__ __forceinline__ void decode(const Raw& r, int, uint32_t* out, const uint2* tables) {
        const uint4* sel = (const uint4*)tables;
        const uint4* flip = sel + 256;
        const float d = half_bits_to_f32(r.d16);
        const float db = d * (0.5f + (float)(r.aux >> 28)) * 0.25f;
        // the three products a weight can be, as bf16: bytes 0..5 of {hi : lo}
        const uint32_t lo = pack_bf16(db * 8.0f, db * 25.0f), hi = pack_bf16(db * 43.0f, 0.0f);
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint4 e = sel[(r.idx4 >> (8 * l)) & 0xFFu];
            const uint4 f = flip[(r.aux >> (7 * l)) & 127u];
            out[4 * l + 0] = __builtin_amdgcn_perm(hi, lo, e.x) ^ f.x;
            out[4 * l + 1] = __builtin_amdgcn_perm(hi, lo, e.y) ^ f.y;
            out[4 * l + 2] = __builtin_amdgcn_perm(hi, lo, e.z) ^ f.z;
            out[4 * l + 3] = __builtin_amdgcn_perm(hi, lo, e.w) ^ f.w;
        }
    }
};

}  // namespace ggq
