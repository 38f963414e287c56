// Pieces shared by the Q4_K kernels whose MFMA-issuing waves decode the packed weights themselves (mmq_direct8.h,
// mmq_direct8_nn.h): the scales of a quant group, the decode of a lane's 16 quant bytes into MFMA operands, the
// description of a row tile.
//
// Forward decode: a lane (column n = lane % 32 of a column block, half h = lane / 32) holds the 16 bytes 16h .. 16h+15 of
// its row's 32-byte quant group of the step.  The low nibbles are elements 16h .. 16h+15 of the group's first sub-block
// (MFMA sub-steps 0, 1), the high nibbles the same elements of the second (2, 3).  An MFMA sums over its 16 contraction
// slots in any order, so lane half h simply feeds contraction elements 16h .. 16h+7 (+8 for the odd sub-steps, +32 for
// the high nibbles) and reads the matching 16-byte slot of the A row.  No decoded weight ever touches LDS.
#pragma once
#include "mmq_tile.h"

namespace ggq {

struct Direct {
    struct Scales {  // sub-block scale * 2^24, -min; dl1 is divided by 16: high nibbles are read at bits 4..7 of a half
        float dl0, nm0, dl1, nm1;
    };
    template <int S>
    static __device__ __forceinline__ Scales chunk_scales(const u32x4_t& hdr) {
        const float d = half_bits_to_f32(hdr.x & 0xFFFFu), dmin = half_bits_to_f32(hdr.x >> 16);
        uint32_t sc0, m0, sc1, m1;
        Tile<kShapeWide>::template q4k_scale_min<2 * S>(hdr, sc0, m0);
        Tile<kShapeWide>::template q4k_scale_min<2 * S + 1>(hdr, sc1, m1);
        Scales s;
        s.dl0 = d * (float)sc0 * kMixScale, s.nm0 = -(dmin * (float)m0);
        s.dl1 = d * (float)sc1 * (kMixScale / 16.0f), s.nm1 = -(dmin * (float)m1);
        return s;
    }
    // Half J (0, 1) of the B operand of sub-step I (0..3), from the lane's 16 bytes of the step: I < 2: the low
    // nibbles of word 2I + J; I >= 2: the high nibbles of word 2(I-2) + J.  Writes out[2J], out[2J+1].
    template <int I, int J>
    static __device__ __forceinline__ void decode_half(const u32x4_t& q, const Scales& s, uint32_t* out) {
        const float dl = I < 2 ? s.dl0 : s.dl1, nm = I < 2 ? s.nm0 : s.nm1;
        const uint32_t w = q[2 * (I & 1) + J];
        constexpr uint32_t kMask = I < 2 ? 0x000F000Fu : 0x00F000F0u;  // a nibble in each 16-bit half: a half-precision denormal
        const uint32_t e02 = w & kMask, e13 = (w >> 8) & kMask;
        out[2 * J] = pack_bf16(mix_lo(e02, dl, nm), mix_lo(e13, dl, nm));
        out[2 * J + 1] = pack_bf16(mix_hi(e02, dl, nm), mix_hi(e13, dl, nm));
        // a use of the results right here: keeps the arithmetic where the caller placed it (between two MFMAs)
        // instead of being sunk to the MFMA that reads them
        asm volatile("" ::"v"(out[2 * J]), "v"(out[2 * J + 1]));
    }
    static __device__ __forceinline__ bf16x8_t as_operand(const uint32_t* r) {
        const u32x4_t v = {r[0], r[1], r[2], r[3]};
        return __builtin_bit_cast(bf16x8_t, v);
    }

    struct RowCtx {  // wave-uniform description of the row tile
        int row_begin, rows_valid;
        int64_t expert;
    };
};

}  // namespace ggq
