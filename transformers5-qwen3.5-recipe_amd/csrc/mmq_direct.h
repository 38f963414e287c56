// Q4_K forward ("NT") tile kernel in which the MFMA-issuing waves decode the packed weights themselves.
//
//   C[m, n] = sum_k A[m, k] * W[n, k]  (+ s * LA[m, :] . LB[n, :])
//
// One workgroup = 256 lanes = four waves, one per SIMD with the whole 512-register file of its lanes,
// computes tiles of up to 192 rows x 256 columns.  Wave w owns columns 64w .. 64w+63 of every row: up to
// six 32-row blocks x two 32-column blocks of MFMA 32x32x16 accumulators.  Per contraction step of 64
//   * the A tile goes global -> LDS directly (no registers), three steps ahead, through a ring of four
//     stages; rows are unpadded with XOR-swizzled 16-byte slots (a_slot), every wave reads all of them;
//   * a lane (column n = lane % 32 of a column block, half h = lane / 32) loads the 16 bytes 16h .. 16h+15
//     of its row's 32-byte quant group of the step, three steps ahead, and decodes them in registers into
//     the operands of the step's four MFMA sub-steps: the low nibbles are elements 16h .. 16h+15 of the
//     group's first sub-block (sub-steps 0, 1), the high nibbles the same elements of the second (2, 3).
//     An MFMA sums over its 16 contraction slots in any order, so lane half h simply feeds contraction
//     elements 16h .. 16h+7 (+8 for the odd sub-steps, +32 for the high nibbles) and reads the matching
//     16-byte slot of the A row.  No decoded weight ever touches LDS, and the tile's rows share one decode.
// The weights are the MFMA's first operand, so a lane's accumulator registers hold four consecutive columns
// of one row; a finished row block goes through a wave-private LDS block and leaves as whole 128-byte rows.
// The LoRA term is added there, from operands loaded straight from global memory (one burst per tile).
// A workgroup takes a run of column tiles of its row tile and treats their steps as one stream, so the loads
// of a tile's first steps are in flight while the tile before it finishes.
// The kernel is instantiated per number of live 32-row blocks, so an expert group of any size up to 192
// rows is one row tile and issues no MFMA on empty blocks.  The packed-weight loads are inline-asm loads
// the compiler does not track; the step waits for them with an exact count (vector memory operations complete
// in issue order).  With one wave per SIMD every instruction of the step, scalar ones included, takes an issue
// slot of that wave: the decode arithmetic is placed by hand between the MFMAs, and the addresses of the loads
// are scalar bases plus lane offsets that never change.
#pragma once
#include "mmq_tile.h"

namespace ggq {

struct Direct {
    static constexpr int kTM = kDirectBM, kTN = kDirectBN;
    static constexpr int kStages = 4;
    static constexpr int kThreadsWG = 256;
    static constexpr int kOutPitch = 144;                              // bytes per row of a wave's output staging block (32 rows x 64 columns)
    static constexpr int kRingBytes = kStages * kTM * kARowBytes;      // 96 KB
    static constexpr int kLaBase = kRingBytes + 4 * 32 * kOutPitch;    // + 18 KB: the row tile's LA rows (rank <= 16), 32 bytes each
    static constexpr int kLdsBytes = kLaBase + kTM * 32;               // + 6 KB

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

    // Column tiles ct0 .. ct1-1 of one row tile, as one stream of steps: the loads run three steps ahead of
    // the MFMAs across tile boundaries, so only the first tile of a workgroup waits for its first loads.
    template <int LIVE>
    static __device__ __forceinline__ void work(const MmqParams& p, const RowCtx& c, int ct0, int ct1) {
        extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
        constexpr int kStageBytes = 32 * LIVE * kARowBytes;
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int lane_c = lane & 31, lane_h = lane >> 5;
        const int steps = p.steps_per_seg, blocks = steps >> 2;
        const int out_cols = p.n;
        const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem_raw;
        // A tile loads: instruction i fills slots 256 i + tid: tile row 32 i + tid / 8, slot tid % 8.  Rows past the
        // group's end repeat its last row (their results are never stored).
        // With a row index the lane offsets carry the whole stored row (the host keeps the matrix under 4 GiB).
        const bf16_t* a_base = p.a[0] + (p.a_rows.on() ? 0 : (int64_t)c.row_begin * p.lda);
        uint32_t a_voff[LIVE];  // (lane offsets stay fixed; the step moves the scalar base)
#pragma unroll
        for (int i = 0; i < LIVE; i++) {
            const int r = 32 * i + (tid >> 3), s = tid & 7;
            const int kc = s ^ ((r >> 1) & 7);
            const int rr = min(r, c.rows_valid - 1);
            const int src = p.a_rows.on() ? p.a_rows.source(c.row_begin + rr) : rr;
            a_voff[i] = (uint32_t)(((int64_t)src * p.lda + kc * 8) * 2);
        }
        // The load cursor: (column tile, step) of the next step to request.  A lane's two packed rows are the
        // columns 64 wave + lane_c (+ 32) of the cursor's tile (columns past the segment's end repeat its last).
        int i_tile = ct0, i_step = 0;
        const uint8_t* w_tile;  // packed row of the cursor tile's first column (scalar)
        uint32_t wq_off[2];     // this lane's byte offset from there: its row, plus 16 h inside a quant group
        auto tile_origin = [&](int ct, int& seg, int& col0) __attribute__((always_inline)) {
            seg = ct / p.col_tiles_per_seg;
            col0 = (ct - seg * p.col_tiles_per_seg) * kTN;
        };
        auto cursor_rows = [&]() __attribute__((always_inline)) {
            int seg, col0;
            tile_origin(i_tile, seg, col0);
            w_tile = (seg ? p.w[1] : p.w[0]) + c.expert * p.w_expert_bytes + (int64_t)col0 * p.w_row_bytes;
#pragma unroll
            for (int cb = 0; cb < 2; cb++)
                wq_off[cb] = (uint32_t)(min(64 * wave + lane_c + 32 * cb, out_cols - 1 - col0) * (int)p.w_row_bytes + 16 * lane_h);
        };
        cursor_rows();
        // Requests one step: its A stage [LIVE loads], the block header when the step opens a 256-wide block [2],
        // its quant bytes [2].  SS = step index % 4 (a segment's step count is a multiple of 4).
        auto issue_group = [&](auto ss_c, u32x4_t* q, u32x4_t* h) __attribute__((always_inline)) {
            constexpr int SS = decltype(ss_c)::value;
            const uint32_t dst = lds_base + SS * kStageBytes + wave * 1024;
            const bf16_t* a_step = a_base + i_step * 64;
#pragma unroll
            for (int i = 0; i < LIVE; i++) load16_to_lds(dst + i * 4096, a_voff[i], a_step);
            const uint8_t* blk = w_tile + (i_step >> 2) * 144;
            if (SS == 0) {
#pragma unroll
                for (int cb = 0; cb < 2; cb++) asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(h[cb]) : "v"(wq_off[cb] - 16 * lane_h), "s"(blk), "n"(0) : "memory");
            }
#pragma unroll
            for (int cb = 0; cb < 2; cb++) asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(q[cb]) : "v"(wq_off[cb]), "s"(blk), "n"(16 + 32 * SS) : "memory");
            if (++i_step == steps) {  // on to the next tile; past the last one its first steps are requested again
                i_step = 0;
                if (i_tile + 1 < ct1) i_tile++, cursor_rows();
            }
        };

        f32x16_t acc[LIVE][2];
        // LDS read addresses: block rb is tile rows 32 rb + lane_c; sub-step I reads chunk 4 (I / 2) + 2 h + (I % 2)
        const uint8_t* a_row = smem_raw + lane_c * kARowBytes;
        int a_koff[4];
#pragma unroll
        for (int i = 0; i < 4; i++) a_koff[i] = a_slot(lane_c, 4 * (i >> 1) + 2 * lane_h + (i & 1)) * 16;
        bf16x8_t ao[LIVE];

        u32x4_t qr[4][2];      // ring over steps (step index % 4)
        u32x4_t hc[2], hn[2];  // headers of the current / next block
        issue_group(std::integral_constant<int, 0>{}, qr[0], hc);
        issue_group(std::integral_constant<int, 1>{}, qr[1], hc);
        issue_group(std::integral_constant<int, 2>{}, qr[2], hc);
        // the row tile's LA rows stay in LDS for all the column tiles of this workgroup (ranks up to 16)
        const bool la_resident = p.r_pad == 16;
        if (la_resident) {
            for (int id = tid; id < LIVE * 64; id += kThreadsWG) {
                const int row = id >> 1, half = id & 1;
                *(uint4*)(smem_raw + kLaBase + row * 32 + half * 16) = *(const uint4*)(p.la + (int64_t)(c.row_begin + min(row, c.rows_valid - 1)) * 16 + half * 8);
            }
        }
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (LIVE + 2)) : "memory");  // the first step's group has landed
        asm volatile("" : "+v"(hc[0]), "+v"(hc[1]), "+v"(qr[0][0]), "+v"(qr[0][1]));
        lds_barrier();
        Scales sc[2];
        uint32_t bx[2][4], by[2][4];  // B operands of the current / next sub-step, per column block
#pragma unroll
        for (int cb = 0; cb < 2; cb++) {
            sc[cb] = chunk_scales<0>(hc[cb]);
            decode_half<0, 0>(qr[0][cb], sc[cb], bx[cb]);
            decode_half<0, 1>(qr[0][cb], sc[cb], bx[cb]);
        }
#pragma unroll
        for (int rb = 0; rb < LIVE; rb++) ao[rb] = *(const bf16x8_t*)(a_row + a_koff[0] + rb * 32 * kARowBytes);
        // One sub-step, row block by row block: the block's two MFMAs, then its operand of the following sub-step
        // is read into the registers they have just released (a read has a whole round of MFMAs to land), then a
        // share of the decode of the next B operands (piece k = 2 cb + half).  A wave issues in order: the
        // decode arithmetic has to sit between the MFMAs to run in their shadow, and the scheduling barriers keep
        // it there.  The weights are the MFMA's first operand: the accumulators hold the transposed block.
        auto sub_step = [&](const uint32_t (*b)[4], int next_stage, int next_i, auto&& piece) __attribute__((always_inline)) {
            const uint8_t* src = a_row + next_stage * kStageBytes + a_koff[next_i];
            const bf16x8_t b0 = as_operand(b[0]), b1 = as_operand(b[1]);
#pragma unroll
            for (int rb = 0; rb < LIVE; rb++) {
                acc[rb][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b0, ao[rb], acc[rb][0], 0, 0, 0);
                acc[rb][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b1, ao[rb], acc[rb][1], 0, 0, 0);
                ao[rb] = *(const bf16x8_t*)(src + rb * 32 * kARowBytes);
                if (0 * LIVE / 4 == rb) piece(std::integral_constant<int, 0>{});
                if (1 * LIVE / 4 == rb) piece(std::integral_constant<int, 1>{});
                if (2 * LIVE / 4 == rb) piece(std::integral_constant<int, 2>{});
                if (3 * LIVE / 4 == rb) piece(std::integral_constant<int, 3>{});
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        bool stores_behind = false;  // the tile before this one went out through the staged store path
        for (int ct = ct0; ct < ct1; ct++) {
#pragma unroll
            for (int i = 0; i < LIVE; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;
            // this lane's two rows of the LoRA factor B (first 16 of the rank), requested ahead of the tile's steps
            bf16x8_t lb0[2];
            if (p.r_pad > 0) {
                int seg0, colz;
                tile_origin(ct, seg0, colz);
#pragma unroll
                for (int cb = 0; cb < 2; cb++)
                    lb0[cb] = *(const bf16x8_t*)(p.lb + c.expert * p.lb_expert_elems + ((int64_t)seg0 * out_cols + min(colz + 64 * wave + lane_c + 32 * cb, out_cols - 1)) * p.r_pad + lane_h * 8);
            }
            for (int kb = 0; kb < blocks; kb++) {
                // the four steps of a 256-wide block, written out so that the quant group index is a constant
                auto step = [&](auto s_c) __attribute__((always_inline)) {
                    constexpr int S = decltype(s_c)::value;
                    // All but the group requested one step ago have landed: the quant bytes of the next step, the
                    // next block's header when that step opens it, and this wave's part of the next A stage.
                    // Behind the barrier every wave's part has, and every wave is done with the stage of the
                    // step before this one, which the group requested now overwrites.
                    // (behind a tile's stores - at least 4 per full row block and one for the last, issued after the groups that are in flight - the first
                    // two steps allow that many more outstanding operations instead of waiting for the stores too)
                    if (S == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LIVE + 4) : "memory");
                    else if (S < 2 && kb == 0 && stores_behind) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(5 * LIVE - 1) : "memory");
                    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LIVE + 2) : "memory");
                    u32x4_t* qn = qr[(S + 1) & 3];
                    asm volatile("" : "+v"(qn[0]), "+v"(qn[1]));
                    if (S == 3) asm volatile("" : "+v"(hn[0]), "+v"(hn[1]));
                    lds_barrier();
                    issue_group(std::integral_constant<int, (S + 3) & 3>{}, qr[(S + 3) & 3], hn);
                    u32x4_t* qc = qr[S];
                    __builtin_amdgcn_sched_barrier(0);
                    sub_step(bx, S, 1, [&](auto k_c) __attribute__((always_inline)) {
                        constexpr int K = decltype(k_c)::value;
                        decode_half<1, K & 1>(qc[K >> 1], sc[K >> 1], by[K >> 1]);
                    });
                    sub_step(by, S, 2, [&](auto k_c) __attribute__((always_inline)) {
                        constexpr int K = decltype(k_c)::value;
                        decode_half<2, K & 1>(qc[K >> 1], sc[K >> 1], bx[K >> 1]);
                    });
                    sub_step(bx, S, 3, [&](auto k_c) __attribute__((always_inline)) {
                        constexpr int K = decltype(k_c)::value;
                        decode_half<3, K & 1>(qc[K >> 1], sc[K >> 1], by[K >> 1]);
                    });
                    // behind the last sub-step's MFMAs: the first operand of the next step (of the next tile behind
                    // a tile's last step), with the scales of its quant group
                    sub_step(by, (S + 1) & 3, 0, [&](auto k_c) __attribute__((always_inline)) {
                        constexpr int K = decltype(k_c)::value;
                        if ((K & 1) == 0) {
                            sc[K >> 1] = chunk_scales<(S + 1) & 3>(S == 3 ? hn[K >> 1] : hc[K >> 1]);
                        }
                        decode_half<0, K & 1>(qn[K >> 1], sc[K >> 1], bx[K >> 1]);
                    });
                };
                step(std::integral_constant<int, 0>{});
                step(std::integral_constant<int, 1>{});
                step(std::integral_constant<int, 2>{});
                step(std::integral_constant<int, 3>{});
                hc[0] = hn[0], hc[1] = hn[1];
            }
            // ---- LoRA term and store.  A lane holds four consecutive columns of one row: acc[rb][cb][i] is tile
            // row 32 rb + lane_c, column 64 wave + 32 cb + 8 (i / 4) + 4 h + (i % 4): a row block goes out as
            // whole rows.
            // (own, opaque copies of the lane coordinates: none of this part's address arithmetic may be hoisted in
            // front of the tile loop, where it would sit in registers through every main loop)
            int lane_e = lane;
            asm volatile("" : "+v"(lane_e));
            const int lane_ce = lane_e & 31, lane_he = lane_e >> 5;
            int seg, col0;
            tile_origin(ct, seg, col0);
            const int64_t ldc = p.ldc;
            bf16_t* const cbase = (bf16_t*)(seg ? p.c[1] : p.c[0]);
            const int rows_valid = c.rows_valid;
            const int col_quad = col0 + 64 * wave + 4 * lane_he;  // first column of this lane's quad at cb = 0, i / 4 = 0
            const bool vec = ((ldc & 7) == 0) && ((((uintptr_t)cbase) & 15) == 0) && col0 + kTN <= out_cols;
            stores_behind = vec;
            const int nl = p.r_pad >> 4;  // LoRA sub-steps (0: no LoRA)
            const float ls = nl > 0 ? p.lora_scale : 0.0f;
            const bf16_t* lb_lane[2];  // this lane's rows of the factor B (its two columns), 8 h elements in
#pragma unroll
            for (int cb = 0; cb < 2; cb++)
                lb_lane[cb] = p.lb + c.expert * p.lb_expert_elems + ((int64_t)seg * out_cols + min(col0 + 64 * wave + lane_ce + 32 * cb, out_cols - 1)) * p.r_pad + lane_he * 8;
            // the operands of the first 16 of the rank: LA rows from LDS (or, for ranks above 16, in one burst from
            // memory, the rest of the rank in place); the factor rows were requested ahead of the tile's steps
            bf16x8_t la0[LIVE];
            if (nl > 0) {
#pragma unroll
                for (int rb = 0; rb < LIVE; rb++)
                    la0[rb] = la_resident ? *(const bf16x8_t*)(smem_raw + kLaBase + (32 * rb + lane_ce) * 32 + lane_he * 16)
                                          : *(const bf16x8_t*)(p.la + (int64_t)(c.row_begin + min(32 * rb + lane_ce, rows_valid - 1)) * p.r_pad + lane_he * 8);
            }
#pragma unroll
            for (int rb = 0; rb < LIVE; rb++) {
                const int row = 32 * rb + lane_ce;
                f32x16_t t[2];  // LB . LA^T for this row block
#pragma unroll
                for (int cb = 0; cb < 2; cb++)
#pragma unroll
                    for (int e = 0; e < 16; e++) t[cb][e] = 0.0f;
                if (nl > 0) {
#pragma unroll
                    for (int cb = 0; cb < 2; cb++) t[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lb0[cb], la0[rb], t[cb], 0, 0, 0);
                    const bf16_t* la = p.la + (int64_t)(c.row_begin + min(row, rows_valid - 1)) * p.r_pad + lane_he * 8;
#pragma nounroll
                    for (int kk = 1; kk < nl; kk++) {
                        const bf16x8_t lao = *(const bf16x8_t*)(la + kk * 16);
#pragma unroll
                        for (int cb = 0; cb < 2; cb++)
                            t[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)(lb_lane[cb] + kk * 16), lao, t[cb], 0, 0, 0);
                    }
                }
                if (vec) {
                    // through this wave's staging block: 8-byte pieces in, whole 128-byte rows out (LDS accesses of
                    // one wave execute in order, so no wait is needed between the two)
                    uint8_t* const stage = smem_raw + kRingBytes + wave * (32 * kOutPitch);
#pragma unroll
                    for (int cb = 0; cb < 2; cb++)
#pragma unroll
                        for (int g = 0; g < 4; g++) {
                            float o[4];
#pragma unroll
                            for (int j = 0; j < 4; j++) o[j] = __builtin_fmaf(ls, t[cb][4 * g + j], acc[rb][cb][4 * g + j]);
                            *(uint2*)(stage + lane_ce * kOutPitch + (32 * cb + 8 * g + 4 * lane_he) * 2) = make_uint2(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]));
                        }
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int r = 8 * i + (lane_e >> 3), ch = lane_e & 7;
                        const uint4 v = *(const uint4*)(stage + r * kOutPitch + ch * 16);
                        if (32 * rb + r < rows_valid) *(uint4*)(cbase + (int64_t)(c.row_begin + 32 * rb + r) * ldc + col0 + 64 * wave + ch * 8) = v;
                    }
                } else if (rb < LIVE - 1 || row < rows_valid) {  // only the last live block can be partial
                    bf16_t* const crow = cbase + (int64_t)(c.row_begin + row) * ldc;
#pragma unroll
                    for (int cb = 0; cb < 2; cb++)
#pragma unroll
                        for (int i = 0; i < 16; i++) {
                            const int col = col_quad + 32 * cb + 8 * (i >> 2) + (i & 3);
                            if (col < out_cols) crow[col] = to_bf16(__builtin_fmaf(ls, t[cb][i], acc[rb][cb][i]));
                        }
                }
                __builtin_amdgcn_sched_barrier(0);  // one row block at a time: keeps the register need of this part small
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may land in LDS after the workgroup has gone
    }

    // Work assignment: a unit is a run of up to col_tiles_per_wg column tiles of one row tile.  Consecutive units
    // (which share an A tile) stay on one XCD; the split uses the number of row tiles that exist, not the
    // launch's upper bound.
    static __device__ __forceinline__ void run(const MmqParams& p) {
        const int col_tiles = p.nseg * p.col_tiles_per_seg;
        const int chunks = (col_tiles + p.col_tiles_per_wg - 1) / p.col_tiles_per_wg;
        const int row_tiles = p.tiles ? min(*p.num_tiles, p.max_row_tiles) : p.max_row_tiles;
        const int units = row_tiles * chunks;
        const int per_xcd = (units + 7) >> 3;
        const int slot = (int)(blockIdx.x >> 3);
        const int unit = (int)(blockIdx.x & 7) * per_xcd + slot;
        if (slot >= per_xcd || unit >= units) return;
        const int row_tile = unit / chunks, chunk = unit - row_tile * chunks;
        RowCtx c;
        int row_end;
        if (p.tiles) {
            const TileDesc t = p.tiles[row_tile];
            c.row_begin = t.row_begin, row_end = t.row_end, c.expert = t.expert;
        } else {
            c.row_begin = row_tile * kTM;
            row_end = min(p.m, c.row_begin + kTM);
            c.expert = 0;
        }
        c.rows_valid = row_end - c.row_begin;
        const int ct0 = chunk * p.col_tiles_per_wg, ct1 = min(col_tiles, ct0 + p.col_tiles_per_wg);
        switch ((c.rows_valid + 31) >> 5) {
            case 1: work<1>(p, c, ct0, ct1); break;
            case 2: work<2>(p, c, ct0, ct1); break;
            case 3: work<3>(p, c, ct0, ct1); break;
            case 4: work<4>(p, c, ct0, ct1); break;
            case 5: work<5>(p, c, ct0, ct1); break;
            default: work<6>(p, c, ct0, ct1); break;
        }
    }
};

__global__ __launch_bounds__(Direct::kThreadsWG) __attribute__((amdgpu_waves_per_eu(1, 1))) void mmq_direct_q4k_kernel(const MmqParams p) {
    Direct::run(p);
}

}  // namespace ggq
