// Q4_K grad-input ("NN") tile kernel, the sibling of the direct forward kernel (mmq_direct.h):
//
//   C[m, k] = sum_seg sum_n A_seg[m, n] * W_seg[n, k]  (+ s * LA[m, :] . LB[:, k])
//
// Same workgroup (four waves, one per SIMD), same A ring, same accumulator layout and store.  A column tile
// is the 256 columns of one packed block per weight row; wave w owns the block's quant group w (64 columns:
// the low nibbles of its 32 bytes are columns 0..31, the high nibbles columns 32..63 of the wave's range).
// Per contraction step of 64 weight rows, lane l loads the header and the 32 quant bytes of row l, three steps
// ahead, decodes them in registers with that row's two sub-block scales and writes the 64 values as one row of
// the wave's own [64 rows][64 columns] LDS block; the MFMA operands (eight consecutive contraction rows of one
// column per lane) come back out of that block through transposing reads.  LDS accesses of one wave execute in
// order, so the block needs neither a barrier nor a second buffer: a step's sixteen operand reads are issued at
// the end of the step before it, behind the writes of its rows, and the writes of the following step's rows
// come after them.
#pragma once
#include "mmq_direct.h"

namespace ggq {

struct DirectNN {
    static constexpr int kTM = kDirectBM, kTN = kDirectBN;
    static constexpr int kStages = 4;
    static constexpr int kThreadsWG = 256;
    static constexpr int kWPitch = 144;                                // bytes per row of a wave's decoded block (64 bf16 + pad)
    static constexpr int kWBlock = 64 * kWPitch;
    static constexpr int kRingBytes = kStages * kTM * kARowBytes;      // 96 KB
    static constexpr int kOutPitch = Direct::kOutPitch;
    static constexpr int kWBase = kRingBytes, kOutBase = kRingBytes + 4 * kWBlock;
    static constexpr int kLaBase = kOutBase + 4 * 32 * kOutPitch;      // the row tile's LA rows (rank <= 16), 32 bytes each
    static constexpr int kLdsBytes = kLaBase + kTM * 32;               // 96 + 36 + 18 + 6 KB

    struct RowCtx {
        int row_begin, rows_valid;
        int64_t expert;
    };
    struct Raw {  // one weight row's share of a step: block header, quant bytes 0..15 and 16..31 of the wave's group
        u32x4_t hdr, q0, q1;
    };
    struct Scales {
        float dl0, nm0, dl1, nm1;
    };
    // (scale, min) of sub-blocks 2w and 2w+1 of the block whose header is `hdr` (w: the wave, uniform)
    static __device__ __forceinline__ Scales wave_scales(const u32x4_t& hdr, int w) {
        const float d = half_bits_to_f32(hdr.x & 0xFFFFu), dmin = half_bits_to_f32(hdr.x >> 16);
        const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
        uint32_t sc0, m0, sc1, m1;
        if (w < 2) {  // sub-blocks 0..3: six low bits of bytes 2w, 2w+1 of the scale / min words
            const int sh = 16 * w;
            sc0 = (s0 >> sh) & 63u, m0 = (s1 >> sh) & 63u;
            sc1 = (s0 >> (sh + 8)) & 63u, m1 = (s1 >> (sh + 8)) & 63u;
        } else {      // sub-blocks 4..7: four bits from the third word, two from the top of the first two
            const int sh = 16 * (w - 2);
            sc0 = ((s2 >> sh) & 0xFu) | (((s0 >> (sh + 6)) & 3u) << 4);
            m0 = ((s2 >> (sh + 4)) & 0xFu) | (((s1 >> (sh + 6)) & 3u) << 4);
            sc1 = ((s2 >> (sh + 8)) & 0xFu) | (((s0 >> (sh + 14)) & 3u) << 4);
            m1 = ((s2 >> (sh + 12)) & 0xFu) | (((s1 >> (sh + 14)) & 3u) << 4);
        }
        Scales s;
        s.dl0 = d * (float)sc0 * kMixScale, s.nm0 = -(dmin * (float)m0);
        s.dl1 = d * (float)sc1 * (kMixScale / 16.0f), s.nm1 = -(dmin * (float)m1);  // high nibbles are read at bits 4..7
        return s;
    }
    // One word of quant bytes (four columns of either half): lo[0..1] = the low nibbles, hi[0..1] = the high ones.
    static __device__ __forceinline__ void decode_word(uint32_t w, const Scales& s, uint32_t* lo, uint32_t* hi) {
        const uint32_t w8 = w >> 8;
        const uint32_t l02 = w & 0x000F000Fu, l13 = w8 & 0x000F000Fu, h02 = w & 0x00F000F0u, h13 = w8 & 0x00F000F0u;
        lo[0] = pack_bf16(mix_lo(l02, s.dl0, s.nm0), mix_lo(l13, s.dl0, s.nm0));
        lo[1] = pack_bf16(mix_hi(l02, s.dl0, s.nm0), mix_hi(l13, s.dl0, s.nm0));
        hi[0] = pack_bf16(mix_lo(h02, s.dl1, s.nm1), mix_lo(h13, s.dl1, s.nm1));
        hi[1] = pack_bf16(mix_hi(h02, s.dl1, s.nm1), mix_hi(h13, s.dl1, s.nm1));
    }

    template <int LIVE>
    static __device__ __forceinline__ void work(const MmqParams& p, const RowCtx& c, int ct0, int ct1) {
        extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
        constexpr int kStageBytes = 32 * LIVE * kARowBytes;
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int lane_c = lane & 31, lane_h = lane >> 5;
        const int sps = p.steps_per_seg, steps = p.nseg * sps;  // contraction steps of 64 weight rows (a multiple of 4)
        const int out_cols = p.k;
        const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem_raw;
        // A tile loads as in the forward kernel: fixed lane offsets, the step moves the scalar base
        uint32_t a_voff[LIVE];
#pragma unroll
        for (int i = 0; i < LIVE; i++) {
            const int r = 32 * i + (tid >> 3), s = tid & 7;
            const int kc = s ^ ((r >> 1) & 7);
            a_voff[i] = (uint32_t)(((int64_t)min(r, c.rows_valid - 1) * p.lda + kc * 8) * 2);
        }
        const uint32_t w_lane = (uint32_t)lane * (uint32_t)p.w_row_bytes;  // this lane's weight row inside a step's 64
        // The load cursor: (column tile, step) of the next step to request.
        int i_tile = ct0, i_step = 0;
        auto issue_group = [&](auto ss_c, Raw& raw) __attribute__((always_inline)) {
            constexpr int SS = decltype(ss_c)::value;
            const int seg = i_step >= sps ? 1 : 0, local = i_step - seg * sps;
            const bf16_t* a_step = (seg ? p.a[1] : p.a[0]) + (int64_t)c.row_begin * p.lda + local * 64;
            const uint32_t dst = lds_base + SS * kStageBytes + wave * 1024;
#pragma unroll
            for (int i = 0; i < LIVE; i++) load16_to_lds(dst + i * 4096, a_voff[i], a_step);
            const uint8_t* blk = (seg ? p.w[1] : p.w[0]) + c.expert * p.w_expert_bytes + (int64_t)local * 64 * p.w_row_bytes + i_tile * 144;
            const uint8_t* grp = blk + 16 + 32 * wave;
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(raw.hdr) : "v"(w_lane), "s"(blk) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(raw.q0) : "v"(w_lane), "s"(grp) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, %2 offset:16" : "=v"(raw.q1) : "v"(w_lane), "s"(grp) : "memory");
            if (++i_step == steps) {  // on to the next tile; past the last one its first steps are requested again
                i_step = 0;
                if (i_tile + 1 < ct1) i_tile++;
            }
        };

        f32x16_t acc[LIVE][2];
        const uint8_t* a_row = smem_raw + lane_c * kARowBytes;
        int a_koff[4];  // sub-step I, lane half h: contraction elements 16 I + 8 h .. + 7 of the step
#pragma unroll
        for (int i = 0; i < 4; i++) a_koff[i] = a_slot(lane_c, 2 * i + lane_h) * 16;
        bf16x8_t ao[LIVE];

        // this wave's decoded block, the row this lane writes, and the transposing reads: within a group of 16 lanes,
        // lane L receives element L % 4 of the 8 bytes addressed by lanes L / 4 + 4 j.  Source lane s = L % 16 points
        // at contraction row s / 4 and columns 4 (s % 4) .. +3 of its group's 16 columns; groups 0, 1 take columns
        // 0..15 / 16..31 of a column block, groups 2, 3 the same columns eight contraction rows further on.
        uint8_t* const wblk = smem_raw + kWBase + wave * kWBlock;
        uint8_t* const w_my_row = wblk + lane * kWPitch;
        const int tr_group = lane >> 4, tr_s = lane & 15;
        const uint8_t* const tr_src = wblk + (8 * (tr_group >> 1) + (tr_s >> 2)) * kWPitch + (16 * (tr_group & 1) + 4 * (tr_s & 3)) * 2;
        auto read_b = [&](bf16x8_t (*b)[2]) __attribute__((always_inline)) {
#pragma unroll
            for (int ks = 0; ks < 4; ks++)
#pragma unroll
                for (int cb = 0; cb < 2; cb++) {
                    const uint8_t* src = tr_src + ks * 16 * kWPitch + cb * 64;
                    const v4i16_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)src);
                    const v4i16_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(src + 4 * kWPitch));
                    b[ks][cb] = __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                }
        };
        // decodes words 2 P, 2 P + 1 of `q` (eight columns of either half) and writes them to this lane's row
        auto decode_store = [&](const u32x4_t& q, int word_pair, int col0, const Scales& s) __attribute__((always_inline)) {
            uint32_t lo[4], hi[4];
            decode_word(q[2 * word_pair], s, lo, hi);
            decode_word(q[2 * word_pair + 1], s, lo + 2, hi + 2);
            *(uint4*)(w_my_row + col0 * 2) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            *(uint4*)(w_my_row + 64 + col0 * 2) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        };

        Raw raw[4];  // ring over steps (step index % 4)
        issue_group(std::integral_constant<int, 0>{}, raw[0]);
        issue_group(std::integral_constant<int, 1>{}, raw[1]);
        issue_group(std::integral_constant<int, 2>{}, raw[2]);
        // the row tile's LA rows stay in LDS for all the column tiles of this workgroup (ranks up to 16)
        const bool la_resident = p.r_pad == 16;
        if (la_resident) {
            for (int id = tid; id < LIVE * 64; id += kThreadsWG) {
                const int row = id >> 1, half = id & 1;
                *(uint4*)(smem_raw + kLaBase + row * 32 + half * 16) = *(const uint4*)(p.la + (int64_t)(c.row_begin + min(row, c.rows_valid - 1)) * 16 + half * 8);
            }
        }
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (LIVE + 3)) : "memory");  // the first step's group has landed
        asm volatile("" : "+v"(raw[0].hdr), "+v"(raw[0].q0), "+v"(raw[0].q1));
        lds_barrier();
        {
            const Scales s = wave_scales(raw[0].hdr, wave);
            decode_store(raw[0].q0, 0, 0, s), decode_store(raw[0].q0, 1, 8, s);
            decode_store(raw[0].q1, 0, 16, s), decode_store(raw[0].q1, 1, 24, s);
        }
#pragma unroll
        for (int rb = 0; rb < LIVE; rb++) ao[rb] = *(const bf16x8_t*)(a_row + a_koff[0] + rb * 32 * kARowBytes);
        bf16x8_t bops[2][4][2];  // B operands of the even / odd steps
        read_b(bops[0]);
        bool stores_behind = false;  // the tile before this one went out through the staged store path
        int t_step = 0;              // step inside the tile
        for (int ct = ct0; ct < ct1; ct++) {
#pragma unroll
            for (int i = 0; i < LIVE; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;
            // rows 0..15 of the LoRA factor x this wave's 64 columns (two 16-byte pieces per lane), requested ahead of
            // the tile's steps
            uint4 lbraw[2];
            if (p.r_pad > 0) {
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    const int id = lane + 64 * i, j = id >> 3, ch = id & 7;
                    lbraw[i] = *(const uint4*)(p.lb + c.expert * p.lb_expert_elems + (int64_t)min(j, p.lora_rank - 1) * out_cols + ct * kTN + 64 * wave + ch * 8);
                }
            }
            for (t_step = 0; t_step < steps; t_step += 4) {
                auto step = [&](auto s_c) __attribute__((always_inline)) {
                    constexpr int S = decltype(s_c)::value;
                    // All but the group requested one step ago have landed (see the forward kernel; behind a tile's
                    // stores the first two steps allow for them)
                    if (S < 2 && t_step == 0 && stores_behind) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(5 * LIVE) : "memory");
                    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LIVE + 3) : "memory");
                    Raw& rn = raw[(S + 1) & 3];
                    asm volatile("" : "+v"(rn.hdr), "+v"(rn.q0), "+v"(rn.q1));
                    lds_barrier();
                    issue_group(std::integral_constant<int, (S + 3) & 3>{}, raw[(S + 3) & 3]);
                    // this step's B operands were read at the end of the step before, behind the writes of its rows
                    bf16x8_t (*b)[2] = bops[S & 1];
                    Scales sn;
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int ks = 0; ks < 4; ks++) {
                        const int next_stage = ks == 3 ? (S + 1) & 3 : S;
                        const uint8_t* src = a_row + next_stage * kStageBytes + a_koff[(ks + 1) & 3];
#pragma unroll
                        for (int rb = 0; rb < LIVE; rb++) {
                            acc[rb][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[ks][0], ao[rb], acc[rb][0], 0, 0, 0);
                            acc[rb][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[ks][1], ao[rb], acc[rb][1], 0, 0, 0);
                            ao[rb] = *(const bf16x8_t*)(src + rb * 32 * kARowBytes);
                            // a share of the next step's decode behind each sub-step's first row block
                            if (rb == 0) {
                                if (ks == 0) sn = wave_scales(rn.hdr, wave);
                                decode_store(ks < 2 ? rn.q0 : rn.q1, ks & 1, 8 * ks, sn);
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                    // the next step's operands: its rows are in the block now (LDS accesses of a wave execute in order),
                    // and the writes of the step after it come behind these reads
                    read_b(bops[(S + 1) & 1]);
                };
                step(std::integral_constant<int, 0>{});
                step(std::integral_constant<int, 1>{});
                step(std::integral_constant<int, 2>{});
                step(std::integral_constant<int, 3>{});
            }
            // ---- LoRA term and store (accumulator layout and staging as in the forward kernel)
            int lane_e = lane;
            asm volatile("" : "+v"(lane_e));
            const int lane_ce = lane_e & 31, lane_he = lane_e >> 5;
            const int col0 = ct * kTN;
            const int64_t ldc = p.ldc;
            bf16_t* const cbase = (bf16_t*)p.c[0];
            const int rows_valid = c.rows_valid;
            const int col_quad = col0 + 64 * wave + 4 * lane_he;
            const bool vec = ((ldc & 7) == 0) && ((((uintptr_t)cbase) & 15) == 0) && col0 + kTN <= out_cols;
            stores_behind = vec;
            const int nl = p.r_pad >> 4;  // LoRA sub-steps (0: no LoRA)
            const float ls = nl > 0 ? p.lora_scale : 0.0f;
            const bf16_t* const lb_exp = p.lb + c.expert * p.lb_expert_elems;  // the factor A of this expert, [lora_rank][k]
            // eight factor rows (16 kk + 8 h ..) of this lane's column of block cb; rows past the rank are zero
            auto factor_operand = [&](int kk, int cb) __attribute__((always_inline)) {
                const int col = min(col0 + 64 * wave + lane_ce + 32 * cb, out_cols - 1);
                uint32_t e[8];
#pragma unroll
                for (int i = 0; i < 8; i++) {  // (unconditional loads of a clamped row, then a select: no branch, one round trip)
                    const int j = kk * 16 + lane_he * 8 + i;
                    const uint32_t v = lb_exp[(int64_t)min(j, p.lora_rank - 1) * out_cols + col];
                    e[i] = j < p.lora_rank ? v : 0u;
                }
                const u32x4_t v = {e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
                return __builtin_bit_cast(bf16x8_t, v);
            };
            // the operands of the first 16 of the rank for the whole tile in one burst (one memory round trip per
            // tile instead of one per row block); ranks above 16 load the rest in place
            bf16x8_t lb0[2], la0[LIVE];
            if (nl > 0) {
                if (col0 + kTN <= out_cols) {
                    // rows 0..15 of the factor x this wave's 64 columns: whole 128-byte rows into the staging block
                    // (rows past the rank as zeros), transposing reads back out - instead of sixteen 2-byte loads per lane
                    uint8_t* const stage = smem_raw + kOutBase + wave * (32 * kOutPitch);
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        const int id = lane_e + 64 * i, j = id >> 3, ch = id & 7;
                        *(uint4*)(stage + j * kOutPitch + ch * 16) = j < p.lora_rank ? lbraw[i] : zero4();
                    }
                    const int g4 = lane_e >> 4, s4 = lane_e & 15;
                    const uint8_t* src = stage + (8 * (g4 >> 1) + (s4 >> 2)) * kOutPitch + (16 * (g4 & 1) + 4 * (s4 & 3)) * 2;
#pragma unroll
                    for (int cb = 0; cb < 2; cb++) {
                        const v4i16_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(src + cb * 64));
                        const v4i16_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(src + cb * 64 + 4 * kOutPitch));
                        lb0[cb] = __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                    }
                } else {
#pragma unroll
                    for (int cb = 0; cb < 2; cb++) lb0[cb] = factor_operand(0, cb);
                }
#pragma unroll
                for (int rb = 0; rb < LIVE; rb++)
                    la0[rb] = la_resident ? *(const bf16x8_t*)(smem_raw + kLaBase + (32 * rb + lane_ce) * 32 + lane_he * 16)
                                          : *(const bf16x8_t*)(p.la + (int64_t)(c.row_begin + min(32 * rb + lane_ce, rows_valid - 1)) * p.r_pad + lane_he * 8);
            }
#pragma unroll
            for (int rb = 0; rb < LIVE; rb++) {
                const int row = 32 * rb + lane_ce;
                f32x16_t t[2];  // LB^T . LA^T for this row block
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
                        for (int cb = 0; cb < 2; cb++) t[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(factor_operand(kk, cb), lao, t[cb], 0, 0, 0);
                    }
                }
                if (vec) {
                    uint8_t* const stage = smem_raw + kOutBase + wave * (32 * kOutPitch);
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
                } else if (rb < LIVE - 1 || row < rows_valid) {
                    bf16_t* const crow = cbase + (int64_t)(c.row_begin + row) * ldc;
#pragma unroll
                    for (int cb = 0; cb < 2; cb++)
#pragma unroll
                        for (int i = 0; i < 16; i++) {
                            const int col = col_quad + 32 * cb + 8 * (i >> 2) + (i & 3);
                            if (col < out_cols) crow[col] = to_bf16(__builtin_fmaf(ls, t[cb][i], acc[rb][cb][i]));
                        }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may land in LDS after the workgroup has gone
    }

    static __device__ __forceinline__ void run(const MmqParams& p) {
        const int col_tiles = p.col_tiles_per_seg;
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

__global__ __launch_bounds__(DirectNN::kThreadsWG) __attribute__((amdgpu_waves_per_eu(1, 1))) void mmq_direct_nn_q4k_kernel(const MmqParams p) {
    DirectNN::run(p);
}

}  // namespace ggq
