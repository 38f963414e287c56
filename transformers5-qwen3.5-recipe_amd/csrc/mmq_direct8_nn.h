// Q4_K grad-input ("NN") tile kernel with register decoding and two waves per SIMD, the sibling of the forward
// kernel in mmq_direct8.h:
//
//   C[m, k] = sum_seg sum_n A_seg[m, n] * W_seg[n, k]  (+ s * LA[m, :] . LB[:, k])
//
// A workgroup is 512 lanes = eight waves; a column tile is the 256 columns of one packed block per weight row, and
// wave w owns sub-block w of it (32 columns: the low or the high nibbles of quant group w / 2), for up to six 32-row
// blocks of 32x32x16 accumulators.  Per contraction step of 64 weight rows
//   * the A tile (cotangent rows) goes global -> LDS directly, as in the forward kernel;
//   * the step's packed bytes - 64 rows x (16-byte header + 128 quant bytes), contiguous per row - go global -> LDS
//     directly too, requested by the whole workgroup with adjacent lanes on adjacent bytes (one row's bytes asked
//     for lane by lane, 16 bytes each, cost the vector cache one access per lane), and are shared by the eight waves;
//   * lane l of every wave decodes weight row l for the wave's 32 columns (one scale and one min per row) and
//     writes the 32 values as one row of the wave's own [64][32] LDS block; the MFMA operands (eight consecutive
//     contraction rows of one column per lane) come back out of that block through transposing reads.  LDS accesses
//     of one wave execute in order, so the block needs neither a barrier nor a second buffer.
// The weights are the MFMA's first operand (accumulator registers hold four consecutive columns of one row), the
// store path and the LoRA term are those of the forward kernel; the factor tile is transposed through the same block.
#pragma once
#include "mmq_direct8.h"

namespace ggq {

struct Direct8NN {
    static constexpr int kTM = kDirectBM, kTN = kDirectBN;
    static constexpr int kWaves = 8;
    static constexpr int kThreadsWG = 64 * kWaves;
    static constexpr int kARingBytes = 9 * 8192;                       // 4 stages x 16 KB (up to 128 rows) or 3 x 24 KB (up to 192)
    static constexpr int kRawStageBytes = 64 * 128 + 64 * 16;          // a step's quant bytes [64 rows][128], then its headers [64][16]
    static constexpr int kRawBase = kARingBytes;
    static constexpr int kDecPitch = 80;                               // bytes per row of a wave's decoded block (32 bf16 + pad)
    static constexpr int kDecBlock = 64 * kDecPitch;
    static constexpr int kDecBase = kRawBase + 4 * kRawStageBytes;
    static constexpr int kLaBase = kDecBase + kWaves * kDecBlock;      // the row tile's LA rows (rank <= 16), 32 bytes each
    static constexpr int kLdsBytes = kLaBase + kTM * 32;               // 72 + 36 + 40 + 6 = 154 KB

    using RowCtx = Direct::RowCtx;

    // (scale * 2^24, -min) of sub-block sb (wave-uniform) of the block whose header is `hdr`; the scale of an odd
    // sub-block is divided by 16: its nibbles are read at bits 4..7
    static __device__ __forceinline__ void sub_block_scale(const u32x4_t& hdr, int sb, float& dl, float& nm) {
        const float d = half_bits_to_f32(hdr.x & 0xFFFFu), dmin = half_bits_to_f32(hdr.x >> 16);
        const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
        uint32_t sc, m;
        if (sb < 4) {
            sc = (s0 >> (8 * sb)) & 63u, m = (s1 >> (8 * sb)) & 63u;
        } else {
            const int sh = 8 * (sb - 4);
            sc = ((s2 >> sh) & 0xFu) | (((s0 >> (sh + 6)) & 3u) << 4);
            m = ((s2 >> (sh + 4)) & 0xFu) | (((s1 >> (sh + 6)) & 3u) << 4);
        }
        dl = d * (float)sc * ((sb & 1) ? kMixScale / 16.0f : kMixScale);
        nm = -(dmin * (float)m);
    }
    // One word of quant bytes -> the four values of this wave's nibble half (mask selects it), as two packed pairs.
    static __device__ __forceinline__ void decode_word(uint32_t w, uint32_t mask, float dl, float nm, uint32_t* out) {
        const uint32_t e02 = w & mask, e13 = (w >> 8) & mask;
        out[0] = pack_bf16(mix_lo(e02, dl, nm), mix_lo(e13, dl, nm));
        out[1] = pack_bf16(mix_hi(e02, dl, nm), mix_hi(e13, dl, nm));
    }
    // Transposing read of eight contraction rows x one column per lane out of a block of rows `pitch` bytes apart:
    // within a group of 16 lanes, lane L receives element L % 4 of the 8 bytes addressed by lanes L / 4 + 4 j.
    static __device__ __forceinline__ bf16x8_t read_tr(const uint8_t* src, int pitch) {
        const v4i16_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)src);
        const v4i16_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(src + 4 * pitch));
        return __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }

    template <int LIVE>
    static __device__ __forceinline__ void work(const MmqParams& p, const RowCtx& c, int ct0, int ct1) {
        extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
        constexpr int NI = (LIVE + 1) / 2;        // direct-to-LDS instructions per A stage and wave
        constexpr int kStages = LIVE <= 4 ? 4 : 3;
        constexpr int kStageBytes = NI * 8192;
        constexpr int kGroup = NI + 1;            // requests per phase and wave: A [NI], quant bytes [1]; wave 0 one more: the headers
        constexpr int kStores = 2 * LIVE - 1;     // 16-byte store instructions a tile certainly issues per wave
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int lane_c = lane & 31, lane_h = lane >> 5;
        const int sps = p.steps_per_seg, steps = p.nseg * sps;  // contraction steps of 64 weight rows (an even number)
        const int out_cols = p.k;
        const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem_raw;
        // A tile loads as in the forward kernel: fixed lane offsets, the step moves the scalar base
        uint32_t a_voff[NI];
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const int r = 64 * i + (tid >> 3), s = tid & 7;
            const int kc = s ^ ((r >> 1) & 7);
            const int rr = min(r, c.rows_valid - 1);
            // with a row index (one cotangent matrix read through it) the lane offsets carry the whole stored row
            const int src = p.a_rows.on() ? p.a_rows.source(c.row_begin + rr) : rr;
            a_voff[i] = (uint32_t)(((int64_t)src * p.lda + kc * 8) * 2);
        }
        // packed bytes of a step: lane t of the workgroup moves quant chunk (t % 8) ^ swizzle of weight row t / 8
        // (the 16-byte chunks of a row are XOR-swizzled like an A row's: the per-row reads below meet no bank conflict);
        // wave 0 moves the 64 headers of the step with one request (eight requests of eight lanes each, one per wave, cost
        // 1.9 % of the configs[2] step more: what a request costs is its issue, not its bytes)
        const uint32_t wq_voff = (uint32_t)((tid >> 3) * (int)p.w_row_bytes + 16 + 16 * ((tid & 7) ^ (((tid >> 3) >> 1) & 7)));
        const uint32_t wh_voff = (uint32_t)(lane * (int)p.w_row_bytes);
        const bool hdr_wave = wave == 0;
        // waits: at most `behind` phases of requests (and `extra` other operations) of this wave outstanding
        auto wait_behind = [&](auto extra_c) __attribute__((always_inline)) {
            constexpr int X = decltype(extra_c)::value;
            if (hdr_wave) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kStages - 2) * (kGroup + 1) + X) : "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kStages - 2) * kGroup + X) : "memory");
        };
        // Cursors: (column tile, step) of the next A stage / packed-byte stage to request; past the last tile they
        // stay on it (what they request again is never used).
        int a_step_i = 0, a_wr = 0;
        int w_tile_i = ct0, w_step_i = 0, w_wr = 0;
        auto step_src_a = [&](int st) __attribute__((always_inline)) {
            const int seg = st >= sps ? 1 : 0, local = st - seg * sps;
            return (seg ? p.a[1] : p.a[0]) + (p.a_rows.on() ? 0 : (int64_t)c.row_begin * p.lda) + local * 64;
        };
        auto step_src_w = [&](int ct, int st) __attribute__((always_inline)) {
            const int seg = st >= sps ? 1 : 0, local = st - seg * sps;
            return (seg ? p.w[1] : p.w[0]) + c.expert * p.w_expert_bytes + (int64_t)local * 64 * p.w_row_bytes + ct * 144;
        };
        uint32_t ph_dst;       // the open phase's A requests (its first goes out at once, the others in the next sub-steps)
        const bf16_t* ph_src;
        auto open_a = [&]() __attribute__((always_inline)) {
            ph_dst = lds_base + a_wr + wave * 1024;
            ph_src = step_src_a(a_step_i);
            a_wr = a_wr == (kStages - 1) * kStageBytes ? 0 : a_wr + kStageBytes;
            if (++a_step_i == steps) a_step_i = 0;
        };
        auto request_a = [&](auto i_c) __attribute__((always_inline)) {
            constexpr int I = decltype(i_c)::value;
            if constexpr (I < NI) load16_to_lds(ph_dst + I * 8192, a_voff[I], ph_src);
        };
        auto request_w = [&]() __attribute__((always_inline)) {
            const uint8_t* src = step_src_w(w_tile_i, w_step_i);
            const uint32_t dst = lds_base + kRawBase + w_wr;
            load16_to_lds(dst + wave * 1024, wq_voff, src);
            if (hdr_wave) load16_to_lds(dst + 64 * 128, wh_voff, src);
            w_wr = w_wr == (kStages - 1) * kRawStageBytes ? 0 : w_wr + kRawStageBytes;
            if (++w_step_i == steps) {
                w_step_i = 0;
                if (w_tile_i + 1 < ct1) w_tile_i++;
            }
        };

        f32x16_t acc[LIVE];
        const uint8_t* a_row = smem_raw + lane_c * kARowBytes;
        int a_koff[4];  // sub-step I, lane half h: contraction elements 16 I + 8 h .. + 7 of the step
#pragma unroll
        for (int i = 0; i < 4; i++) a_koff[i] = a_slot(lane_c, 2 * i + lane_h) * 16;
        bf16x8_t ao[LIVE];
        // this lane's weight row in a packed-byte stage: the two chunks of its wave's quant group, and its header
        const int grp = wave >> 1;
        const uint8_t* const raw_row = smem_raw + kRawBase + lane * 128;
        const int raw_qoff[2] = {((2 * grp) ^ ((lane >> 1) & 7)) * 16, ((2 * grp + 1) ^ ((lane >> 1) & 7)) * 16};
        const uint8_t* const raw_hdr = smem_raw + kRawBase + 64 * 128 + lane * 16;
        const uint32_t nib_mask = (wave & 1) ? 0x00F000F0u : 0x000F000Fu;
        // this wave's decoded block, the row this lane writes, and where its transposing reads start
        uint8_t* const dblk = smem_raw + kDecBase + wave * kDecBlock;
        uint8_t* const d_my_row = dblk + lane * kDecPitch;
        const int tr_group = lane >> 4, tr_s = lane & 15;
        const uint8_t* const tr_src = dblk + (8 * (tr_group >> 1) + (tr_s >> 2)) * kDecPitch + (16 * (tr_group & 1) + 4 * (tr_s & 3)) * 2;
        auto read_b = [&](bf16x8_t* b) __attribute__((always_inline)) {
#pragma unroll
            for (int ks = 0; ks < 4; ks++) b[ks] = read_tr(tr_src + ks * 16 * kDecPitch, kDecPitch);
        };
        u32x4_t rq0, rq1, rh;  // raw bytes of the step being decoded
        float dl, nm;
        auto raw_fetch = [&](int off) __attribute__((always_inline)) {
            rq0 = *(const u32x4_t*)(raw_row + off + raw_qoff[0]);
            rq1 = *(const u32x4_t*)(raw_row + off + raw_qoff[1]);
            rh = *(const u32x4_t*)(raw_hdr + off);
        };
        // quarter Q (0..3) of the row: words 2 Q, 2 Q + 1 of the 32 quant bytes -> columns 8 Q .. 8 Q + 7
        auto decode_quarter = [&](auto q_c) __attribute__((always_inline)) {
            constexpr int Q = decltype(q_c)::value;
            const u32x4_t& src = Q < 2 ? rq0 : rq1;
            uint32_t o[4];
            decode_word(src[2 * (Q & 1)], nib_mask, dl, nm, o);
            decode_word(src[2 * (Q & 1) + 1], nib_mask, dl, nm, o + 2);
            *(uint4*)(d_my_row + Q * 16) = make_uint4(o[0], o[1], o[2], o[3]);
        };

        // ---- prologue: packed bytes of steps 0 and 1 and the A stage of step 0 first, then the phases before phase 0
        request_w();
        request_w();
        open_a();
        request_a(std::integral_constant<int, 0>{});
        request_a(std::integral_constant<int, 1>{});
        request_a(std::integral_constant<int, 2>{});
#pragma unroll
        for (int q = 0; q < kStages - 2; q++) {
            open_a();
            request_a(std::integral_constant<int, 0>{});
            request_a(std::integral_constant<int, 1>{});
            request_a(std::integral_constant<int, 2>{});
            request_w();
        }
        // the first 16 rank columns of the row tile's LA rows stay in LDS for all the column tiles of this workgroup: the
        // epilogue then reads them with LDS reads, which no pending store or request stands in front of
        if (p.r_pad > 0) {
            for (int id = tid; id < LIVE * 64; id += kThreadsWG) {
                const int row = id >> 1, half = id & 1;
                *(uint4*)(smem_raw + kLaBase + row * 32 + half * 16) = *(const uint4*)(p.la + (int64_t)(c.row_begin + min(row, c.rows_valid - 1)) * p.r_pad + half * 8);
            }
        }
        wait_behind(std::integral_constant<int, 0>{});
        lds_barrier();
        int a_rd = 0;   // byte offset of the A stage of the current step
        int w_rd = 0;   // byte offset of the packed-byte stage of the step being decoded (one ahead of the A stage)
        bf16x8_t bops[2][4];  // B operands of the even / odd steps
        raw_fetch(0);
        sub_block_scale(rh, wave, dl, nm);
        decode_quarter(std::integral_constant<int, 0>{});
        decode_quarter(std::integral_constant<int, 1>{});
        decode_quarter(std::integral_constant<int, 2>{});
        decode_quarter(std::integral_constant<int, 3>{});
        read_b(bops[0]);
        w_rd = kRawStageBytes;
#pragma unroll
        for (int rb = 0; rb < LIVE; rb++) ao[rb] = *(const bf16x8_t*)(a_row + a_koff[0] + rb * 32 * kARowBytes);
        // phase 0: A of step kStages - 1, packed bytes of step kStages (into the stage of step 0: every wave has read it)
        lds_barrier();
        request_w();
        open_a();
        request_a(std::integral_constant<int, 0>{});

        // One sub-step: the row blocks' MFMAs one by one, each followed by the read of its operand of the following
        // sub-step (into the registers it has just released) and by whatever `slot` puts behind that MFMA.
        auto sub_step = [&](const bf16x8_t& b0, int next_stage_off, int next_i, auto&& slot) __attribute__((always_inline)) {
            const uint8_t* src = a_row + next_stage_off + a_koff[next_i];
            auto one = [&](auto rb_c) __attribute__((always_inline)) {
                constexpr int RB = decltype(rb_c)::value;
                if constexpr (RB < LIVE) {
                    acc[RB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b0, ao[RB], acc[RB], 0, 0, 0);
                    ao[RB] = *(const bf16x8_t*)(src + RB * 32 * kARowBytes);
                    slot(rb_c);
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            one(std::integral_constant<int, 0>{}), one(std::integral_constant<int, 1>{}), one(std::integral_constant<int, 2>{});
            one(std::integral_constant<int, 3>{}), one(std::integral_constant<int, 4>{}), one(std::integral_constant<int, 5>{});
        };
        bool stores_behind = false;  // the tile before this one went out through the staged store path
        int relax = 0;               // steps of this tile whose wait still allows for the stores of the tile before
        for (int ct = ct0; ct < ct1; ct++) {
#pragma unroll
            for (int i = 0; i < LIVE; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][e] = 0.0f;
            // rows 0..15 of the LoRA factor x this wave's 32 columns (one 16-byte piece per lane), requested ahead of
            // the tile's steps
            // (a load of the same untracked kind as the other requests; without a LoRA term: 16 bytes of the packed weights,
            // unused.  A load the compiler tracks would be waited for at its use in the epilogue with vmcnt(0): behind the
            // next tile's first requests, and behind the stores of the row blocks before it, one round trip each.)
            u32x4_t lbraw;
            {
                const void* src = p.r_pad > 0 ? (const void*)(p.lb + c.expert * p.lb_expert_elems + (int64_t)min(lane >> 2, p.lora_rank - 1) * out_cols + min(ct * kTN + 32 * wave + (lane & 3) * 8, out_cols - 8))
                                              : (const void*)(p.w[0] + c.expert * p.w_expert_bytes);
                asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(lbraw) : "v"(src) : "memory");
            }
            relax = kStages - 2;
            for (int st = 0; st < steps; st += 2) {
                // One step.  Its B operands were read at the end of the step before; the next step's weight rows are
                // decoded behind its MFMAs (a half of a quarter row per slot) and read back at its end.
                auto step = [&](auto par_c) __attribute__((always_inline)) {
                    constexpr int P = decltype(par_c)::value;
                    const bf16x8_t* b = bops[P];
                    raw_fetch(w_rd);
                    const int a_rd_next = a_rd == (kStages - 1) * kStageBytes ? 0 : a_rd + kStageBytes;
                    __builtin_amdgcn_sched_barrier(0);
                    // The next step's weight row of this lane is decoded in eight pieces (one quant word = four columns
                    // each) spread evenly over the 3 LIVE MFMA slots of the first three sub-steps, so that the block is
                    // complete before the phase ends; its transposing reads are spread over the last sub-step's slots and
                    // have landed when the next step starts.
                    uint32_t o[4];
                    auto decode_piece = [&](auto hp_c) __attribute__((always_inline)) {
                        constexpr int HP = decltype(hp_c)::value, Q = HP >> 1, K = HP & 1;
                        const u32x4_t& src = Q < 2 ? rq0 : rq1;
                        if (HP == 0) sub_block_scale(rh, wave, dl, nm);
                        decode_word(src[2 * (Q & 1) + K], nib_mask, dl, nm, o + 2 * K);
                        if (K == 1) *(uint4*)(d_my_row + Q * 16) = make_uint4(o[0], o[1], o[2], o[3]);
                    };
                    auto decode_slots = [&](auto i_c) __attribute__((always_inline)) {  // sub-step I's share
                        return [&](auto rb_c) __attribute__((always_inline)) {
                            constexpr int T = decltype(i_c)::value * LIVE + decltype(rb_c)::value;
                            auto maybe = [&](auto hp_c) __attribute__((always_inline)) {
                                if constexpr (decltype(hp_c)::value * 3 * LIVE / 8 == T) decode_piece(hp_c);
                            };
                            maybe(std::integral_constant<int, 0>{}), maybe(std::integral_constant<int, 1>{}), maybe(std::integral_constant<int, 2>{}), maybe(std::integral_constant<int, 3>{});
                            maybe(std::integral_constant<int, 4>{}), maybe(std::integral_constant<int, 5>{}), maybe(std::integral_constant<int, 6>{}), maybe(std::integral_constant<int, 7>{});
                            if constexpr (decltype(rb_c)::value == 0 && decltype(i_c)::value == 0) request_a(std::integral_constant<int, 1>{});
                            if constexpr (decltype(rb_c)::value == 0 && decltype(i_c)::value == 1) request_a(std::integral_constant<int, 2>{});
                        };
                    };
                    sub_step(b[0], a_rd, 1, decode_slots(std::integral_constant<int, 0>{}));
                    sub_step(b[1], a_rd, 2, decode_slots(std::integral_constant<int, 1>{}));
                    sub_step(b[2], a_rd, 3, decode_slots(std::integral_constant<int, 2>{}));
                    // End of the phase: all but the requests of this phase (and, with four stages, the one before it)
                    // have landed - this wave's parts of the next step's A stage and of the packed bytes of the step
                    // after it.  Behind the barrier every wave's parts have, and every wave is done with the stages the
                    // next phase's requests overwrite.  (Behind a tile's stores and the request of the LoRA factor piece, which went out
                    // inside a phase's requests, the steps whose awaited requests are older than that phase allow for them.)
                    if (relax > 0 && stores_behind) wait_behind(std::integral_constant<int, kStores + 1>{});
                    else if (relax > 0) wait_behind(std::integral_constant<int, 1>{});
                    else wait_behind(std::integral_constant<int, 0>{});
                    lds_barrier();
                    open_a();
                    bf16x8_t* bn = bops[P ^ 1];
                    sub_step(b[3], a_rd_next, 0, [&](auto rb_c) __attribute__((always_inline)) {
                        constexpr int RB = decltype(rb_c)::value;
                        if constexpr (RB == 0) {
                            request_w();
                            request_a(std::integral_constant<int, 0>{});
                        }
                        // the next step's operands: its rows are in the block (LDS accesses of a wave execute in order), and
                        // the writes of the step after it come behind these reads
#pragma unroll
                        for (int ks = 0; ks < 4; ks++)
                            if (ks * LIVE / 4 == RB) bn[ks] = read_tr(tr_src + ks * 16 * kDecPitch, kDecPitch);
                    });
                    a_rd = a_rd_next;
                    w_rd = w_rd == (kStages - 1) * kRawStageBytes ? 0 : w_rd + kRawStageBytes;
                    relax--;
                };
                step(std::integral_constant<int, 0>{});
                step(std::integral_constant<int, 1>{});
            }
            // ---- LoRA term and store (accumulator layout and staging as in the forward kernel; the staging block is this
            // wave's decoded block, whose rows have been read)
            int lane_e = lane;
            asm volatile("" : "+v"(lane_e));
            const int lane_ce = lane_e & 31, lane_he = lane_e >> 5;
            const int col0 = ct * kTN;
            const int64_t ldc = p.ldc;
            bf16_t* const cbase = (bf16_t*)p.c[0];
            const int rows_valid = c.rows_valid;
            const int col_quad = col0 + 32 * wave + 4 * lane_he;
            const bool vec = ((ldc & 7) == 0) && ((((uintptr_t)cbase) & 15) == 0);
            stores_behind = vec;
            const int nl = p.r_pad >> 4;  // LoRA sub-steps (0: no LoRA)
            const float ls = nl > 0 ? p.lora_scale : 0.0f;
            const bf16_t* const lb_exp = p.lb + c.expert * p.lb_expert_elems;  // the factor A of this expert, [lora_rank][k]
            // eight factor rows (16 kk + 8 h ..) of this lane's column; rows past the rank are zero
            auto factor_operand = [&](int kk) __attribute__((always_inline)) {
                const int col = col0 + 32 * wave + lane_ce;
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
            bf16x8_t lb0, la0[LIVE];
            if (nl > 0) {
                // rows 0..15 of the factor x this wave's 32 columns: whole 64-byte rows into the block (rows past the rank
                // as zeros), one transposing read back out
                const int j = lane_e >> 2, ch = lane_e & 3;
                // The piece has landed: the first wait of the tile that no longer allows for it (step kStages - 2 <= 2) is
                // behind us; the host launches this kernel for contractions of four steps or more.
                asm volatile("" : "+v"(lbraw));
                *(u32x4_t*)(dblk + j * kDecPitch + ch * 16) = j < p.lora_rank ? lbraw : u32x4_t{0u, 0u, 0u, 0u};
                const int g4 = lane_e >> 4, s4 = lane_e & 15;
                lb0 = read_tr(dblk + (8 * (g4 >> 1) + (s4 >> 2)) * kDecPitch + (16 * (g4 & 1) + 4 * (s4 & 3)) * 2, kDecPitch);
#pragma unroll
                for (int rb = 0; rb < LIVE; rb++)
                    la0[rb] = *(const bf16x8_t*)(smem_raw + kLaBase + (32 * rb + lane_ce) * 32 + lane_he * 16);
            }
            uint8_t* const stage = dblk + 32 * kDecPitch;  // 2 KB behind the factor rows
#pragma unroll
            for (int rb = 0; rb < LIVE; rb++) {
                const int row = 32 * rb + lane_ce;
                f32x16_t t;  // LB^T . LA^T for this row block
#pragma unroll
                for (int e = 0; e < 16; e++) t[e] = 0.0f;
                if (nl > 0) {
                    t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lb0, la0[rb], t, 0, 0, 0);
                    const bf16_t* la = p.la + (int64_t)(c.row_begin + min(row, rows_valid - 1)) * p.r_pad + lane_he * 8;
#pragma nounroll
                    for (int kk = 1; kk < nl; kk++) t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(factor_operand(kk), *(const bf16x8_t*)(la + kk * 16), t, 0, 0, 0);
                }
                if (vec) {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        float o[4];
#pragma unroll
                        for (int j = 0; j < 4; j++) o[j] = __builtin_fmaf(ls, t[4 * g + j], acc[rb][4 * g + j]);
                        *(uint2*)(stage + lane_ce * 64 + ((g ^ ((lane_ce >> 2) & 3)) * 16) + 8 * lane_he) = make_uint2(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]));
                    }
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        const int r = 16 * i + (lane_e >> 2), ch = (lane_e & 3) ^ ((r >> 2) & 3);
                        const uint4 v = *(const uint4*)(stage + r * 64 + (lane_e & 3) * 16);
                        if (32 * rb + r < rows_valid) *(uint4*)(cbase + (int64_t)(c.row_begin + 32 * rb + r) * ldc + col0 + 32 * wave + ch * 8) = v;
                    }
                } else if (rb < LIVE - 1 || row < rows_valid) {
                    bf16_t* const crow = cbase + (int64_t)(c.row_begin + row) * ldc;
#pragma unroll
                    for (int i = 0; i < 16; i++) crow[col_quad + 8 * (i >> 2) + (i & 3)] = to_bf16(__builtin_fmaf(ls, t[i], acc[rb][i]));
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
        // Row tile rt runs on XCD rt % 8 (the table lists the tiles with the most rows first: every XCD gets its
        // share of them, and takes its own in that order); the column-tile runs of a row tile follow one another there.
        const int slot = (int)(blockIdx.x >> 3);
        const int row_tile = (slot / chunks) * 8 + (int)(blockIdx.x & 7), chunk = slot % chunks;
        if (row_tile >= row_tiles) return;
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
        if (c.rows_valid <= 0) return;  // (the table builders emit no empty tile; a descriptor that is one must not index row -1)
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

__global__ __launch_bounds__(Direct8NN::kThreadsWG) __attribute__((amdgpu_waves_per_eu(2, 2))) void mmq_direct8_nn_q4k_kernel(const MmqParams p) {
    Direct8NN::run(p);
}

}  // namespace ggq
