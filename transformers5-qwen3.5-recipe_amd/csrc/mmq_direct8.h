// Q4_K forward ("NT") tile kernel in which the waves that issue the MFMAs decode the packed weights themselves.
//
//   C[m, n] = sum_k A[m, k] * W[n, k]  (+ s * LA[m, :] . LB[n, :])
//
// A workgroup is 512 lanes = eight waves, two per SIMD with 256 registers each, and computes tiles of up to 192 rows x
// 256 columns; wave w owns the 32 columns at 32 w of every row: up to six 32-row blocks of MFMA 32x32x16 accumulators.
// The kernel is instantiated per number of live 32-row blocks, so an expert group of any size up to 192 rows is one row
// tile and issues no MFMA on empty blocks.  Per contraction step of 64
//   * the A tile goes global -> LDS directly (no registers), three steps ahead, through a ring of four stages; rows are
//     unpadded with XOR-swizzled 16-byte slots (a_slot), every wave reads all of them;
//   * the packed quant bytes go global -> LDS directly as well, half a 256-wide block (two steps) of the wave's 32
//     columns at a time, four lanes per row so that a row's bytes are requested by adjacent lanes, into a ring of three
//     wave-private buffers; a block's 16-byte headers follow the same way, one lane per column, a block ahead;
//   * a lane reads its 16 quant bytes of the step from its wave's buffer and decodes them in registers into the operands
//     of the step's four MFMA sub-steps (mmq_direct.h).  No decoded weight ever touches LDS.
// A single wave issues at most one instruction per four to five cycles, whatever its kind, so a step's decode
// arithmetic, LDS reads, requests and waits (about eight instructions per MFMA) cannot hide behind that wave's own
// MFMAs; with two waves per SIMD one wave's MFMAs run while the other decodes, reads and waits.
// The weights are the MFMA's first operand, so a lane's accumulator registers hold four consecutive columns of one row;
// a finished row block goes through a wave-private LDS block and leaves as 64-byte row pieces.  The LoRA term is added
// there.  A workgroup takes a run of column tiles of its row tile and treats their steps as one stream, so the requests
// of a tile's first steps are in flight while the tile before it finishes.  The requests are inline-asm loads the
// compiler does not track; the step waits for them with exact counts (vector memory operations complete in issue order).
#pragma once
#include "mmq_direct.h"

namespace ggq {

struct Direct8 {
    static constexpr int kTM = kDirectBM, kTN = kDirectBN;
    static constexpr int kStages = 4;
    static constexpr int kWaves = 8;
    static constexpr int kThreadsWG = 64 * kWaves;
    static constexpr int kMaxLoadsPerStage = (kTM / 32 + 1) / 2;            // one direct-to-LDS instruction of the workgroup moves 64 rows
    static constexpr int kRingBytes = kStages * kMaxLoadsPerStage * 8192;  // 96 KB
    // Packed weights: per wave a ring of three buffers of 32 rows x 64 bytes, the quant bytes of two steps (half a
    // 256-wide block) of the wave's 32 columns.  A finished tile's output rows are staged in the buffer just read.
    static constexpr int kWBufBytes = 32 * 64, kWBufs = 3;
    static constexpr int kWBase = kRingBytes;
    static constexpr int kLaBase = kWBase + kWaves * kWBufs * kWBufBytes;  // + 48 KB: then the row tile's LA rows (rank <= 16), 32 bytes each
    static constexpr int kHdrBase = kLaBase + kTM * 32;                    // + 6 KB: then per wave the 16-byte headers of a block of its 32 columns
    static constexpr int kLdsBytes = kHdrBase + kWaves * 512;              // + 4 KB = 154 KB

    using Scales = Direct::Scales;
    using RowCtx = Direct::RowCtx;

    template <int LIVE>
    static __device__ __forceinline__ void work(const MmqParams& p, const RowCtx& c, int ct0, int ct1) {
        extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
        constexpr int NI = (LIVE + 1) / 2;       // direct-to-LDS instructions per A stage and wave
        constexpr int kStageBytes = NI * 8192;   // (an odd block count leaves the last 32 rows of a stage as copies of the last row)
        constexpr int kStores = 2 * LIVE - 1;    // 16-byte store instructions a tile certainly issues per wave (two per full row block, one for the last)
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int lane_c = lane & 31, lane_h = lane >> 5;
        const int steps = p.steps_per_seg, blocks = steps >> 2;
        const int out_cols = p.n;
        const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem_raw;
        // A tile loads: instruction i fills slots 512 i + tid: tile row 64 i + tid / 8, slot tid % 8.  Rows past the
        // group's end repeat its last row (their results are never stored).  With a row index the lane offsets carry
        // the whole stored row (the host keeps the matrix under 4 GiB).
        const bf16_t* a_base = p.a[0] + (p.a_rows.on() ? 0 : (int64_t)c.row_begin * p.lda);
        uint32_t a_voff[NI];
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const int r = 64 * i + (tid >> 3), s = tid & 7;
            const int kc = s ^ ((r >> 1) & 7);
            const int rr = min(r, c.rows_valid - 1);
            const int src = p.a_rows.on() ? p.a_rows.source(c.row_begin + rr) : rr;
            a_voff[i] = (uint32_t)(((int64_t)src * p.lda + kc * 8) * 2);
        }
        auto tile_origin = [&](int ct, int& seg, int& col0) __attribute__((always_inline)) {
            seg = ct / p.col_tiles_per_seg;
            col0 = (ct - seg * p.col_tiles_per_seg) * kTN;
        };
        // The A cursor: (column tile, step) of the next step to request; it only moves the contraction offset.
        int i_step = 0;
        int a_wr = 0;  // byte offset of the stage the next request fills
        auto issue_a = [&]() __attribute__((always_inline)) {
            const uint32_t dst = lds_base + a_wr + wave * 1024;
            const bf16_t* a_step = a_base + i_step * 64;
#pragma unroll
            for (int i = 0; i < NI; i++) load16_to_lds(dst + i * 8192, a_voff[i], a_step);
            a_wr = a_wr == (kStages - 1) * kStageBytes ? 0 : a_wr + kStageBytes;
            if (++i_step == steps) i_step = 0;
        };
        // The W cursor: (column tile, 256-wide block) of the next block to request.  Packed quant bytes go global ->
        // LDS directly, half a block (two steps) of the wave's 32 columns per buffer: instruction j moves 64 bytes of
        // each of the rows 16 j .. 16 j + 15, four lanes per row, so that a row's bytes are requested by adjacent lanes
        // (a lane-per-row load of 16 bytes costs the vector cache one access per lane).  The 16-byte chunks of a row
        // are XOR-swizzled with (row / 2) % 4: the reads below (lane = row, 16 bytes) meet no bank conflict.
        int w_tile_i = ct0, w_blk = 0;
        const uint8_t* w_next;  // packed row of the cursor tile's first column, at the cursor's block (scalar)
        uint32_t wq_voff[2];    // this lane's byte offset from there in instruction j
        uint32_t wh_voff;       // and for the block header of its column (both lane halves read the same 16 bytes)
        auto w_cursor_rows = [&]() __attribute__((always_inline)) {
            int seg, col0;
            tile_origin(w_tile_i, seg, col0);
            w_next = (seg ? p.w[1] : p.w[0]) + c.expert * p.w_expert_bytes + (int64_t)col0 * p.w_row_bytes;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int row = 16 * j + (lane >> 2), kc = (lane & 3) ^ ((row >> 1) & 3);
                wq_voff[j] = (uint32_t)min(32 * wave + row, out_cols - 1 - col0) * (uint32_t)p.w_row_bytes + 16u * kc;
            }
            wh_voff = (uint32_t)min(32 * wave + lane_c, out_cols - 1 - col0) * (uint32_t)p.w_row_bytes;
        };
        w_cursor_rows();
        int w_wr = 0;  // byte offset (inside the wave's ring) of the buffer the next request fills
        const uint32_t w_lds = lds_base + kWBase + wave * (kWBufs * kWBufBytes);
        auto issue_w_half = [&](auto half_c) __attribute__((always_inline)) {  // quant bytes 64 half .. +63 of the cursor's block
            constexpr int HALF = decltype(half_c)::value;
            // (no immediate offset: a direct-to-LDS load adds it to the LDS address as well)
            const uint8_t* src = w_next + w_blk * 144 + 16 + 64 * HALF;
#pragma unroll
            for (int j = 0; j < 2; j++) load16_to_lds(w_lds + w_wr + j * 1024, wq_voff[j], src);
            w_wr = w_wr == (kWBufs - 1) * kWBufBytes ? 0 : w_wr + kWBufBytes;
        };
        // The headers of the cursor's block go global -> LDS as well, one lane per column (a load of 64 lanes that names
        // each of 32 addresses twice costs the vector cache twice the accesses), into the wave's one header buffer: a
        // block's headers are read out of it (below) a whole step before the request of the next block's goes out.
        const uint32_t hdr_lds = lds_base + kHdrBase + wave * 512;
        const uint8_t* const hdr_row = smem_raw + kHdrBase + wave * 512 + lane_c * 16;
        auto issue_w_header = [&]() __attribute__((always_inline)) {
            if (lane_h == 0) load16_to_lds(hdr_lds, wh_voff, w_next + w_blk * 144);
        };
        auto w_cursor_advance = [&]() __attribute__((always_inline)) {  // past the last block of the last tile the cursor stays
            if (w_blk + 1 < blocks) w_blk++;
            else if (w_tile_i + 1 < ct1) w_tile_i++, w_blk = 0, w_cursor_rows();
        };

        f32x16_t acc[LIVE];
        // LDS read addresses: block rb is tile rows 32 rb + lane_c; sub-step I reads chunk 4 (I / 2) + 2 h + (I % 2)
        const uint8_t* a_row = smem_raw + lane_c * kARowBytes;
        int a_koff[4];
#pragma unroll
        for (int i = 0; i < 4; i++) a_koff[i] = a_slot(lane_c, 4 * (i >> 1) + 2 * lane_h + (i & 1)) * 16;
        bf16x8_t ao[LIVE];
        // this lane's 16 quant bytes of the first / second step of a buffer
        const uint8_t* const w_rows = smem_raw + kWBase + wave * (kWBufs * kWBufBytes) + lane_c * 64;
        const int w_roff[2] = {((lane_h) ^ ((lane_c >> 1) & 3)) * 16, ((2 + lane_h) ^ ((lane_c >> 1) & 3)) * 16};
        int w_rd = 0;  // byte offset of the buffer of the current pair of steps
        int a_rd = 0;  // byte offset of the A stage of the current step

        u32x4_t qc, qn;  // quant bytes of the current / next step
        u32x4_t hc, hn;  // headers of the current / next block
        issue_w_header();
        issue_w_half(std::integral_constant<int, 0>{});
        issue_w_half(std::integral_constant<int, 1>{});
        w_cursor_advance();
        issue_a();
        issue_a();
        issue_a();
        // the first 16 rank columns of the row tile's LA rows stay in LDS for all the column tiles of this workgroup: the
        // epilogue then reads them with LDS reads, which no pending store or request stands in front of
        if (p.r_pad > 0) {
            for (int id = tid; id < LIVE * 64; id += kThreadsWG) {
                const int row = id >> 1, half = id & 1;
                *(uint4*)(smem_raw + kLaBase + row * 32 + half * 16) = *(const uint4*)(p.la + (int64_t)(c.row_begin + min(row, c.rows_valid - 1)) * p.r_pad + half * 8);
            }
        }
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NI) : "memory");  // the first block's bytes and the first step's A stage have landed
        lds_barrier();
        hc = *(const u32x4_t*)hdr_row;
        asm volatile("" : "+v"(hc));  // (read out before the request below refills the buffer)
        // Phase p = the last sub-step of step p - 1 and the first three of step p: it reads A stage p only, and its
        // requests (behind the barrier that opens it) fill the stage of step p - 1.  A phase's first A instruction goes
        // out in its first sub-step, the others in the next step's first two; ph_dst / ph_src carry them across.
        uint32_t ph_dst;
        const bf16_t* ph_src;
        auto phase_open = [&]() __attribute__((always_inline)) {
            ph_dst = lds_base + a_wr + wave * 1024;
            ph_src = a_base + i_step * 64;
            a_wr = a_wr == (kStages - 1) * kStageBytes ? 0 : a_wr + kStageBytes;
            if (++i_step == steps) i_step = 0;
        };
        auto request_a = [&](auto i_c) __attribute__((always_inline)) {
            constexpr int I = decltype(i_c)::value;
            if constexpr (I < NI) load16_to_lds(ph_dst + I * 8192, a_voff[I], ph_src);
        };
        issue_w_half(std::integral_constant<int, 0>{});  // phase 0: the first half of block 1 and its headers, A of step 3
        issue_w_header();
        phase_open();
        request_a(std::integral_constant<int, 0>{});
        qc = *(const u32x4_t*)(w_rows + w_roff[0]);
        Scales sc;
        uint32_t bx[4], by[4];  // B operands of the current / next sub-step
        sc = Direct::chunk_scales<0>(hc);
        Direct::decode_half<0, 0>(qc, sc, bx);
        Direct::decode_half<0, 1>(qc, sc, bx);
#pragma unroll
        for (int rb = 0; rb < LIVE; rb++) ao[rb] = *(const bf16x8_t*)(a_row + a_koff[0] + rb * 32 * kARowBytes);
        // One sub-step, row block by row block: the block's MFMA, then its operand of the following sub-step is read
        // into the registers it has just released, then a half of the decode of the next B operand.
        auto sub_step = [&](const uint32_t* b, int next_stage_off, int next_i, auto&& piece, auto&& request) __attribute__((always_inline)) {
            const uint8_t* src = a_row + next_stage_off + a_koff[next_i];
            const bf16x8_t b0 = Direct::as_operand(b);
#pragma unroll
            for (int rb = 0; rb < LIVE; rb++) {
                acc[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b0, ao[rb], acc[rb], 0, 0, 0);
                if (rb == 0) request();  // this sub-step's share of the step's memory requests, behind its first MFMA
                ao[rb] = *(const bf16x8_t*)(src + rb * 32 * kARowBytes);
                if (0 * LIVE / 2 == rb) piece(std::integral_constant<int, 0>{});
                if (1 * LIVE / 2 == rb) piece(std::integral_constant<int, 1>{});
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        bool stores_behind = false;  // the tile before this one went out through the staged store path
        for (int ct = ct0; ct < ct1; ct++) {
#pragma unroll
            for (int i = 0; i < LIVE; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][e] = 0.0f;
            // This lane's row of the LoRA factor B (first 16 of the rank), requested ahead of the tile's steps with a load of
            // the same untracked kind as the other requests (without a LoRA term: 16 bytes of the packed weights, unused).
            // A load the compiler tracks would be waited for at its use in the epilogue with vmcnt(0): behind the next
            // tile's first requests, and behind the stores of the row blocks before it, one round trip each.
            u32x4_t lb0_raw;
            {
                int seg0, colz;
                tile_origin(ct, seg0, colz);
                const void* src = p.r_pad > 0 ? (const void*)(p.lb + c.expert * p.lb_expert_elems + ((int64_t)seg0 * out_cols + min(colz + 32 * wave + lane_c, out_cols - 1)) * p.r_pad + lane_h * 8)
                                              : (const void*)(p.w[0] + c.expert * p.w_expert_bytes);
                asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(lb0_raw) : "v"(src) : "memory");
            }
            // the first half of the next block's quant bytes goes out with a block's last sub-step, except behind a
            // tile's last block, where the store path below still uses the buffer it would fill
            if (ct > ct0) issue_w_half(std::integral_constant<int, 0>{});
            for (int kb = 0; kb < blocks; kb++) {
                // Requests per phase P (= step index % 4): the A stage three steps on [NI]; P = 0: the first half of the
                // next block's quant bytes [2] and its headers [1]; P = 2: the second half [2].
                auto step = [&](auto s_c) __attribute__((always_inline)) {
                    constexpr int S = decltype(s_c)::value;
                    // the quant bytes of the next step: second step of this buffer, or the first of the next one
                    const int w_rd_next = w_rd == (kWBufs - 1) * kWBufBytes ? 0 : w_rd + kWBufBytes;
                    qn = *(const u32x4_t*)(w_rows + ((S & 1) ? w_rd_next + w_roff[0] : w_rd + w_roff[1]));
                    if (S == 3) hn = *(const u32x4_t*)hdr_row;  // the next block's headers: requested a block ago, landed by the last step's wait
                    const int a_rd_next = a_rd == (kStages - 1) * kStageBytes ? 0 : a_rd + kStageBytes;
                    __builtin_amdgcn_sched_barrier(0);
                    sub_step(bx, a_rd, 1, [&](auto k_c) __attribute__((always_inline)) { Direct::decode_half<1, decltype(k_c)::value>(qc, sc, by); },
                             [&]() __attribute__((always_inline)) { request_a(std::integral_constant<int, 1>{}); });
                    sub_step(by, a_rd, 2, [&](auto k_c) __attribute__((always_inline)) { Direct::decode_half<2, decltype(k_c)::value>(qc, sc, bx); },
                             [&]() __attribute__((always_inline)) { request_a(std::integral_constant<int, 2>{}); });
                    sub_step(bx, a_rd, 3, [&](auto k_c) __attribute__((always_inline)) { Direct::decode_half<3, decltype(k_c)::value>(qc, sc, by); },
                             [&]() __attribute__((always_inline)) {});
                    // End of phase S.  All but the requests of this phase and the one before it have landed: this wave's
                    // part of A stage S + 1 (requested two phases ago) and every packed byte requested before that.  Behind
                    // the barrier every wave's part has, and every wave is done reading stage S, which the next phase's
                    // requests overwrite.  Requests complete in order, so the distance matters: packed bytes come from
                    // HBM, and a wait that covered requests only one step old stalled on them.
                    // (Behind a tile's stores and the request of the LoRA factor row, which went out inside phase 0's requests,
                    // the first two steps allow for them.)
                    constexpr int kGroup[4] = {NI + 3, NI, NI + 2, NI};
                    constexpr int kBehind = kGroup[S] + kGroup[(S + 3) & 3];
                    if (S < 2 && kb == 0 && stores_behind) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kBehind + kStores + 1) : "memory");
                    else if (S < 2 && kb == 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kBehind + 1) : "memory");
                    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kBehind) : "memory");
                    lds_barrier();
                    phase_open();
                    // behind the last sub-step's MFMAs: the first operand of the next step (of the next tile behind a
                    // tile's last step), with the scales of its quant group
                    sub_step(by, a_rd_next, 0, [&](auto k_c) __attribute__((always_inline)) {
                        constexpr int K = decltype(k_c)::value;
                        if (K == 0) sc = Direct::chunk_scales<(S + 1) & 3>(S == 3 ? hn : hc);
                        Direct::decode_half<0, K>(qn, sc, bx);
                    }, [&]() __attribute__((always_inline)) {
                        if (S == 3 && kb + 1 < blocks) issue_w_half(std::integral_constant<int, 0>{});
                        if (S == 3) issue_w_header();  // (behind the barrier: every read of the buffer's last contents has returned)
                        if (S == 1) issue_w_half(std::integral_constant<int, 1>{});
                        request_a(std::integral_constant<int, 0>{});
                    });
                    qc = qn;
                    a_rd = a_rd_next;
                    if (S & 1) w_rd = w_rd_next;
                    if (S == 2) w_cursor_advance();
                };
                step(std::integral_constant<int, 0>{});
                step(std::integral_constant<int, 1>{});
                step(std::integral_constant<int, 2>{});
                step(std::integral_constant<int, 3>{});
                hc = hn;
            }
            // ---- LoRA term and store.  A lane holds four consecutive columns of one row: acc[rb][i] is tile row
            // 32 rb + lane_c, column 32 wave + 8 (i / 4) + 4 h + (i % 4): a row block goes out as 64-byte row pieces.
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
            const int col_quad = col0 + 32 * wave + 4 * lane_he;  // first column of this lane's quad at i / 4 = 0
            const bool vec = ((ldc & 7) == 0) && ((((uintptr_t)cbase) & 15) == 0) && col0 + kTN <= out_cols;
            stores_behind = vec;
            const int nl = p.r_pad >> 4;  // LoRA sub-steps (0: no LoRA)
            const float ls = nl > 0 ? p.lora_scale : 0.0f;
            const bf16_t* const lb_lane = p.lb + c.expert * p.lb_expert_elems + ((int64_t)seg * out_cols + min(col0 + 32 * wave + lane_ce, out_cols - 1)) * p.r_pad + lane_he * 8;
            // (the factor row landed long ago: every step's wait leaves only the requests of two phases outstanding)
            asm volatile("" : "+v"(lb0_raw));
            const bf16x8_t lb0 = __builtin_bit_cast(bf16x8_t, lb0_raw);
            bf16x8_t la0[LIVE];
            if (nl > 0) {
#pragma unroll
                for (int rb = 0; rb < LIVE; rb++)
                    la0[rb] = *(const bf16x8_t*)(smem_raw + kLaBase + (32 * rb + lane_ce) * 32 + lane_he * 16);
            }
            // the staging block: the buffer of the pair of steps just finished (the next request into it comes with the
            // next tile's first step, after the reads below have returned their data to the stores)
            uint8_t* const stage = smem_raw + kWBase + wave * (kWBufs * kWBufBytes) + (w_rd == 0 ? (kWBufs - 1) * kWBufBytes : w_rd - kWBufBytes);
#pragma unroll
            for (int rb = 0; rb < LIVE; rb++) {
                const int row = 32 * rb + lane_ce;
                f32x16_t t;  // LB . LA^T for this row block
#pragma unroll
                for (int e = 0; e < 16; e++) t[e] = 0.0f;
                if (nl > 0) {
                    t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lb0, la0[rb], t, 0, 0, 0);
                    const bf16_t* la = p.la + (int64_t)(c.row_begin + min(row, rows_valid - 1)) * p.r_pad + lane_he * 8;
#pragma nounroll
                    for (int kk = 1; kk < nl; kk++)
                        t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)(lb_lane + kk * 16), *(const bf16x8_t*)(la + kk * 16), t, 0, 0, 0);
                }
                if (vec) {
                    // 8-byte pieces in (the 16-byte chunk g of a row sits at position g ^ (row / 4) % 4), 64-byte row pieces
                    // out; LDS accesses of one wave execute in order, so no wait is needed between the two
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
                } else if (rb < LIVE - 1 || row < rows_valid) {  // only the last live block can be partial
                    bf16_t* const crow = cbase + (int64_t)(c.row_begin + row) * ldc;
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int col = col_quad + 8 * (i >> 2) + (i & 3);
                        if (col < out_cols) crow[col] = to_bf16(__builtin_fmaf(ls, t[i], acc[rb][i]));
                    }
                }
                __builtin_amdgcn_sched_barrier(0);  // one row block at a time: keeps the register need of this part small
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may land in LDS after the workgroup has gone
    }

    // Work assignment as in the four-wave kernel: a unit is a run of up to col_tiles_per_wg column tiles of one row
    // tile; consecutive units (which share an A tile) stay on one XCD.
    static __device__ __forceinline__ void run(const MmqParams& p) {
        const int col_tiles = p.nseg * p.col_tiles_per_seg;
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

__global__ __launch_bounds__(Direct8::kThreadsWG) __attribute__((amdgpu_waves_per_eu(2, 2))) void mmq_direct8_q4k_kernel(const MmqParams p) {
    Direct8::run(p);
}

}  // namespace ggq
