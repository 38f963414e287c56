// IQ2_XXS forward ("NT") kernel for expert groups of a few dozen rows, in which the waves that issue the MFMAs decode the
// packed weights themselves.
//
//   C[m, n] = sum_k A[m, k] * W[n, k]  (+ s * LA[m, :] . LB[n, :])
//
// With 64 rows per expert a decoded weight feeds two 32-row MFMA blocks: there is too little matrix work per weight to hide
// a producer / consumer pipeline behind (decode -> LDS store -> barrier -> LDS read), and that chain paces the tile kernel.
// Here a workgroup is 512 lanes = eight waves and computes tiles of up to 128 rows x 256 columns; wave w owns the 32 columns
// at 32 w.  Per contraction step of 64
//   * the A tile (rows x 128 bytes) goes global -> LDS directly, three steps ahead, through a ring of four stages (one
//     instruction per wave and 64 rows; rows unpadded with XOR-swizzled 16-byte slots, a_slot);
//   * lane (column lane % 32, half h = lane / 32) loads the 8 bytes of run 2 step + h of its column's packed row, four
//     steps ahead, into one of four register sets (and a block's scale one block ahead), decodes the run's 32 weights in
//     registers (the selector and sign tables of Fmt<kIQ2_XXS> in LDS, read two groups of 8 weights ahead of their use) and
//     feeds group i of the run to MFMA i of the step: an MFMA sums its 16 contraction slots in any order, so the lane half
//     reads the matching 16-byte slot (4 h + i) of the A row.  No decoded weight touches LDS.
// All requests of the loop are inline-asm loads the compiler does not track: one per 64 rows and one run per wave and step,
// and a scale on the first step of a block, in a fixed order, waited for with exact counts (vector memory operations
// complete in issue order).  A register such a load writes must not be touched before its wait: the waits name the
// registers they cover as operands, and a landed run moves to registers of its own through an instruction the compiler
// cannot fold away, so that its register pair is dead until the next request names it (the compiler otherwise carries
// the pair into the next loop iteration with a copy made while the load is still on its way).
// The workgroup keeps 74 KB of LDS (68 KB dynamic, the tables static) and at most 128 registers per lane, so two workgroups share a compute unit and cover
// each other's barriers.  The weights are the MFMA's first operand, so a lane's accumulator registers hold four consecutive
// columns of one row; a finished row block goes through a wave-private LDS block (in the ring, idle by then) and leaves as
// 64-byte row pieces, the LoRA term added there.
#pragma once
#include "mmq_direct.h"

namespace ggq {

typedef uint32_t dw_u32x2_t __attribute__((ext_vector_type(2)));

struct SmallIq2 {
    static constexpr int kTM = kSmallBM, kTN = kSmallBN;
    static constexpr int kStages = 4;
    static constexpr int kWaves = 8;
    static constexpr int kThreadsWG = 64 * kWaves;
    static constexpr int kStageBytes = kTM * 128;                                   // 16 KB
    static constexpr int kLaBase = kStages * kStageBytes;                           // 64 KB: then the row tile's LA rows, 32 bytes each
    static constexpr int kLdsBytes = kLaBase + kTM * 32;                            // + 4 KB = 68 KB of dynamic LDS
    // (the decoder's tables, 6 KB, are a static array: it sits at LDS address 0, which the compiler then folds into the lookups)
    static constexpr int kOutBase = 0;  // eight 2 KB staging blocks of the epilogue: over the ring, which a finished tile no longer needs

    using RowCtx = Direct::RowCtx;

    template <int LIVE>
    static __device__ __forceinline__ void work(const MmqParams& p, const RowCtx& c, int ct0, int ct1, uint32_t* table_words) {
        extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int lane_c = lane & 31, lane_h = lane >> 5;
        const int steps = p.steps_per_seg;  // a multiple of 4: the contraction is a whole number of 256-wide blocks
        const int out_cols = p.n;
        const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem_raw;
        for (int i = tid; i < Fmt<kIQ2_XXS>::kTableWords; i += kThreadsWG) table_words[i] = Fmt<kIQ2_XXS>::table_word(i, i < 1024 ? d_iq2xxs_grid_mm[i >> 2] : 0);
        const uint2* const tables = (const uint2*)table_words;
        // the first 16 rank columns of the row tile's LA rows stay in LDS for all the column tiles of this workgroup
        if (p.r_pad > 0) {
            for (int id = tid; id < LIVE * 64; id += kThreadsWG) {
                const int row = id >> 1, half = id & 1;
                *(uint4*)(smem_raw + kLaBase + row * 32 + half * 16) = *(const uint4*)(p.la + (int64_t)(c.row_begin + min(row, c.rows_valid - 1)) * p.r_pad + half * 8);
            }
        }
        __syncthreads();
        // A tile loads: the workgroup's one instruction fills slots tid: tile row tid / 8, slot tid % 8.  Rows past the
        // group's end repeat its last row (their results are never stored).  With a row index the lane offsets carry the
        // whole stored row (the host keeps the matrix under 4 GiB).
        const bf16_t* const a_base = p.a[0] + (p.a_rows.on() ? 0 : (int64_t)c.row_begin * p.lda);
        constexpr int NA = (LIVE + 1) / 2;  // instructions per step: 64 rows each
        uint32_t a_voff[NA];
#pragma unroll
        for (int i = 0; i < NA; i++) {
            const int r = 64 * i + (tid >> 3), s = tid & 7;
            const int kc = s ^ ((r >> 1) & 7);
            const int rr = min(r, c.rows_valid - 1);
            const int src = p.a_rows.on() ? p.a_rows.source(c.row_begin + rr) : rr;
            a_voff[i] = (uint32_t)(((int64_t)src * p.lda + kc * 8) * 2);
        }
        auto issue_a = [&](int step, int stage) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < NA; i++) load16_to_lds(lds_base + stage * kStageBytes + i * 8192 + wave * 1024, a_voff[i], a_base + min(step, steps - 1) * 64);
        };
        auto tile_origin = [&](int ct, int& seg, int& col0) __attribute__((always_inline)) {
            seg = ct / p.col_tiles_per_seg;
            col0 = (ct - seg * p.col_tiles_per_seg) * kTN;
        };
        // LDS read addresses: block rb is tile rows 32 rb + lane_c; MFMA i of a step reads contraction elements
        // 32 h + 8 i .. + 7 of the step: chunk 4 h + i
        const uint8_t* const a_row = smem_raw + lane_c * 128;
        const int a_koff0 = a_slot(lane_c, 4 * lane_h) * 16;  // chunk 4 h + i sits at this offset ^ 16 i

        f32x16_t acc[LIVE];
        for (int ct = ct0; ct < ct1; ct++) {
#pragma unroll
            for (int i = 0; i < LIVE; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][e] = 0.0f;
            int seg, col0;
            tile_origin(ct, seg, col0);
            // packed row of this lane's column (columns past the end repeat the last one; their results are never stored):
            // run 2 step + h sits at block (step / 4) * 66 + 2 + 8 (2 (step % 4) + h), the block's scale at its first two bytes
            const uint8_t* const w_base = (seg ? p.w[1] : p.w[0]) + c.expert * p.w_expert_bytes;
            const uint32_t wd_voff = (uint32_t)min(col0 + 32 * wave + lane_c, out_cols - 1) * (uint32_t)p.w_row_bytes;  // (unsigned: a weight plane may pass 2 GiB)
            const uint32_t wq_voff = wd_voff + 2 + 8 * lane_h;
            dw_u32x2_t q[4];  // the runs of steps 4 b .. 4 b + 3, each reloaded for the next block as soon as it is decoded
            uint32_t d_cur = 0, d_next;  // the scales of this block and of the next
            auto issue_q = [&](dw_u32x2_t& qr, int step) __attribute__((always_inline)) {
                const int st = min(step, steps - 1);
                asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(qr) : "v"(wq_voff), "s"(w_base + (st >> 2) * 66 + 16 * (st & 3)) : "memory");
            };
            auto issue_d = [&](uint32_t& dr, int step) __attribute__((always_inline)) {
                asm volatile("global_load_ushort %0, %1, %2" : "=v"(dr) : "v"(wd_voff), "s"(w_base + (min(step, steps - 1) >> 2) * 66) : "memory");
            };
            // The order every step keeps: [A of step t + 3] [run of step t + 4], and the first step of a block then asks for the
            // next block's scale.  The requests ahead of the loop follow the same order.
            issue_d(d_next, 0);
            issue_q(q[0], 0);
            issue_a(0, 0);
            issue_q(q[1], 1);
            issue_a(1, 1);
            issue_q(q[2], 2);
            issue_a(2, 2);
            issue_q(q[3], 3);
            // Table reads run two groups of 8 weights ahead of the MFMAs, over the step boundaries too: the selectors and sign
            // words of the first two groups of step 0 are asked for here, once its run has landed.
            const uint4* const sel = (const uint4*)tables;
            const uint4* const flip = sel + 256;
            // (the registers a wait covers are operands of the wait itself: their readers cannot be moved ahead of it)
            asm volatile("s_waitcnt vmcnt(%1)" : "+v"(q[0]) : "n"(3 * NA + 3) : "memory");
            // The words of a landed run move to registers of their own through an instruction the compiler cannot fold
            // away: the run's register pair is then dead until its next request, so that request can name the same pair, and
            // no value that is still on its way is ever carried into the next loop iteration by a compiler-made copy.
            uint32_t cur_idx, cur_aux;
            auto take_run = [&](const dw_u32x2_t& qr) __attribute__((always_inline)) {
                asm volatile("v_mov_b32 %0, %2\n\tv_mov_b32 %1, %3" : "=&v"(cur_idx), "=&v"(cur_aux) : "v"(qr.x), "v"(qr.y));
            };
            take_run(q[0]);
            uint4 e[2], f[2];  // selectors and sign words of the next two groups
            auto ask = [&](int slot, int l) __attribute__((always_inline)) {
                e[slot] = sel[(cur_idx >> (8 * l)) & 0xFFu], f[slot] = flip[(cur_aux >> (7 * l)) & 127u];
            };
            ask(0, 0);
            ask(1, 1);
            for (int t0 = 0; t0 < steps; t0 += 4) {
                auto step = [&](auto s_c) __attribute__((always_inline)) {
                    constexpr int S = decltype(s_c)::value;
                    // A step needs its A stage (NA instructions, which opened the requests of the step three back) and the
                    // run of the step after it (requested right behind that stage): the NA + 1 requests of each of the two
                    // steps since, and the scale request if one of those three steps made one, may still be on their way.
                    // Behind the barrier every wave's part of the stage has landed, and every wave is done reading the
                    // stage of the step before, which this step's request overwrites.
                    if (S == 0) {  // and the block's scale: requested by the first step of the block before (ahead of the loop for block 0)
                        asm volatile("s_waitcnt vmcnt(%2)" : "+v"(q[1]), "+v"(d_next) : "n"(2 * NA + 2) : "memory");
                        asm volatile("v_mov_b32 %0, %1" : "=v"(d_cur) : "v"(d_next));  // (a copy the compiler cannot fold: see take_run)
                    } else {
                        asm volatile("s_waitcnt vmcnt(%1)" : "+v"(q[(S + 1) & 3]) : "n"(2 * NA + 3) : "memory");
                    }
                    lds_barrier();
                    issue_a(t0 + S + 3, (S + 3) & 3);
                    issue_q(q[S], t0 + S + 4);  // (its words sit in cur_idx, cur_aux since the step before)
                    if (S == 0) issue_d(d_next, t0 + 4);
                    const float db = half_bits_to_f32(d_cur & 0xFFFFu) * (0.5f + (float)(cur_aux >> 28)) * 0.25f;
                    // the three products a weight can be, as bf16: bytes 0..5 of {hi : lo}
                    const uint32_t lo = pack_bf16(db * 8.0f, db * 25.0f), hi = pack_bf16(db * 43.0f, 0.0f);
                    const uint8_t* src = a_row + S * kStageBytes;
                    // the step's scale leaves cur_aux here: group 2 below moves the next run's words in
                    constexpr int kFirst = LIVE < 4 ? LIVE : 2;  // (four row blocks: the A operands come in two halves, for registers)
                    constexpr bool kAhead = LIVE <= 2;           // (few row blocks: the A operands of a group are read during the group before)
                    bf16x8_t a[kFirst], a_next[kFirst];
                    if (kAhead) {
#pragma unroll
                        for (int rb = 0; rb < kFirst; rb++) a_next[rb] = *(const bf16x8_t*)(src + a_koff0 + rb * 32 * 128);
                    }
#pragma unroll
                    for (int l = 0; l < 4; l++) {
                        if (kAhead) {
#pragma unroll
                            for (int rb = 0; rb < kFirst; rb++) a[rb] = a_next[rb];
                            if (l < 3) {
#pragma unroll
                                for (int rb = 0; rb < kFirst; rb++) a_next[rb] = *(const bf16x8_t*)(src + (a_koff0 ^ (16 * (l + 1))) + rb * 32 * 128);
                            }
                        } else {
#pragma unroll
                            for (int rb = 0; rb < kFirst; rb++) a[rb] = *(const bf16x8_t*)(src + (a_koff0 ^ (16 * l)) + rb * 32 * 128);
                        }
                        u32x4_t w;
                        w[0] = __builtin_amdgcn_perm(hi, lo, e[l & 1].x) ^ f[l & 1].x;
                        w[1] = __builtin_amdgcn_perm(hi, lo, e[l & 1].y) ^ f[l & 1].y;
                        w[2] = __builtin_amdgcn_perm(hi, lo, e[l & 1].z) ^ f[l & 1].z;
                        w[3] = __builtin_amdgcn_perm(hi, lo, e[l & 1].w) ^ f[l & 1].w;
                        // the slot is free: the group two ahead, which from group 2 on belongs to the next step's run
                        if (l == 2) take_run(q[(S + 1) & 3]);
                        ask(l & 1, (l + 2) & 3);
                        const bf16x8_t b = __builtin_bit_cast(bf16x8_t, w);
#pragma unroll
                        for (int rb = 0; rb < kFirst; rb++) acc[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, a[rb], acc[rb], 0, 0, 0);
                        if (LIVE == 4) {
                            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                            for (int rb = 0; rb < 2; rb++) a[rb] = *(const bf16x8_t*)(src + (a_koff0 ^ (16 * l)) + (rb + 2) * 32 * 128);
#pragma unroll
                            for (int rb = 0; rb < 2; rb++) acc[rb + 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, a[rb], acc[rb + 2], 0, 0, 0);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                };
                step(std::integral_constant<int, 0>{});
                step(std::integral_constant<int, 1>{});
                step(std::integral_constant<int, 2>{});
                step(std::integral_constant<int, 3>{});
            }
            asm volatile("" ::"v"(e[0].x), "v"(f[0].x), "v"(e[1].x), "v"(f[1].x));  // (the table reads past the last step)
            // every request has landed (the ones past the last step repeat it); every wave is done with the ring
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(q[0]), "+v"(q[1]), "+v"(q[2]), "+v"(q[3]), "+v"(d_next) : : "memory");
            lds_barrier();
            // ---- LoRA term and store.  A lane holds four consecutive columns of one row: acc[rb][i] is tile row
            // 32 rb + lane_c, column 32 wave + 8 (i / 4) + 4 h + (i % 4): a row block goes out as 64-byte row pieces.
            const int64_t ldc = p.ldc;
            bf16_t* const cbase = (bf16_t*)(seg ? p.c[1] : p.c[0]);
            const int rows_valid = c.rows_valid;
            const int col_quad = col0 + 32 * wave + 4 * lane_h;  // first column of this lane's quad at i / 4 = 0
            const bool vec = ((ldc & 7) == 0) && ((((uintptr_t)cbase) & 15) == 0) && col0 + kTN <= out_cols;
            const int nl = p.r_pad >> 4;  // LoRA sub-steps (0: no LoRA)
            const float ls = nl > 0 ? p.lora_scale : 0.0f;
            const bf16_t* const lb_lane = p.lb + c.expert * p.lb_expert_elems + ((int64_t)seg * out_cols + min(col0 + 32 * wave + lane_c, out_cols - 1)) * p.r_pad + lane_h * 8;
            bf16x8_t lb0;  // this lane's row of the LoRA factor B (first 16 of the rank)
            if (nl > 0) lb0 = *(const bf16x8_t*)lb_lane;
            uint8_t* const stage = smem_raw + kOutBase + wave * 2048;
#pragma unroll
            for (int rb = 0; rb < LIVE; rb++) {
                const int row = 32 * rb + lane_c;
                f32x16_t t;  // LB . LA^T for this row block
#pragma unroll
                for (int e = 0; e < 16; e++) t[e] = 0.0f;
                if (nl > 0) {
                    const bf16_t* la = p.la + (int64_t)(c.row_begin + min(row, rows_valid - 1)) * p.r_pad + lane_h * 8;
                    const bf16x8_t la0 = *(const bf16x8_t*)(smem_raw + kLaBase + row * 32 + lane_h * 16);
                    t = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lb0, la0, t, 0, 0, 0);
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
                        *(uint2*)(stage + lane_c * 64 + ((g ^ ((lane_c >> 2) & 3)) * 16) + 8 * lane_h) = make_uint2(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]));
                    }
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        const int r = 16 * i + (lane >> 2), ch = (lane & 3) ^ ((r >> 2) & 3);
                        const uint4 v = *(const uint4*)(stage + r * 64 + (lane & 3) * 16);
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
                __builtin_amdgcn_sched_barrier(0);
            }
            // the stores count among the outstanding vector memory operations: gone before the next tile's requests are
            // counted; and every wave is done with its staging block before the next tile's requests land in the ring
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (ct + 1 < ct1) lds_barrier();
        }
    }

    // Work assignment: a unit is a run of up to col_tiles_per_wg column tiles of one row tile; the units of a row tile
    // (which share its A rows) follow one another on one XCD.
    static __device__ __forceinline__ void run(const MmqParams& p) {
        const int col_tiles = p.nseg * p.col_tiles_per_seg;
        const int chunks = (col_tiles + p.col_tiles_per_wg - 1) / p.col_tiles_per_wg;
        const int row_tiles = p.tiles ? min(*p.num_tiles, p.max_row_tiles) : p.max_row_tiles;
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
        // the decoder's tables: the kernel's one static LDS array, so it sits at LDS address 0 and the lookups need no base
        __shared__ __attribute__((aligned(16))) uint32_t table_words[Fmt<kIQ2_XXS>::kTableWords];
        switch ((c.rows_valid + 31) >> 5) {
            case 1: work<1>(p, c, ct0, ct1, table_words); break;
            case 2: work<2>(p, c, ct0, ct1, table_words); break;
            case 3: work<3>(p, c, ct0, ct1, table_words); break;
            default: work<4>(p, c, ct0, ct1, table_words); break;
        }
    }
};

__global__ __launch_bounds__(SmallIq2::kThreadsWG) __attribute__((amdgpu_waves_per_eu(4, 4))) void mmq_small_iq2xxs_kernel(const MmqParams p) {
    SmallIq2::run(p);
}

}  // namespace ggq
