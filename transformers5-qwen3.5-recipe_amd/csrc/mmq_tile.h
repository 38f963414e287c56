// Tile kernel for matmuls against packed GGUF weights on gfx950 (MI355X, 64-wide waves, bf16 MFMA).
//
//   NT ("forward")    C[m, n] = sum_k A[m, k] * W[n, k]      A = activations [M, K]
//   NN ("grad input") C[m, k] = sum_n A[m, n] * W[n, k]      A = output cotangents [M, N]
//
// with W [N, K] stored as packed blocks, optionally two weight segments ("pair": gate and up), optional
// expert groups (row ranges of A/C that use different experts' W), and an optional rank-r LoRA term
// s * LA[m, :] . LB[col, :] folded in as extra contraction steps ahead of the main loop.
//
// One workgroup = 512 lanes (8 waves) computes a 256 x 128 tile of C: tall, because every decoded
// weight is reused by all rows of the tile and an expert's rows (about 128 on average in the MoE
// shapes this is built for) should fit one tile.  The waves are specialised; per contraction step of 64
//   * producer waves 4..7 move the A tile (up to 256 x 64 bf16) global -> registers -> LDS with 128-bit
//     accesses (32-row slabs past the end of the group are skipped), and each producer lane loads the
//     packed bytes of one 32-element run of one W row, unpacks scales/mins/codebook in registers
//     (blocks.h) and writes bf16 into the LDS W tile laid out [output column][contraction]; in NN mode
//     that write is the transposition (2-byte stores, the 64 lanes of a wave = 64 consecutive
//     contraction rows).  Global loads run one step ahead of the LDS fill;
//   * consumer waves 0..3 (2 x 2) each own four 32-row blocks (interleaved: block 2*i + wave_m, so
//     short groups load both wave rows evenly) x two 32-column blocks of MFMA 32x32x16 accumulators
//     and run the MFMAs of the previous step out of the other LDS buffer; the whole consumer path is
//     instantiated per number of live row blocks, so ragged groups issue no MFMA on empty blocks.
// One barrier per step hands the buffers over; decode VALU work and MFMA work overlap on every SIMD.
#pragma once
#include "blocks.h"
#include "iq2xxs_grid.h"
#include "mmq_host.h"

#include <type_traits>

namespace ggq {

static __device__ const uint64_t d_iq2xxs_grid_mm[256] = GGQ_IQ2XXS_GRID_INIT;

constexpr int kRowBlocks = kBM / 64;  // 32-row MFMA blocks per consumer wave (4)
constexpr int kColBlocks = kBN / 64;  // 32-column MFMA blocks per consumer wave (2)
constexpr int kASlabs = kBM / 32;     // A-tile load slabs of 32 rows (one uint4 per producer lane each)
constexpr int kATile = kBM * kLdsStride, kBTile = kBN * kLdsStride;  // bf16 elements per LDS buffer
constexpr int kLoadDepth = 3;         // steps of global loads a producer lane keeps in flight

__device__ __forceinline__ uint4 zero4() { return make_uint4(0, 0, 0, 0); }

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains every outstanding
// global load (s_waitcnt vmcnt(0)), which would serialise the producers' register-ring prefetch behind
// each step; here only LDS operations are waited for, and the compiler still places its own vmcnt
// waits in front of the first use of a loaded register.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// 8 consecutive bf16 from a row, zero-filled past `valid` elements (element-wise path for rows that
// are not 16-byte aligned or that end inside the run).
__device__ __forceinline__ uint4 load8_slow(const bf16_t* p, int valid) {
    uint4 v = zero4();
    if (valid <= 0) return v;
    uint32_t e[8];
#pragma unroll
    for (int i = 0; i < 8; i++) e[i] = i < valid ? (uint32_t)p[i] : 0u;
    v.x = e[0] | (e[1] << 16), v.y = e[2] | (e[3] << 16), v.z = e[4] | (e[5] << 16), v.w = e[6] | (e[7] << 16);
    return v;
}

struct TileCtx {  // wave-uniform description of the tile this workgroup computes
    int row_begin, rows_valid, col0, col_tile, seg_c, out_cols, contraction, total_steps, base;
    int64_t expert;
    bf16_t* as;  // [2][kATile]
    bf16_t* bs;  // [2][kBTile]
    const uint2* grid;
};

// ---- producer waves: global -> registers one step ahead, registers -> LDS (with decode) per step.
#define GGQ_FOR_SLABS(X) X(0) X(1) X(2) X(3) X(4) X(5) X(6) X(7)
static_assert(kASlabs == 8, "GGQ_FOR_SLABS enumerates eight A slabs");
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));  // native vector: loads/stores stay typed
struct ARegs {  // 16 bytes per 32-row slab of the A tile, held in registers between load and LDS store
    u32x4_t r0, r1, r2, r3, r4, r5, r6, r7;
};

struct ProducerLane {  // per-lane constants of a producer
    int ptid, pw, lane, a_row, a_ch, a_slabs, last_row, w_ksub_nn, w_row_nt;
    bool a_fast;
};

template <int QT, int MODE>
__device__ __forceinline__ void producer_issue_loads(const MmqParams& p, const TileCtx& c, const ProducerLane& l, int step,
                                                     ARegs& a_reg, typename Fmt<QT>::Raw& w_reg) {
    const int seg_k = MODE == kModeNN ? step / p.steps_per_seg : 0;
    const int kc0 = (step - seg_k * p.steps_per_seg) * kBK;
    if (l.a_fast) {
        // rows past the end of the group are clamped to its last row: they only feed output rows that
        // are never stored (and the repeated row stays in cache)
        const bf16_t* abase = p.a[MODE == kModeNN ? seg_k : 0] + kc0 + l.a_ch * 8;
#define GGQ_LOAD_SLAB(i) a_reg.r##i = *(const u32x4_t*)(abase + (int64_t)(c.row_begin + min(32 * i + l.a_row, l.last_row)) * p.lda);
        GGQ_FOR_SLABS(GGQ_LOAD_SLAB)
#undef GGQ_LOAD_SLAB
    }
    const int wrow = MODE == kModeNT ? l.w_row_nt : min(kc0 + l.lane, p.n - 1);
    const int ksub = MODE == kModeNT ? 2 * step + (l.ptid & 1) : l.w_ksub_nn;
    const int seg = MODE == kModeNT ? c.seg_c : seg_k;
    Fmt<QT>::load(w_reg, p.w[seg] + c.expert * p.w_expert_bytes + (int64_t)wrow * p.w_row_bytes, ksub);
}

template <int QT, int MODE>
__device__ __forceinline__ void producer_fill(const MmqParams& p, const TileCtx& c, const ProducerLane& l, int step, int buf,
                                              const ARegs& a_reg, const typename Fmt<QT>::Raw& w_reg) {
    bf16_t* at = c.as + buf * kATile;
    bf16_t* bt = c.bs + buf * kBTile;
    if (l.a_fast) {
#define GGQ_STORE_SLAB(i) if (i < l.a_slabs) *(u32x4_t*)&at[(32 * i + l.a_row) * kLdsStride + l.a_ch * 8] = a_reg.r##i;
        GGQ_FOR_SLABS(GGQ_STORE_SLAB)
#undef GGQ_STORE_SLAB
    } else {
        // unaligned rows or a contraction that ends inside the step: element-wise, zero-filled
        const int seg_k = MODE == kModeNN ? step / p.steps_per_seg : 0;
        const int kc0 = (step - seg_k * p.steps_per_seg) * kBK;
        const bf16_t* abase = p.a[MODE == kModeNN ? seg_k : 0] + kc0 + l.a_ch * 8;
        const int a_valid = c.contraction - (kc0 + l.a_ch * 8);
        for (int i = 0; i < l.a_slabs; i++)
            *(uint4*)&at[(32 * i + l.a_row) * kLdsStride + l.a_ch * 8] =
                load8_slow(abase + (int64_t)(c.row_begin + min(32 * i + l.a_row, l.last_row)) * p.lda, a_valid);
    }
    uint32_t wv[16];
    Fmt<QT>::decode(w_reg, MODE == kModeNT ? 2 * step + (l.ptid & 1) : l.w_ksub_nn, wv, c.grid);
    if (MODE == kModeNT) {
        bf16_t* dst = &bt[(l.ptid >> 1) * kLdsStride + (l.ptid & 1) * 32];
#pragma unroll
        for (int i = 0; i < 4; i++) *(uint4*)(dst + 8 * i) = make_uint4(wv[4 * i], wv[4 * i + 1], wv[4 * i + 2], wv[4 * i + 3]);
    } else {
        // transpose: element e of this lane's row n is output column 32*pw + e, contraction index lane
#pragma unroll
        for (int e2 = 0; e2 < 16; e2++) {
            bt[(l.pw * 32 + 2 * e2) * kLdsStride + l.lane] = (bf16_t)(wv[e2] & 0xFFFFu);
            bt[(l.pw * 32 + 2 * e2 + 1) * kLdsStride + l.lane] = (bf16_t)(wv[e2] >> 16);
        }
    }
}

template <int QT, int MODE>
__device__ __forceinline__ void produce(const MmqParams& p, const TileCtx& c, int ptid, int pw) {
    ProducerLane l;
    l.ptid = ptid, l.pw = pw, l.lane = ptid & 63;
    // fast A path: every run of 8 is 16-byte aligned and every step is entirely inside the contraction
    l.a_fast = ((p.lda & 7) == 0) && ((c.contraction & 63) == 0) &&
               ((((uintptr_t)p.a[0]) | ((uintptr_t)p.a[MODE == kModeNN && p.nseg > 1 ? 1 : 0])) & 15) == 0;
    l.a_slabs = (c.rows_valid + 31) >> 5;     // 32-row slabs of the A tile that hold a valid row
    l.a_row = ptid >> 3, l.a_ch = ptid & 7;   // lane's (row within a 32-row slab, 16-byte chunk)
    l.last_row = c.rows_valid - 1;
    // W run owned by this lane: NT -> (output column n = col0 + ptid/2, run 2*step + ptid%2);
    //                           NN -> (contraction row n = kc0 + lane, run col0/32 + producer wave).
    // Rows / runs past the end are clamped to the last valid one: what they produce is either never
    // stored (output columns) or multiplied by the zero-filled tail of the A tile (contraction rows).
    l.w_ksub_nn = min((c.col0 >> 5) + pw, (p.k >> 5) - 1);
    l.w_row_nt = min(c.col0 + (ptid >> 1), p.n - 1);
    // Register ring: global loads run kLoadDepth steps ahead of the LDS fill, which itself runs one
    // step ahead of the MFMAs.  Memory latency is several MFMA phases long at these tile sizes.
    ARegs a_ring[kLoadDepth];
    typename Fmt<QT>::Raw w_ring[kLoadDepth];
#pragma unroll
    for (int j = 0; j < kLoadDepth; j++)
        if (j < c.total_steps) producer_issue_loads<QT, MODE>(p, c, l, j, a_ring[j], w_ring[j]);

    // phase for main step s (ring slot J = s % kLoadDepth): fill it into buffer (s + base) & 1, reuse the
    // slot for step s + kLoadDepth, then meet the consumers at the barrier.  s == total_steps is the
    // drain phase (barrier only).
    auto phase = [&](auto slot_c, int s) __attribute__((always_inline)) {
        constexpr int J = decltype(slot_c)::value;
        if (s < c.total_steps) {
            producer_fill<QT, MODE>(p, c, l, s, (s + c.base) & 1, a_ring[J], w_ring[J]);
            if (s + kLoadDepth < c.total_steps) producer_issue_loads<QT, MODE>(p, c, l, s + kLoadDepth, a_ring[J], w_ring[J]);
        }
        lds_barrier();
    };
    // without a LoRA phase the consumers' first phase already needs step 0: fill it before their first
    // barrier; with one, step 0 is filled while they run the LoRA sub-steps
    const int s_first = 1 - c.base;
    if (c.base == 0) phase(std::integral_constant<int, 0>{}, 0);
    static_assert(kLoadDepth == 3, "the phase loop below is unrolled for a ring of three");
    for (int s3 = 0; s3 <= c.total_steps; s3 += 3) {
        if (s3 >= s_first && s3 <= c.total_steps) phase(std::integral_constant<int, 0>{}, s3);
        if (s3 + 1 >= s_first && s3 + 1 <= c.total_steps) phase(std::integral_constant<int, 1>{}, s3 + 1);
        if (s3 + 2 >= s_first && s3 + 2 <= c.total_steps) phase(std::integral_constant<int, 2>{}, s3 + 2);
    }
}

// ---- consumer waves, instantiated per number of live 32-row blocks.
template <int QT, int MODE, int EPI, int LIVE>
__device__ __forceinline__ void consume(const MmqParams& p, const TileCtx& c, int lane, int wave_m, int wave_n) {
    const int lane_c = lane & 31, lane_h = lane >> 5;
    f32x16_t acc[LIVE][kColBlocks];
#pragma unroll
    for (int i = 0; i < LIVE; i++)
#pragma unroll
        for (int j = 0; j < kColBlocks; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;
    const int a_off = (32 * wave_m + lane_c) * kLdsStride + lane_h * 8;
    const int b_off = (wave_n * 64 + lane_c) * kLdsStride + lane_h * 8;

    // Operands of one sub-step (16 of the contraction): LIVE row-block runs of A, two column-block runs of W.
    struct Operands {
        bf16x8_t a[LIVE], b[kColBlocks];
    };
    auto load_operands = [&](Operands& o, int buf, int kk) __attribute__((always_inline)) {
        const bf16_t* a_lds = c.as + buf * kATile + a_off + kk * 16;
        const bf16_t* b_lds = c.bs + buf * kBTile + b_off + kk * 16;
#pragma unroll
        for (int cb = 0; cb < kColBlocks; cb++) o.b[cb] = *(const bf16x8_t*)(b_lds + cb * 32 * kLdsStride);
#pragma unroll
        for (int rb = 0; rb < LIVE; rb++) o.a[rb] = *(const bf16x8_t*)(a_lds + rb * 64 * kLdsStride);
    };
    auto mfma_operands = [&](const Operands& o) __attribute__((always_inline)) {
#pragma unroll
        for (int rb = 0; rb < LIVE; rb++)
#pragma unroll
            for (int cb = 0; cb < kColBlocks; cb++)
                acc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.a[rb], o.b[cb], acc[rb][cb], 0, 0, 0);
    };

    if (c.base == 0) lds_barrier();
    int t = 0;
    if (c.base == 1) {  // LoRA tiles sit in buffer 0: acc = s * LA . LB^T, r_pad / 16 sub-steps
        const int n = p.r_pad >> 4;
#pragma unroll
        for (int kk = 0; kk < 4; kk++)
            if (kk < n) {
                Operands o;
                load_operands(o, 0, kk);
                mfma_operands(o);
            }
        const float s = p.lora_scale;
#pragma unroll
        for (int i = 0; i < LIVE; i++)
#pragma unroll
            for (int j = 0; j < kColBlocks; j++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][j][e] *= s;
        lds_barrier();
        t = 1;
    }
    // Main steps, software pipelined inside the wave: the operands of sub-step k+1 are read from LDS
    // while the MFMAs of sub-step k run, and the barrier that releases the buffer sits between the last
    // LDS read of a step and its last MFMAs, so the first read of the next step hides behind them.
    // Main step t - base lives in buffer t & 1.
    const int phases = c.total_steps + c.base;
    if (t < phases) {
        Operands x, y;
        load_operands(x, t & 1, 0);
        for (; t < phases; t++) {
            const int buf = t & 1;
            load_operands(y, buf, 1);
            mfma_operands(x);
            __builtin_amdgcn_sched_barrier(0);
            load_operands(x, buf, 2);
            mfma_operands(y);
            __builtin_amdgcn_sched_barrier(0);
            load_operands(y, buf, 3);
            mfma_operands(x);
            __builtin_amdgcn_sched_barrier(0);
            lds_barrier();  // every LDS read of this step has landed; the producers may refill the buffer
            if (t + 1 < phases) load_operands(x, buf ^ 1, 0);
            mfma_operands(y);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- epilogue.  acc[rb][cb][i]: tile row = 32*(2*rb + wave_m) + 8*(i/4) + 4*lane_h + (i%4),
    //                                 tile col = 64*wave_n + 32*cb + lane_c
    const int col_base = c.col0 + wave_n * 64 + lane_c;
    if (EPI == kEpiStore || EPI == kEpiAccumF32 || EPI == kEpiCeGrad) {
#pragma unroll
        for (int rb = 0; rb < LIVE; rb++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int r = 32 * (2 * rb + wave_m) + (i >> 2) * 8 + lane_h * 4 + (i & 3);
                if (r >= c.rows_valid) continue;
                const int64_t grow = c.row_begin + r;
                float lse = 0.f, rs = 0.f;
                int64_t label = -1;
                if (EPI == kEpiCeGrad) {
                    lse = p.lse[grow];
                    rs = p.row_scale[grow];
                    label = p.labels[grow];
                }
#pragma unroll
                for (int cb = 0; cb < kColBlocks; cb++) {
                    const int col = col_base + cb * 32;
                    if (col >= c.out_cols) continue;
                    const float v = acc[rb][cb][i];
                    if (EPI == kEpiStore) {
                        ((bf16_t*)p.c[c.seg_c])[grow * p.ldc + col] = to_bf16(v);
                    } else if (EPI == kEpiAccumF32) {
                        ((float*)p.c[0])[grow * p.ldc + col] += v;
                    } else {
                        const float logit = bf16_to_f32(to_bf16(v));  // the path's logits are bf16 values
                        float g = __expf(logit - lse);
                        if ((int64_t)(col + p.ce_col_offset) == label) g -= 1.0f;
                        ((bf16_t*)p.c[0])[grow * p.ldc + col] = to_bf16(g * rs);
                    }
                }
            }
        }
    } else {  // kEpiCeStats
#pragma unroll
        for (int rb = 0; rb < LIVE; rb++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int r = 32 * (2 * rb + wave_m) + (i >> 2) * 8 + lane_h * 4 + (i & 3);
                const bool row_ok = r < c.rows_valid;
                const int64_t grow = c.row_begin + (row_ok ? r : 0);
                const int64_t label = row_ok ? p.labels[grow] : -1;
                float v[kColBlocks];
                float mx = -INFINITY;
#pragma unroll
                for (int cb = 0; cb < kColBlocks; cb++) {
                    const int col = col_base + cb * 32;
                    v[cb] = col < c.out_cols ? bf16_to_f32(to_bf16(acc[rb][cb][i])) : -INFINITY;
                    mx = fmaxf(mx, v[cb]);
                    if (row_ok && col < c.out_cols && (int64_t)(col + p.ce_col_offset) == label) p.ce_target_logit[grow] = v[cb];
                }
                // reduce over the 32 lanes that share this row (lanes with equal lane_h)
#pragma unroll
                for (int off = 16; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
                float sum = 0.f;
#pragma unroll
                for (int cb = 0; cb < kColBlocks; cb++) sum += v[cb] == -INFINITY ? 0.f : __expf(v[cb] - mx);
#pragma unroll
                for (int off = 16; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, 64);
                if (row_ok && lane_c == 0)
                    p.ce_partials[grow * p.ce_partials_ld + p.ce_partial_offset + c.col_tile * 2 + wave_n] = make_float2(mx, sum);
            }
        }
    }
}

// A consumer wave without a live row block only keeps the barriers company.
__device__ __forceinline__ void consume_idle(const TileCtx& c) {
    if (c.base == 0) lds_barrier();
    for (int t = 0; t < c.total_steps + c.base; t++) lds_barrier();
}

template <int QT, int MODE, int EPI>
__global__ __launch_bounds__(kThreads, 1) __attribute__((amdgpu_waves_per_eu(2, 2))) void mmq_tile_kernel(const MmqParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
    TileCtx c;
    c.as = (bf16_t*)smem_raw;
    c.bs = c.as + 2 * kATile;
    uint2* grid_lds = (uint2*)(c.bs + 2 * kBTile);  // [256], IQ2_XXS only
    c.grid = grid_lds;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps control flow scalar
    const int cw = wave & 3;  // index inside the consumer / producer quartet

    // ---- tile assignment.  Hardware deals consecutive workgroup ids round-robin over the 8 XCDs; remap
    // so that consecutive logical tiles (which share an A tile) land on one XCD and hit its L2.
    const int col_tiles = (MODE == kModeNT ? p.nseg : 1) * p.col_tiles_per_seg;
    const int per_xcd = (int)(gridDim.x >> 3);  // the launcher pads the grid to a multiple of 8
    const int logical = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    const int row_tile = logical / col_tiles;
    c.col_tile = logical - row_tile * col_tiles;
    int group = 0, row_end;
    if (p.tiles) {
        if (row_tile >= p.max_row_tiles || row_tile >= *p.num_tiles) return;
        const TileDesc t = p.tiles[row_tile];
        group = t.group, c.row_begin = t.row_begin, row_end = t.row_end;
    } else {
        if (row_tile >= p.max_row_tiles) return;
        c.row_begin = row_tile * kBM;
        row_end = min(p.m, c.row_begin + kBM);
    }
    c.rows_valid = row_end - c.row_begin;  // 1..kBM
    c.expert = p.expert_ids ? p.expert_ids[group] : 0;
    // column tile -> (segment, first output column inside the segment)
    c.seg_c = MODE == kModeNT ? c.col_tile / p.col_tiles_per_seg : 0;
    c.col0 = (c.col_tile - c.seg_c * p.col_tiles_per_seg) * kBN;
    c.out_cols = MODE == kModeNT ? p.n : p.k;     // output columns per segment
    c.contraction = MODE == kModeNT ? p.k : p.n;  // contraction length per segment
    c.total_steps = (MODE == kModeNN ? p.nseg : 1) * p.steps_per_seg;
    c.base = p.r_pad > 0 ? 1 : 0;

    if (QT == kIQ2_XXS && tid < 256) {
        const uint64_t g = d_iq2xxs_grid_mm[tid];
        grid_lds[tid] = make_uint2((uint32_t)g, (uint32_t)(g >> 32));
    }
    // ---- LoRA tiles go to buffer 0 (all lanes load): LA[rows, :r] and LB[cols, :r]
    if (p.r_pad > 0) {
        const int chunks = p.r_pad >> 3;  // 16-byte chunks per row (r_pad % 16 == 0)
        for (int id = tid; id < kBM * 8; id += kThreads) {
            const int r = id >> 3, ch = id & 7;
            uint4 v = zero4();
            if (r < c.rows_valid && ch < chunks) v = *(const uint4*)(p.la + (int64_t)(c.row_begin + r) * p.r_pad + ch * 8);
            *(uint4*)&c.as[r * kLdsStride + ch * 8] = v;
        }
        const bf16_t* lb = p.lb + c.expert * p.lb_expert_elems + (int64_t)(c.seg_c * c.out_cols + c.col0) * p.r_pad;
        for (int id = tid; id < kBN * 8; id += kThreads) {
            const int cidx = id >> 3, ch = id & 7;
            uint4 v = zero4();
            if (c.col0 + cidx < c.out_cols && ch < chunks) v = *(const uint4*)(lb + (int64_t)cidx * p.r_pad + ch * 8);
            *(uint4*)&c.bs[cidx * kLdsStride + ch * 8] = v;
        }
    }
    __syncthreads();  // LoRA tiles and the codebook are visible

    if (wave >= 4) {
        produce<QT, MODE>(p, c, tid & 255, cw);
    } else {
        const int wave_m = cw >> 1, wave_n = cw & 1;
        // this wave's row block i covers tile rows 32*(2*i + wave_m) .. +31; blocks fill up from row 0
        const int live = c.rows_valid > 32 * wave_m ? min(kRowBlocks, (c.rows_valid - 32 * wave_m + 63) >> 6) : 0;
        switch (live) {
            case 0: consume_idle(c); break;
            case 1: consume<QT, MODE, EPI, 1>(p, c, lane, wave_m, wave_n); break;
            case 2: consume<QT, MODE, EPI, 2>(p, c, lane, wave_m, wave_n); break;
            case 3: consume<QT, MODE, EPI, 3>(p, c, lane, wave_m, wave_n); break;
            default: consume<QT, MODE, EPI, 4>(p, c, lane, wave_m, wave_n); break;
        }
    }
}

}  // namespace ggq
