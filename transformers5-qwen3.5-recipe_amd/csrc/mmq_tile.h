// Tile kernel for matmuls against packed GGUF weights on gfx950 (MI355X, 64-wide waves, bf16 MFMA).
//
//   NT ("forward")    C[m, n] = sum_k A[m, k] * W[n, k]      A = activations [M, K]
//   NN ("grad input") C[m, k] = sum_n A[m, n] * W[n, k]      A = output cotangents [M, N]
//
// with W [N, K] stored as packed blocks, optionally two weight segments ("pair": gate and up), optional
// expert groups (row ranges of A/C that use different experts' W), and an optional rank-r LoRA term
// s * LA[m, :] . LB[col, :] folded in as extra contraction steps ahead of the main loop.
//
// One workgroup = 1024 lanes (16 waves, four per SIMD, 128 VGPRs each) computes a 256 x 128 tile of C:
// tall, because every decoded weight is reused by all rows of the tile and an expert's rows (about 128
// on average in the MoE shapes this is built for) should fit one tile.  The waves are specialised; per
// contraction step of 64
//   * consumer waves 0..7 (4 x 2) each own two 32-row blocks (blocks wave_m and wave_m + 4, so short
//     groups still spread over all eight waves) x two 32-column blocks of MFMA 32x32x16 accumulators.
//     Two MFMA-issuing waves share each SIMD: whenever one waits (LDS read cadence, memory queue,
//     barrier skew) the other keeps the matrix pipe busy.  The consumer path is instantiated per number
//     of live row blocks, so ragged groups issue no MFMA on empty blocks.  Consumers also move the A
//     tile: global -> LDS directly (no registers), 1 KB = 8 rows x 128 bytes per wave instruction, two
//     steps ahead of the MFMAs through a ring of three LDS stages; 8-row groups past the end of the
//     expert group are skipped.  A rows sit unpadded in LDS with their 16-byte slots XOR-swizzled so
//     that both the 1 KB writes and the MFMA operand reads are bank-conflict free;
//   * producer waves 8..15 own the weights, as two quartets that take alternate steps: a quartet
//     decodes its step into registers during one phase (packed bytes global -> registers, scales / mins
//     / codebook unpacked in registers, blocks.h) and stores the bf16 W tile, laid out [output
//     column][contraction] for forward, during the next, while the other quartet decodes; for grad-input
//     the tile is stored as decoded, [contraction row][output column], and the consumers transpose it
//     on the way out of LDS (ds_read_b64_tr_b16).  For Q4_K forward a lane loads its share of a 256-wide block once and keeps it
//     for the block's steps, so every cache line of the packed row is requested in one burst.
// One barrier per step hands the buffers over; decode VALU work and MFMA work overlap on every SIMD.
#pragma once
#include "blocks.h"
#include "iq2xxs_grid.h"
#include "mmq_host.h"

#include <type_traits>

namespace ggq {

static __device__ const uint64_t d_iq2xxs_grid_mm[256] = GGQ_IQ2XXS_GRID_INIT;

constexpr int kColBlocks = 2;                   // 32-column MFMA blocks per consumer wave
constexpr int kARowBytes = kBK * 2;             // A rows are unpadded: 128 bytes = eight 16-byte slots

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef short v4i16_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4i16_t* lds_v4i16_ptr;  // native vector: loads/stores stay typed

__device__ __forceinline__ uint4 zero4() { return make_uint4(0, 0, 0, 0); }

// A 16-byte global load that the compiler does not see as a load.  Its own wait-count pass drains every
// outstanding load in front of a register set that was requested before a loop back-edge or a join, which
// puts a full memory round trip into each step of a two-steps-ahead prefetch.  With this form the caller
// waits itself (wait_loads_at_most, loads return in issue order) and fences the registers
// (asm volatile "+v") between that wait and their first use; nothing may touch them before.
__device__ __forceinline__ void load16_untracked(u32x4_t& dst, const void* ptr) {
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(ptr) : "memory");
}
__device__ __forceinline__ uint4 as_uint4(const u32x4_t& v) { return make_uint4(v.x, v.y, v.z, v.w); }

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

// All-reduce over each half of a wave (lanes 0..31, 32..63): four data-parallel-primitive steps inside the rows of 16
// lanes (neighbour, pair of a quad, mirror of 8, mirror of 16: every lane of a row ends with the row's result) and one
// cross-lane exchange between the two rows of a half.  Five exchanges through the LDS crossbar cost several times more.
template <int CTRL>
static __device__ __forceinline__ float dpp_f32(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}
static __device__ __forceinline__ float half_wave_max(float x) {
    x = fmaxf(x, dpp_f32<0xB1>(x));   // quad_perm [1,0,3,2]
    x = fmaxf(x, dpp_f32<0x4E>(x));   // quad_perm [2,3,0,1]
    x = fmaxf(x, dpp_f32<0x141>(x));  // row_half_mirror
    x = fmaxf(x, dpp_f32<0x140>(x));  // row_mirror
    return fmaxf(x, __shfl_xor(x, 16, 64));
}
static __device__ __forceinline__ float half_wave_sum(float x) {
    x += dpp_f32<0xB1>(x);
    x += dpp_f32<0x4E>(x);
    x += dpp_f32<0x141>(x);
    x += dpp_f32<0x140>(x);
    return x + __shfl_xor(x, 16, 64);
}

struct TileCtx {  // wave-uniform description of the tile this workgroup computes
    int row_begin, rows_valid, col0, col_tile, seg_c, out_cols, contraction, total_steps, base;
    int64_t expert;
    uint8_t* as;      // [kAStages][A stage bytes]
    bf16_t* bs;       // [2][W tile elements]
    uint32_t as_lds;  // LDS byte address of `as`
    bool a_fast;      // A rows can be moved with aligned 16-byte accesses and every step is whole
    const uint2* grid;
    const float* row_scale;  // accumulate epilogue: the tile rows' factors, staged in LDS
};

// (segment, first contraction index) of a step; at most two segments.
template <int MODE>
__device__ __forceinline__ void step_origin(const MmqParams& p, int step, int& seg_k, int& kc0) {
    seg_k = (MODE == kModeNN && step >= p.steps_per_seg) ? 1 : 0;
    kc0 = (step - seg_k * p.steps_per_seg) * kBK;
}

// Everything below depends on the tile shape.  SH = 0: 256 x 128 ("tall": dense launches and expert
// groups with many rows); SH = 1: 128 x 256 ("wide": expert groups of about a hundred rows, where two row
// blocks per wave keep the LDS operand traffic at one read per MFMA and one decode of the weights serves
// 256 output columns).  The eight consumer waves form a kWavesM x kWavesN grid; wave (wave_m, wave_n) owns
// row blocks wave_m and wave_m + kWavesM and the 64 columns at 64 * wave_n.
template <int SH>
struct Tile {
static constexpr int kTM = SH == 0 ? 256 : 128, kTN = SH == 0 ? 128 : 256;
static constexpr int kWavesM = kTM / 64, kWavesN = kTN / 64;
static constexpr int kCW = kWavesM * kWavesN;       // consumer waves (8), as many producer waves
static constexpr int kProducerLanes = 64 * kCW;
static constexpr int kThreadsWG = 128 * kCW;
static constexpr int kAStageBytes = kTM * kARowBytes;   // 32 KB / 16 KB
// LDS ring of A tiles: the loads of a step are issued kAStages - 1 steps ahead of its MFMAs.  Memory latency
// under load is about two thousand cycles; the wide shape's short steps need the longer ring.
static constexpr int kAStages = SH == 0 ? 3 : 5;
static constexpr int kAhead = kAStages - 1;
static constexpr int kAGroups = kTM / 8;                // 8-row groups (one direct-to-LDS instruction each)
static constexpr int kGroupsPerWave = kAGroups / kCW;   // groups one consumer wave moves per step (4 / 2)
// W buffer: forward [output column][64 + 8]; grad-input [contraction row][columns + 32], as the rows are
// decoded (the consumers transpose on the way out of LDS).  Sized for the larger of the two.
static constexpr int kNnPitch = kTN + 32;
// Position of 16-byte chunk q of contraction row `row` in the grad-input W tile: the two low bits of q are
// XOR-ed with a row-dependent value so that the lanes of one 16-byte store instruction (which differ in
// row and run, and would otherwise meet four deep on the same banks) hit distinct banks, while the four
// rows of a transposing read keep their 32-byte pieces on distinct banks.
static __device__ __forceinline__ int nn_chunk(int row, int q) {
    const int sw = SH == 0 ? (((row >> 2) & 3) ^ (row & 1)) : ((row & 1) ^ (((q >> 4) & 1) << 1));
    return q ^ sw;
}
static constexpr int kBTile = kTN * kLdsStride > kBK * kNnPitch ? kTN * kLdsStride : kBK * kNnPitch;  // bf16 elements
static constexpr int kTileLdsBytes = kAStages * kAStageBytes + 2 * kBTile * 2;

// ---- A tile, fast path: each of the eight waves of the consumer octet moves the 8-row groups
// g = 8*j + cw (j = 0..3) with one direct-to-LDS instruction per group.
struct ALoader {
    uint32_t voff[kGroupsPerWave];  // byte offset of this lane's 16 bytes inside the tile's rows, per group j
    uint32_t lds0;                  // LDS byte address of stage 0, group cw
    int n;                          // groups this wave moves per step (0 when the fast path is off)
};

static __device__ __forceinline__ void a_loader_init(ALoader& a, const MmqParams& p, const TileCtx& c, int lane, int cw) {
    const int sub = 8 * cw + (lane >> 3);         // row inside a slab of 8 rows per consumer wave
    const int kc = (lane & 7) ^ ((sub >> 1) & 7);  // the chunk that belongs in this lane's LDS slot
#pragma unroll
    for (int j = 0; j < kGroupsPerWave; j++) {
        // rows past the end of the group are clamped to its last row: they only feed output rows that
        // are never stored
        int row = min(8 * kCW * j + sub, c.rows_valid - 1);
        // with a row index the offset carries the whole stored row (the host keeps that matrix under 4 GiB)
        if (p.a_rows.on()) row = c.rows_valid > 0 ? p.a_rows.source(c.row_begin + row) : 0;
        a.voff[j] = ((uint32_t)row * (uint32_t)p.lda + (uint32_t)kc * 8u) * 2u;
    }
    a.lds0 = c.as_lds + cw * 1024;
    const int groups = (c.rows_valid + 7) >> 3;
    a.n = c.a_fast ? max(0, (groups - cw + kCW - 1) / kCW) : 0;
}

template <int MODE, int J0, int J1>
static __device__ __forceinline__ void a_issue(const ALoader& a, const MmqParams& p, const TileCtx& c, int step, int stage) {
    int seg_k, kc0;
    step_origin<MODE>(p, step, seg_k, kc0);
    const bf16_t* sbase = p.a[MODE == kModeNN ? seg_k : 0] + (p.a_rows.on() ? 0 : (int64_t)c.row_begin * p.lda) + kc0;
    const uint32_t lds = a.lds0 + stage * kAStageBytes;
#pragma unroll
    for (int j = J0; j < J1 && j < kGroupsPerWave; j++)
        if (j < a.n)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                         :
                         : "s"(lds + j * (kCW * 1024)), "v"(a.voff[j]), "s"(sbase)
                         : "memory");
}

// Issue schedule shared by all waves of the consumer octet: steps 0 and 1 before the first barrier,
// step t + 2 during main phase t (into the stage the MFMAs of step t - 1 have just released), one
// group per sub-step between the MFMAs.
struct AIssuer {
    ALoader ld;
    int next_step, next_stage;
};
template <int MODE, int J0, int J1>
static __device__ __forceinline__ void a_issue_part(const AIssuer& s, const MmqParams& p, const TileCtx& c) {
    if (s.next_step < c.total_steps) a_issue<MODE, J0, J1>(s.ld, p, c, s.next_step, s.next_stage);
}
static __device__ __forceinline__ void a_issue_advance(AIssuer& s) {
    s.next_step++;
    s.next_stage = s.next_stage == kAStages - 1 ? 0 : s.next_stage + 1;
}
template <int MODE>
static __device__ __forceinline__ void a_issue_next(AIssuer& s, const MmqParams& p, const TileCtx& c) {
    a_issue_part<MODE, 0, kGroupsPerWave>(s, p, c);
    a_issue_advance(s);
}
// Before the barrier that ends the phase of step t - 1 (t = 0: the first barrier): step t has landed
// when only the loads of the steps issued after it may still be in flight.
static __device__ __forceinline__ void a_wait_step(const AIssuer& s, const TileCtx& c, int t) {
    const int younger = max(0, min(s.next_step, c.total_steps) - (t + 1));
    wait_loads_at_most(younger * s.ld.n);
}

// ---- producer waves: packed weights global -> registers -> (decode) -> LDS W tile.
struct ProducerLane {  // per-lane constants of a producer
    int ptid, pw, lane, w_ksub_nn, w_row_nt;
};

// Element-wise A tile for shapes the fast path cannot take (unaligned rows, a contraction that ends
// inside the step): producers write the same swizzled layout, zero-filled past the contraction.
template <int MODE>
static __device__ __forceinline__ void fill_a_slow(const MmqParams& p, const TileCtx& c, const ProducerLane& l, int step, int stage) {
    int seg_k, kc0;
    step_origin<MODE>(p, step, seg_k, kc0);
    uint8_t* at = c.as + stage * kAStageBytes;
    for (int id = l.ptid; id < kTM * 8; id += 256) {
        const int r = id >> 3, ch = id & 7;
        if (r >= c.rows_valid) break;
        const bf16_t* src = p.a[MODE == kModeNN ? seg_k : 0] + (int64_t)p.a_rows.source(c.row_begin + r) * p.lda + kc0 + ch * 8;
        *(uint4*)(at + r * kARowBytes + a_slot(r, ch) * 16) = load8_slow(src, c.contraction - (kc0 + ch * 8));
    }
}

template <int QT, int MODE>
static __device__ __forceinline__ void w_issue_run(const MmqParams& p, const TileCtx& c, const ProducerLane& l, int step,
                                            typename Fmt<QT>::Raw& w_reg) {
    int seg_k, kc0;
    step_origin<MODE>(p, step, seg_k, kc0);
    // Rows / runs past the end are clamped to the last valid one: what they produce is either never
    // stored (output columns) or multiplied by the zero-filled tail of the A tile (contraction rows).
    const int wrow = MODE == kModeNT ? l.w_row_nt : min(kc0 + l.lane, p.n - 1);
    const int ksub = MODE == kModeNT ? 2 * step + (l.ptid & 1) : l.w_ksub_nn;
    const int seg = MODE == kModeNT ? c.seg_c : seg_k;
    Fmt<QT>::load(w_reg, p.w[seg] + c.expert * p.w_expert_bytes + (int64_t)wrow * p.w_row_bytes, ksub);
}

// The 32 decoded weights of a run (16 packed bf16 pairs) -> LDS W tile.
template <int MODE>
static __device__ __forceinline__ void w_store_run(const TileCtx& c, const ProducerLane& l, int buf, const uint32_t* wv) {
    bf16_t* bt = c.bs + buf * kBTile;
    if (MODE == kModeNT) {
        bf16_t* dst = &bt[(l.ptid >> 1) * kLdsStride + (l.ptid & 1) * 32];
#pragma unroll
        for (int i = 0; i < 4; i++) *(uint4*)(dst + 8 * i) = make_uint4(wv[4 * i], wv[4 * i + 1], wv[4 * i + 2], wv[4 * i + 3]);
    } else {
        // grad-input: this lane's contraction row, columns 32*pw .. +31, stored as decoded
        bf16_t* dst = &bt[l.lane * kNnPitch];
#pragma unroll
        for (int i = 0; i < 4; i++) *(uint4*)(dst + 8 * nn_chunk(l.lane, l.pw * 4 + i)) = make_uint4(wv[4 * i], wv[4 * i + 1], wv[4 * i + 2], wv[4 * i + 3]);
    }
}

// Q4_K forward, wide shape: lane (output column n = ptid / 2, half h = ptid % 2) keeps, for a 256-wide
// block, the block header and bytes 16h .. 16h+15 of each of the four 32-byte quant groups.  Group S
// feeds step S of the block: its low nibbles are elements 16h .. 16h+15 of sub-block 2S, its high
// nibbles the same elements of sub-block 2S+1.
struct Q4KChunk {
    u32x4_t hdr, g0, g1, g2, g3;
};
static __device__ __forceinline__ void q4k_chunk_load(Q4KChunk& ch, const uint8_t* row, int block, int h) {
    const uint8_t* blk = row + (int64_t)block * 144;
    ch.hdr = *(const u32x4_t*)blk;
    const uint8_t* q = blk + 16 + 16 * h;
    ch.g0 = *(const u32x4_t*)q;
    ch.g1 = *(const u32x4_t*)(q + 32);
    ch.g2 = *(const u32x4_t*)(q + 64);
    ch.g3 = *(const u32x4_t*)(q + 96);
}
// Keeps every use of the block registers after this point in program order (in particular after the
// barrier in front of it), so that no wait for a freshly issued reload is pulled forward.
static __device__ __forceinline__ void q4k_chunk_pin(Q4KChunk& ch) {
    asm volatile("" : "+v"(ch.hdr), "+v"(ch.g0), "+v"(ch.g1), "+v"(ch.g2), "+v"(ch.g3));
}
template <int J>  // 6-bit (scale, min) of sub-block J
static __device__ __forceinline__ void q4k_scale_min(const u32x4_t& hdr, uint32_t& sc, uint32_t& m) {
    const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
    if (J < 4) {
        sc = (s0 >> (8 * J)) & 63u;
        m = (s1 >> (8 * J)) & 63u;
    } else {
        constexpr int sh = 8 * (J - 4);
        sc = ((s2 >> sh) & 0xFu) | (((s0 >> (sh + 6)) & 3u) << 4);
        m = ((s2 >> (sh + 4)) & 0xFu) | (((s1 >> (sh + 6)) & 3u) << 4);
    }
}
// wv[0..7]: elements 16h .. 16h+15 of sub-block 2S; wv[8..15]: the same elements of sub-block 2S+1.
template <int S>
static __device__ __forceinline__ void q4k_chunk_decode(const u32x4_t& hdr, const u32x4_t& q, uint32_t* wv) {
    const float d = half_bits_to_f32(hdr.x & 0xFFFFu), dmin = half_bits_to_f32(hdr.x >> 16);
    uint32_t sc0, m0, sc1, m1;
    q4k_scale_min<2 * S>(hdr, sc0, m0);
    q4k_scale_min<2 * S + 1>(hdr, sc1, m1);
    const float dl0 = d * (float)sc0 * kMixScale, nm0 = -(dmin * (float)m0);
    const float dl1 = d * (float)sc1 * kMixScale, nm1 = -(dmin * (float)m1);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        // byte b of the word: low nibble = element b of sub-block 2S, high nibble = element b of 2S+1;
        // each nibble lands in its own 16-bit half (bytes 0, 2 / bytes 1, 3) for the mixed-precision fma
        const uint32_t lo02 = q[i] & 0x000F000Fu, hi02 = (q[i] >> 4) & 0x000F000Fu;
        const uint32_t lo13 = (q[i] >> 8) & 0x000F000Fu, hi13 = (q[i] >> 12) & 0x000F000Fu;
        wv[2 * i] = pack_bf16(mix_lo(lo02, dl0, nm0), mix_lo(lo13, dl0, nm0));
        wv[2 * i + 1] = pack_bf16(mix_hi(lo02, dl0, nm0), mix_hi(lo13, dl0, nm0));
        wv[8 + 2 * i] = pack_bf16(mix_lo(hi02, dl1, nm1), mix_lo(hi13, dl1, nm1));
        wv[8 + 2 * i + 1] = pack_bf16(mix_hi(hi02, dl1, nm1), mix_hi(hi13, dl1, nm1));
    }
}
static __device__ __forceinline__ void q4k_chunk_store(const TileCtx& c, const ProducerLane& l, int buf, const uint32_t* wv) {
    bf16_t* dst = c.bs + buf * kBTile + (l.ptid >> 1) * kLdsStride + (l.ptid & 1) * 16;
    *(uint4*)(dst) = make_uint4(wv[0], wv[1], wv[2], wv[3]);
    *(uint4*)(dst + 8) = make_uint4(wv[4], wv[5], wv[6], wv[7]);
    *(uint4*)(dst + 32) = make_uint4(wv[8], wv[9], wv[10], wv[11]);
    *(uint4*)(dst + 40) = make_uint4(wv[12], wv[13], wv[14], wv[15]);
}

// One producer quartet (256 lanes).  Barrier b closes the phase in which step b must reach LDS (A
// stage (b + base) % 3 when the direct path is off, W buffer (b + base) & 1); the MFMAs of step b run
// after it.  Quartet Q takes the steps of parity Q: it decodes step u into registers during phase
// u - 1 (step 0: before the first phase) and stores them during phase u.  steps + 1 barriers in all.
// The phase sequence is written out per period (no data-dependent branches between a load and its
// use), so that the waits on the packed-weight loads stay exact instead of draining every load.
// `after_issue` runs once the first packed-weight loads are on their way: the LoRA tiles are fetched
// there by all waves, and the workgroup meets at the barrier that makes them visible.
template <int QT, int MODE, int Q, class AfterIssue>
static __device__ __forceinline__ void produce(const MmqParams& p, const TileCtx& c, int ptid, int pw, AfterIssue&& after_issue) {
    ProducerLane l;
    l.ptid = ptid;
    // W run owned by this lane: NT -> (output column n = col0 + ptid/2, run 2*step + ptid%2);
    //                           NN -> (contraction row n = kc0 + l.lane, run col0/32 + l.pw): a quartet wave takes
    //                           16 rows, the four lanes of a row the four runs, so that they read adjacent bytes
    //                           of the row's block (a lane-per-row split costs one cache access per lane).
    l.lane = MODE == kModeNN ? 16 * pw + ((ptid & 63) >> 2) : (ptid & 63);
    l.pw = MODE == kModeNN ? (ptid & 3) : pw;
    l.w_ksub_nn = min((c.col0 >> 5) + l.pw, (p.k >> 5) - 1);
    l.w_row_nt = min(c.col0 + (ptid >> 1), p.n - 1);
    const int steps = c.total_steps;
    uint32_t wv[16];
    int stage = c.base, buf = c.base;
    auto close_phase = [&]() __attribute__((always_inline)) {
        lds_barrier();
        stage = stage == kAStages - 1 ? 0 : stage + 1;
        buf ^= 1;
    };
    auto store = [&](int u) __attribute__((always_inline)) {
        if (!c.a_fast) fill_a_slow<MODE>(p, c, l, u, stage);
        w_store_run<MODE>(c, l, buf, wv);
    };
    // Decoded values are fenced the same way: the decode belongs in front of the barrier that follows it.
    auto pin_decoded = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 16; i++) asm volatile("" : "+v"(wv[i]));
    };
    {
        // Two register sets alternate between this quartet's steps (u = Q, Q + 2, ...): the packed run of
        // step u + 4 is requested as soon as step u is decoded, three phases before its own decode.
        typename Fmt<QT>::Raw raw_a, raw_b;
        auto decode = [&](typename Fmt<QT>::Raw& raw, int u) __attribute__((always_inline)) {
            if (u >= steps) return;
            Fmt<QT>::pin(raw);
            Fmt<QT>::decode(raw, MODE == kModeNT ? 2 * u + (l.ptid & 1) : l.w_ksub_nn, wv, c.grid);
            pin_decoded();
            w_issue_run<QT, MODE>(p, c, l, u + 4 < steps ? u + 4 : u, raw);  // unconditional (a load under a branch is drained at the join)
        };
        if (Q < steps) w_issue_run<QT, MODE>(p, c, l, Q, raw_a);
        if (Q + 2 < steps) w_issue_run<QT, MODE>(p, c, l, Q + 2, raw_b);
        after_issue();
        if (Q == 0) {
            decode(raw_a, 0);
            for (int b = 0; b < steps; b += 4) {
                store(b);
                close_phase();
                if (b + 1 < steps) {
                    decode(raw_b, b + 2);
                    close_phase();
                }
                if (b + 2 < steps) {
                    store(b + 2);
                    close_phase();
                }
                if (b + 3 < steps) {
                    decode(raw_a, b + 4);
                    close_phase();
                }
            }
        } else {
            for (int b = 0; b < steps; b += 4) {
                decode(raw_a, b + 1);
                close_phase();
                if (b + 1 < steps) {
                    store(b + 1);
                    close_phase();
                }
                if (b + 2 < steps) {
                    decode(raw_b, b + 3);
                    close_phase();
                }
                if (b + 3 < steps) {
                    store(b + 3);
                    close_phase();
                }
            }
        }
    }
    lds_barrier();
}

// ---- Wide shape, every block format but Q4_K: all 512 producer lanes work on every step, one 32-wide run each
// (forward: lane = (output column ptid / 2, run 2 * step + ptid % 2); grad-input: lane = (contraction row ptid / 8, run
// ptid % 8 of the tile's 256 columns, so that the eight lanes of a row read adjacent bytes)).  A step is decoded and
// stored in its own phase; its register set is reloaded for a later step as soon as it is decoded.
// Expert groups of a few dozen rows give the consumers little to do per step, so the tile's time is the producers' chain
// of load, decode, store and barrier: the wide tile runs that chain once per 256 output columns instead of once per 128.
template <int QT, int MODE, class AfterIssue>
static __device__ __forceinline__ void produce_all(const MmqParams& p, const TileCtx& c, int ptid, AfterIssue&& after_issue) {
    static_assert(SH == 1, "the wide shape's producer");
    ProducerLane l;
    l.ptid = ptid;
    l.lane = MODE == kModeNN ? (ptid >> 3) : (ptid & 63);
    l.pw = MODE == kModeNN ? (ptid & 7) : (ptid >> 6);
    l.w_ksub_nn = min((c.col0 >> 5) + l.pw, (p.k >> 5) - 1);
    l.w_row_nt = min(c.col0 + (ptid >> 1), p.n - 1);
    const int steps = c.total_steps;
    uint32_t wv[16];
    int stage = c.base, buf = c.base;
    // The packed bytes of a step are requested kDepth steps ahead, in as many register sets as the block format's packed run
    // allows (a step cannot take less than the memory latency / kDepth; measured, two sets and eight differ by 2 % at 64
    // rows per group, so the latency is not what paces these tiles).
    constexpr int kRawRegs = (int)(sizeof(typename Fmt<QT>::Raw) / 4);
    constexpr int kDepth = kRawRegs <= 4 ? 8 : kRawRegs <= 12 ? 4 : 2;
    typename Fmt<QT>::Raw raw[kDepth];
#pragma unroll
    for (int i = 0; i < kDepth; i++) w_issue_run<QT, MODE>(p, c, l, min(i, steps - 1), raw[i]);  // unconditional: a load under a branch is drained at the join
    after_issue();
    auto phase = [&](typename Fmt<QT>::Raw& r, int u) __attribute__((always_inline)) {
        if (!c.a_fast && ptid < 256) fill_a_slow<MODE>(p, c, l, u, stage);
        Fmt<QT>::pin(r);
        Fmt<QT>::decode(r, MODE == kModeNT ? 2 * u + (ptid & 1) : l.w_ksub_nn, wv, c.grid);
#pragma unroll
        for (int i = 0; i < 16; i++) asm volatile("" : "+v"(wv[i]));  // the decode stays in front of the reload and the barrier
        w_issue_run<QT, MODE>(p, c, l, min(u + kDepth, steps - 1), r);
        w_store_run<MODE>(c, l, buf, wv);
        lds_barrier();
        stage = stage == kAStages - 1 ? 0 : stage + 1;
        buf ^= 1;
    };
    for (int u = 0; u < steps; u += kDepth) {
#pragma unroll
        for (int i = 0; i < kDepth; i++)
            if (u + i < steps) phase(raw[i], u + i);
    }
    lds_barrier();
}

// ---- Q4_K: both producer quartets (512 lanes) work on every step, half a run each.  The decode of a
// step is the longest thing between two barriers when an expert group has few rows; splitting it over
// all eight producer waves halves it.
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// Forward: lane (output column n = ptid / 4, quarter q = ptid % 4) keeps, for a 256-wide block, the
// block header and bytes 8q .. 8q+7 of each of the four 32-byte quant groups.  Group S feeds step S:
// low nibbles are elements 8q .. 8q+7 of sub-block 2S, high nibbles the same elements of sub-block 2S+1.
struct Q4KQuarter {
    u32x4_t hdr;
    u32x2_t g0, g1, g2, g3;
};
static __device__ __forceinline__ void q4k_quarter_load(Q4KQuarter& ch, const uint8_t* row, int block, int q) {
    const uint8_t* blk = row + (int64_t)block * 144;
    ch.hdr = *(const u32x4_t*)blk;
    const uint8_t* g = blk + 16 + 8 * q;
    ch.g0 = *(const u32x2_t*)g;
    ch.g1 = *(const u32x2_t*)(g + 32);
    ch.g2 = *(const u32x2_t*)(g + 64);
    ch.g3 = *(const u32x2_t*)(g + 96);
}
static __device__ __forceinline__ void q4k_quarter_pin(Q4KQuarter& ch) {
    asm volatile("" : "+v"(ch.hdr), "+v"(ch.g0), "+v"(ch.g1), "+v"(ch.g2), "+v"(ch.g3));
}
// lo[0..3]: elements 8q .. 8q+7 of sub-block 2S; hi[0..3]: the same elements of sub-block 2S+1.
template <int S>
static __device__ __forceinline__ void q4k_quarter_decode(const u32x4_t& hdr, const u32x2_t& g, uint32_t* lo, uint32_t* hi) {
    const float d = half_bits_to_f32(hdr.x & 0xFFFFu), dmin = half_bits_to_f32(hdr.x >> 16);
    uint32_t sc0, m0, sc1, m1;
    q4k_scale_min<2 * S>(hdr, sc0, m0);
    q4k_scale_min<2 * S + 1>(hdr, sc1, m1);
    const float dl0 = d * (float)sc0 * kMixScale, nm0 = -(dmin * (float)m0);
    const float dl1 = d * (float)sc1 * kMixScale, nm1 = -(dmin * (float)m1);
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const uint32_t lo02 = g[i] & 0x000F000Fu, hi02 = (g[i] >> 4) & 0x000F000Fu;
        const uint32_t lo13 = (g[i] >> 8) & 0x000F000Fu, hi13 = (g[i] >> 12) & 0x000F000Fu;
        lo[2 * i] = pack_bf16(mix_lo(lo02, dl0, nm0), mix_lo(lo13, dl0, nm0));
        lo[2 * i + 1] = pack_bf16(mix_hi(lo02, dl0, nm0), mix_hi(lo13, dl0, nm0));
        hi[2 * i] = pack_bf16(mix_lo(hi02, dl1, nm1), mix_lo(hi13, dl1, nm1));
        hi[2 * i + 1] = pack_bf16(mix_hi(hi02, dl1, nm1), mix_hi(hi13, dl1, nm1));
    }
}

// Grad-input, tall shape: a lane decodes 16 consecutive output columns (half a run) of its contraction row.
struct Q4KHalfRun {
    u32x4_t hdr, q;
};
static __device__ __forceinline__ void q4k_half_run_pin(Q4KHalfRun& r) { asm volatile("" : "+v"(r.hdr), "+v"(r.q)); }
static __device__ __forceinline__ void q4k_half_run_decode(const Q4KHalfRun& r, int j, uint32_t* out) {  // j: sub-block 0..7
    const float d = half_bits_to_f32(r.hdr.x & 0xFFFFu), dmin = half_bits_to_f32(r.hdr.x >> 16);
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
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t e02 = (r.q[i] >> shift) & 0x000F000Fu, e13 = (r.q[i] >> (shift + 8)) & 0x000F000Fu;
        out[2 * i] = pack_bf16(mix_lo(e02, dl, nm), mix_lo(e13, dl, nm));
        out[2 * i + 1] = pack_bf16(mix_hi(e02, dl, nm), mix_hi(e13, dl, nm));
    }
}

// Barrier b closes the phase in which step b reaches LDS; steps + 1 barriers in all (the last one
// pairs with the consumers' final step).
template <int MODE, class AfterIssue>
static __device__ __forceinline__ void produce_q4k(const MmqParams& p, const TileCtx& c, int ptid, int pw, AfterIssue&& after_issue) {
    // ptid 0..511 over both quartets; pw 0..7
    const int steps = c.total_steps;
    int stage = c.base, buf = c.base;
    ProducerLane slow;  // the element-wise A path is the first quartet's job
    slow.ptid = ptid, slow.pw = pw, slow.lane = ptid & 63, slow.w_ksub_nn = 0, slow.w_row_nt = 0;
    auto open_phase = [&](int u) __attribute__((always_inline)) {
        if (!c.a_fast && ptid < 256) fill_a_slow<MODE>(p, c, slow, u, stage);
    };
    auto close_phase = [&]() __attribute__((always_inline)) {
        lds_barrier();
        stage = stage == kAStages - 1 ? 0 : stage + 1;
        buf ^= 1;
    };
    if (MODE == kModeNT && SH != 0) {
        // wide / half: lane = (column ptid / 2, half ptid % 2), 32 weights per lane and step
        ProducerLane l = slow;
        const int h = ptid & 1;
        const uint8_t* wrow = p.w[c.seg_c] + c.expert * p.w_expert_bytes + (int64_t)min(c.col0 + (ptid >> 1), p.n - 1) * p.w_row_bytes;
        const int blocks = steps >> 2;  // K is a whole number of 256-wide blocks
        Q4KChunk even, odd;             // alternate between blocks; a set is loaded four phases before its first use
        q4k_chunk_load(even, wrow, 0, h);
        after_issue();
        auto fill = [&](auto s_c, const Q4KChunk& ch, int u) __attribute__((always_inline)) {
            constexpr int S = decltype(s_c)::value;
            open_phase(u);
            uint32_t wv[16];
            q4k_chunk_decode<S>(ch.hdr, S == 0 ? ch.g0 : S == 1 ? ch.g1 : S == 2 ? ch.g2 : ch.g3, wv);
            q4k_chunk_store(c, l, buf, wv);
            close_phase();
        };
        auto block_phases = [&](Q4KChunk& cur, Q4KChunk& nxt, int k) __attribute__((always_inline)) {
            // (unconditional, the last block simply loads itself again: a load under a branch makes the
            // compiler drain every outstanding load at the join, right after this one was issued)
            q4k_chunk_load(nxt, wrow, min(k + 1, blocks - 1), h);
            q4k_chunk_pin(cur);
            fill(std::integral_constant<int, 0>{}, cur, 4 * k);
            q4k_chunk_pin(cur);
            fill(std::integral_constant<int, 1>{}, cur, 4 * k + 1);
            q4k_chunk_pin(cur);
            fill(std::integral_constant<int, 2>{}, cur, 4 * k + 2);
            q4k_chunk_pin(cur);
            fill(std::integral_constant<int, 3>{}, cur, 4 * k + 3);
        };
        for (int k = 0; k < blocks; k += 2) {
            block_phases(even, odd, k);
            if (k + 1 < blocks) block_phases(odd, even, k + 1);
        }
    } else if (MODE == kModeNN && SH != 0) {
        // wide: the 256 output columns of a step are exactly one block of each of the 64 contraction rows;
        // producer wave w takes rows 8w .. 8w+7, lane = (row, run of 32 columns), so that the eight lanes of
        // a row ask for one header and four adjacent 32-byte groups (a lane-per-row split costs the vector
        // cache one access per lane and load).  Stored as decoded: [row][column]; the consumers transpose
        // on the way out of LDS.
        constexpr int kRuns = kTN / 32;                             // lanes per contraction row (8 wide, 4 half)
        const int lane = (64 / kRuns) * pw + (ptid & 63) / kRuns;  // contraction row inside the step
        const int run = ptid % kRuns;
        const int ksub = min((c.col0 >> 5) + run, (p.k >> 5) - 1);  // runs past the end are clamped, never stored
        struct Raw {  // header and the 32-byte quant group of the run: three untracked loads
            u32x4_t hdr, q0, q1;
        };
        const int64_t blk_off = (int64_t)(ksub >> 3) * 144;
        const int q_off = 16 + 32 * ((ksub & 7) >> 1);
        auto issue = [&](Raw& r, int u) __attribute__((always_inline)) {
            int seg_k, kc0;
            step_origin<MODE>(p, u, seg_k, kc0);
            const int wrow = min(kc0 + lane, p.n - 1);  // rows past the end meet the zero-filled tail of the A tile
            const uint8_t* blk = p.w[seg_k] + c.expert * p.w_expert_bytes + (int64_t)wrow * p.w_row_bytes + blk_off;
            load16_untracked(r.hdr, blk);
            load16_untracked(r.q0, blk + q_off);
            load16_untracked(r.q1, blk + q_off + 16);
        };
        bf16_t* const dst0 = c.bs + lane * kNnPitch;
        auto fill = [&](Raw& r, int u) __attribute__((always_inline)) {
            open_phase(u);
            wait_loads_at_most(3);  // the other set's three loads may still be on their way
            asm volatile("" : "+v"(r.hdr), "+v"(r.q0), "+v"(r.q1));
            typename Fmt<kQ4_K>::Raw rr;
            rr.hdr = as_uint4(r.hdr), rr.q0 = as_uint4(r.q0), rr.q1 = as_uint4(r.q1);
            uint32_t wv[16];
            Fmt<kQ4_K>::decode(rr, ksub, wv, nullptr);
            issue(r, min(u + 2, steps - 1));  // always three loads: the count above stays exact
            bf16_t* dst = dst0 + buf * kBTile;
#pragma unroll
            for (int i = 0; i < 4; i++) *(uint4*)(dst + 8 * nn_chunk(lane, run * 4 + i)) = make_uint4(wv[4 * i], wv[4 * i + 1], wv[4 * i + 2], wv[4 * i + 3]);
            close_phase();
        };
        Raw ra, rb;  // even / odd steps, each reloaded two steps ahead
        issue(ra, 0);
        issue(rb, min(1, steps - 1));
        after_issue();
        for (int u = 0; u < steps; u += 2) {
            fill(ra, u);
            if (u + 1 < steps) fill(rb, u + 1);
        }
    } else if (MODE == kModeNT) {
        const int q = ptid & 3, n_local = ptid >> 2;
        const uint8_t* wrow = p.w[c.seg_c] + c.expert * p.w_expert_bytes + (int64_t)min(c.col0 + n_local, p.n - 1) * p.w_row_bytes;
        const int blocks = steps >> 2;  // K is a whole number of 256-wide blocks
        bf16_t* const dst0 = c.bs + n_local * kLdsStride + q * 8;
        Q4KQuarter even, odd;  // alternate between blocks; a set is loaded four phases before its first use
        q4k_quarter_load(even, wrow, 0, q);
        after_issue();
        auto fill = [&](auto s_c, const Q4KQuarter& ch, int u) __attribute__((always_inline)) {
            constexpr int S = decltype(s_c)::value;
            open_phase(u);
            uint32_t lo[4], hi[4];
            q4k_quarter_decode<S>(ch.hdr, S == 0 ? ch.g0 : S == 1 ? ch.g1 : S == 2 ? ch.g2 : ch.g3, lo, hi);
            bf16_t* dst = dst0 + buf * kBTile;
            *(uint4*)dst = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            *(uint4*)(dst + 32) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
            close_phase();
        };
        auto block_phases = [&](Q4KQuarter& cur, Q4KQuarter& nxt, int k) __attribute__((always_inline)) {
            q4k_quarter_load(nxt, wrow, min(k + 1, blocks - 1), q);  // unconditional: see the wide path
            q4k_quarter_pin(cur);
            fill(std::integral_constant<int, 0>{}, cur, 4 * k);
            q4k_quarter_pin(cur);
            fill(std::integral_constant<int, 1>{}, cur, 4 * k + 1);
            q4k_quarter_pin(cur);
            fill(std::integral_constant<int, 2>{}, cur, 4 * k + 2);
            q4k_quarter_pin(cur);
            fill(std::integral_constant<int, 3>{}, cur, 4 * k + 3);
        };
        for (int k = 0; k < blocks; k += 2) {
            block_phases(even, odd, k);
            if (k + 1 < blocks) block_phases(odd, even, k + 1);
        }
    } else {
        // tall: 128 output columns = four runs per row; producer wave w takes rows 8w .. 8w+7,
        // lane = (row, run, half of the run): the eight lanes of a row ask for one header and 64 adjacent bytes
        const int lane = 8 * pw + ((ptid & 63) >> 3);  // contraction row inside the step
        const int run_w = (ptid & 7) >> 1, half = ptid & 1;
        const int ksub = min((c.col0 >> 5) + run_w, (p.k >> 5) - 1);  // runs past the end are clamped, never stored
        const int j = ksub & 7;
        const int64_t blk_off = (int64_t)(ksub >> 3) * 144;
        const int q_off = 16 + 32 * (j >> 1) + 16 * half;
        auto issue = [&](Q4KHalfRun& r, int u) __attribute__((always_inline)) {
            int seg_k, kc0;
            step_origin<MODE>(p, u, seg_k, kc0);
            const int wrow = min(kc0 + lane, p.n - 1);  // rows past the end meet the zero-filled tail of the A tile
            const uint8_t* blk = p.w[seg_k] + c.expert * p.w_expert_bytes + (int64_t)wrow * p.w_row_bytes + blk_off;
            load16_untracked(r.hdr, blk);
            load16_untracked(r.q, blk + q_off);
        };
        bf16_t* const dst0 = c.bs + lane * kNnPitch;
        auto fill = [&](Q4KHalfRun& r, int u) __attribute__((always_inline)) {
            open_phase(u);
            wait_loads_at_most(2);  // the other set's two loads may still be on their way
            q4k_half_run_pin(r);
            uint32_t wv[8];
            q4k_half_run_decode(r, j, wv);
            issue(r, min(u + 2, steps - 1));  // always two loads: the count above stays exact
            bf16_t* dst = dst0 + buf * kBTile;
            *(uint4*)(dst + 8 * nn_chunk(lane, run_w * 4 + half * 2)) = make_uint4(wv[0], wv[1], wv[2], wv[3]);
            *(uint4*)(dst + 8 * nn_chunk(lane, run_w * 4 + half * 2 + 1)) = make_uint4(wv[4], wv[5], wv[6], wv[7]);
            close_phase();
        };
        Q4KHalfRun ra, rb;  // even / odd steps, each reloaded two steps ahead
        issue(ra, 0);
        issue(rb, min(1, steps - 1));
        after_issue();
        for (int u = 0; u < steps; u += 2) {
            fill(ra, u);
            if (u + 1 < steps) fill(rb, u + 1);
        }
    }
    lds_barrier();
}

// ---- consumer waves, instantiated per number of live 32-row blocks.
template <int QT, int MODE, int EPI, int LIVE, class AfterIssue>
static __device__ __forceinline__ void consume(const MmqParams& p, const TileCtx& c, int lane, int cw, AfterIssue&& after_issue) {
    const int wave_m = cw / kWavesN, wave_n = cw % kWavesN;
    const int lane_c = lane & 31, lane_h = lane >> 5;
    f32x16_t acc[LIVE][kColBlocks];
#pragma unroll
    for (int i = 0; i < LIVE; i++)
#pragma unroll
        for (int j = 0; j < kColBlocks; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;
    // this lane's A row inside a 128-row half of the tile, and the swizzled slot of each sub-step's chunk
    const uint8_t* a_row = c.as + (32 * wave_m + lane_c) * kARowBytes;
    int a_koff[4];
#pragma unroll
    for (int kk = 0; kk < 4; kk++) a_koff[kk] = a_slot(lane_c, 2 * kk + lane_h) * 16;
    const int b_off = (wave_n * 64 + lane_c) * kLdsStride + lane_h * 8;
    // transposing read: within a group of 16 lanes, lane L receives element L % 4 of the 8 bytes addressed
    // by lanes L / 4 + 4 j (j = 0..3).  Source lane s = L % 16 therefore points at contraction row s / 4 and
    // columns 4 (s % 4) .. +3 of its group's 16 columns; groups 0, 1 take columns 0..15 / 16..31 of the
    // block, groups 2, 3 the same columns eight contraction rows further on.
    const int tr_group = lane >> 4, tr_s = lane & 15;
    // (the 16-byte chunk that holds them sits at its swizzled position, nn_chunk; the row's low bits do not
    // depend on the sub-step, 16 rows on)
    const int tr_row = 8 * (tr_group >> 1) + (tr_s >> 2);
    int tr_lo[kColBlocks], tr_hi[kColBlocks];
#pragma unroll
    for (int cb = 0; cb < kColBlocks; cb++) {
        const int col = wave_n * 64 + cb * 32 + 16 * (tr_group & 1) + 4 * (tr_s & 3);
        tr_lo[cb] = tr_row * kNnPitch + nn_chunk(tr_row, col >> 3) * 8 + (col & 7);
        tr_hi[cb] = (tr_row + 4) * kNnPitch + nn_chunk(tr_row + 4, col >> 3) * 8 + (col & 7);
    }

    // Operands of one sub-step (16 of the contraction): LIVE row-block runs of A, two column-block runs of W.
    struct Operands {
        bf16x8_t a[LIVE], b[kColBlocks];
    };
    // (the LoRA tiles ahead of the main steps use the same two W layouts)
    auto load_operands = [&](Operands& o, int stage, int buf, int kk) __attribute__((always_inline)) {
        const uint8_t* a_lds = a_row + stage * kAStageBytes + a_koff[kk];
        if (MODE == kModeNN) {
            // W tile is [contraction row][output column]: each transposing 8-byte read hands this lane
            // four consecutive contraction values of its column, two reads make the MFMA operand
            const bf16_t* t_lds = c.bs + buf * kBTile + kk * 16 * kNnPitch;
#pragma unroll
            for (int cb = 0; cb < kColBlocks; cb++) {
                const v4i16_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(t_lds + tr_lo[cb]));
                const v4i16_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(t_lds + tr_hi[cb]));
                o.b[cb] = __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
            }
        } else {
            const bf16_t* b_lds = c.bs + buf * kBTile + b_off + kk * 16;
#pragma unroll
            for (int cb = 0; cb < kColBlocks; cb++) o.b[cb] = *(const bf16x8_t*)(b_lds + cb * 32 * kLdsStride);
        }
#pragma unroll
        for (int rb = 0; rb < LIVE; rb++) o.a[rb] = *(const bf16x8_t*)(a_lds + rb * kWavesM * 32 * kARowBytes);
    };
    auto mfma_operands = [&](const Operands& o) __attribute__((always_inline)) {
#pragma unroll
        for (int rb = 0; rb < LIVE; rb++)
#pragma unroll
            for (int cb = 0; cb < kColBlocks; cb++)
                acc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.a[rb], o.b[cb], acc[rb][cb], 0, 0, 0);
    };

    AIssuer ai;
    a_loader_init(ai.ld, p, c, lane, cw);
    ai.next_step = 0, ai.next_stage = c.base;
#pragma unroll
    for (int d = 0; d < kAhead; d++) a_issue_next<MODE>(ai, p, c);
    after_issue();
    if (c.base == 1) {  // LoRA tiles sit in stage 0 / buffer 0: acc = s * LA . LB^T, r_pad / 16 sub-steps
        const int n = p.r_pad >> 4;
#pragma unroll
        for (int kk = 0; kk < 4; kk++)
            if (kk < n) {
                Operands o;
                load_operands(o, 0, 0, kk);
                mfma_operands(o);
            }
        const float s = p.lora_scale;
#pragma unroll
        for (int i = 0; i < LIVE; i++)
#pragma unroll
            for (int j = 0; j < kColBlocks; j++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][j][e] *= s;
    }
    a_wait_step(ai, c, 0);
    lds_barrier();
    // Main steps, software pipelined inside the wave: the operands of sub-step k+1 are read from LDS
    // while the MFMAs of sub-step k run, and the barrier that releases the buffers sits between the last
    // LDS read of a step and its last MFMAs, so the first read of the next step hides behind them.
    // Step t lives in A stage (t + base) % 3 and W buffer (t + base) & 1.  A wave gets one
    // 16-byte-per-lane LDS read through roughly every 32 cycles, the same cadence as its MFMAs: reads
    // and MFMAs alternate one by one; each sub-step also issues one group of the A tile of step t + 2.
#define GGQ_MFMA_READ_PAIRS()                                                                              \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); \
    __builtin_amdgcn_sched_barrier(0)
#define GGQ_STAGE(NEXT, CUR, KK, J)            \
    a_issue_part<MODE, J, J + 1>(ai, p, c);    \
    load_operands(NEXT, stage, buf, KK);       \
    mfma_operands(CUR);                        \
    GGQ_MFMA_READ_PAIRS()
    if (LIVE == 1) {
        // One live row block: two MFMAs per sub-step are too few to hide the LDS latency of the next
        // sub-step's reads, so all twelve reads of the step go out at once behind the barrier and the
        // MFMAs follow them as they land.
        const int steps = c.total_steps;
        int stage = c.base, buf = c.base;
        for (int t = 0; t < steps; t++) {  // the A loads issued in here are those of step t + kAhead
            a_issue_part<MODE, 0, kGroupsPerWave>(ai, p, c);
            a_issue_advance(ai);
            Operands o[4];
#pragma unroll
            for (int kk = 0; kk < 4; kk++) load_operands(o[kk], stage, buf, kk);
#pragma unroll
            for (int kk = 0; kk < 4; kk++) mfma_operands(o[kk]);
            a_wait_step(ai, c, t + 1);
            lds_barrier();
            stage = stage == kAStages - 1 ? 0 : stage + 1;
            buf ^= 1;
        }
    } else {
        const int steps = c.total_steps;
        int stage = c.base, buf = c.base;
        Operands x, y;
        load_operands(x, stage, buf, 0);
        for (int t = 0; t < steps; t++) {  // the A loads issued in here are those of step t + kAhead
            // (a ring of two stages has one step of lead: all of the next step's groups go out at once)
            if (kAhead == 1) a_issue_part<MODE, 1, kGroupsPerWave>(ai, p, c);
            GGQ_STAGE(y, x, 1, 0);
            if (kAhead > 1) {
                GGQ_STAGE(x, y, 2, 1);
                GGQ_STAGE(y, x, 3, 2);
                a_issue_part<MODE, 3, 4>(ai, p, c);
            } else {
                GGQ_STAGE(x, y, 2, kGroupsPerWave);
                GGQ_STAGE(y, x, 3, kGroupsPerWave);
            }
            a_issue_advance(ai);
            a_wait_step(ai, c, t + 1);
            lds_barrier();  // every LDS read of this step has landed; its stage and buffer may be refilled
            stage = stage == kAStages - 1 ? 0 : stage + 1;
            buf ^= 1;
            if (t + 1 < steps) load_operands(x, stage, buf, 0);
            mfma_operands(y);
            GGQ_MFMA_READ_PAIRS();
        }
    }
#undef GGQ_MFMA_READ_PAIRS
#undef GGQ_STAGE

    // ---- epilogue.  acc[rb][cb][i]: tile row = 32*(kWavesM*rb + wave_m) + 8*(i/4) + 4*lane_h + (i%4),
    //                                 tile col = 64*wave_n + 32*cb + lane_c
    const int col_base = c.col0 + wave_n * 64 + lane_c;
    {
        // everything that does not depend on the element is read once, up front
        const int64_t ldc = p.ldc;
        char* const cbase = (char*)p.c[EPI == kEpiStore ? c.seg_c : 0];
        const int rows_valid = c.rows_valid;
        const bool col_ok[kColBlocks] = {col_base < c.out_cols, col_base + 32 < c.out_cols};
#pragma unroll
        for (int rb = 0; rb < LIVE; rb++) {
            const int r_lane = 32 * (kWavesM * rb + wave_m) + lane_h * 4;  // this lane's first row of the block
            const int64_t lane_elem = (int64_t)(c.row_begin + r_lane) * ldc + col_base;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int dr = (i >> 2) * 8 + (i & 3);  // uniform row step inside the block
                if (r_lane + dr >= rows_valid) continue;
                const int64_t elem = lane_elem + (int64_t)dr * ldc;
                float rs = 1.0f;
                if (EPI == kEpiAccumF32 && p.row_scale) rs = c.row_scale[r_lane + dr];
#pragma unroll
                for (int cb = 0; cb < kColBlocks; cb++) {
                    if (!col_ok[cb]) continue;
                    const float v = acc[rb][cb][i];
                    if (EPI == kEpiStore) ((bf16_t*)cbase)[elem + cb * 32] = to_bf16(v);
                    else ((float*)cbase)[elem + cb * 32] = fmaf(((float*)cbase)[elem + cb * 32], rs, v);
                }
            }
        }
    }
}

// A consumer wave without a live row block still moves its share of the A tile and keeps the
// barriers company.
template <int MODE, class AfterIssue>
static __device__ __forceinline__ void consume_idle(const MmqParams& p, const TileCtx& c, int lane, int cw, AfterIssue&& after_issue) {
    AIssuer ai;
    a_loader_init(ai.ld, p, c, lane, cw);
    ai.next_step = 0, ai.next_stage = c.base;
#pragma unroll
    for (int d = 0; d < kAhead; d++) a_issue_next<MODE>(ai, p, c);
    after_issue();
    a_wait_step(ai, c, 0);
    lds_barrier();
    for (int t = 0; t < c.total_steps; t++) {
        a_issue_next<MODE>(ai, p, c);
        a_wait_step(ai, c, t + 1);
        lds_barrier();
    }
}

// Tile assignment of a single-shape launch.  Hardware deals consecutive workgroup ids round-robin over
// the 8 XCDs; remap so that consecutive logical tiles (which share an A tile) land on one XCD and hit
// its L2.  The split uses the number of tiles that exist (read from the device-built table for grouped
// launches), not the launch's upper bound, so all eight XCDs get an equal share of real work.
template <int QT, int MODE, int EPI>
static __device__ __forceinline__ void run(const MmqParams& p) {
    const int col_tiles = (MODE == kModeNT ? p.nseg : 1) * p.col_tiles_per_seg;
    const int row_tiles = p.tiles ? min(*p.num_tiles, p.max_row_tiles) : p.max_row_tiles;
    const int total_tiles = row_tiles * col_tiles;
    const int per_xcd = (total_tiles + 7) >> 3;
    const int slot = (int)(blockIdx.x >> 3);
    const int logical = (int)(blockIdx.x & 7) * per_xcd + slot;
    if (slot >= per_xcd || logical >= total_tiles) return;
    const int row_tile = logical / col_tiles;
    run_tile<QT, MODE, EPI>(p, p.tiles, row_tile, logical - row_tile * col_tiles, p.col_tiles_per_seg);
}

// One output tile: row tile `row_tile` of `tiles` (or of the dense row range), column tile `col_tile`.
template <int QT, int MODE, int EPI>
static __device__ __forceinline__ void run_tile(const MmqParams& p, const TileDesc* tiles, int row_tile, int col_tile, int col_tiles_per_seg) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
    TileCtx c;
    c.as = smem_raw;
    c.as_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem_raw;
    c.bs = (bf16_t*)(smem_raw + kAStages * kAStageBytes);
    uint2* grid_lds = (uint2*)(smem_raw + kTileLdsBytes);  // the decoder's tables, IQ2_XXS only
    c.grid = grid_lds;
    // the accumulate epilogue's factor per tile row, read once per tile: one dependent global load per row and lane in the
    // epilogue costs a memory round trip each
    float* row_scale = (float*)(smem_raw + kTileLdsBytes + (QT == kIQ2_XXS ? Fmt<kIQ2_XXS>::kTableWords * 4 : 0));
    c.row_scale = row_scale;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps control flow scalar

    c.col_tile = col_tile;
    int row_end;
    if (tiles) {
        const TileDesc t = tiles[row_tile];
        c.row_begin = t.row_begin, row_end = t.row_end, c.expert = t.expert;
    } else {
        c.row_begin = row_tile * kTM;
        row_end = min(p.m, c.row_begin + kTM);
        c.expert = 0;
    }
    c.rows_valid = row_end - c.row_begin;  // 1..kTM
    // column tile -> (segment, first output column inside the segment)
    c.seg_c = MODE == kModeNT ? c.col_tile / col_tiles_per_seg : 0;
    c.col0 = (c.col_tile - c.seg_c * col_tiles_per_seg) * kTN;
    c.out_cols = MODE == kModeNT ? p.n : p.k;     // output columns per segment
    c.contraction = MODE == kModeNT ? p.k : p.n;  // contraction length per segment
    c.total_steps = (MODE == kModeNN ? p.nseg : 1) * p.steps_per_seg;
    c.base = p.r_pad > 0 ? 1 : 0;
    c.a_fast = ((p.lda & 7) == 0) && ((c.contraction & 63) == 0 || p.a_zero_padded) &&
               ((((uintptr_t)p.a[0]) | ((uintptr_t)p.a[MODE == kModeNN && p.nseg > 1 ? 1 : 0])) & 15) == 0;

    if (QT == kIQ2_XXS) {  // selector and sign tables of the decoder (6 KB)
        uint32_t* words = (uint32_t*)grid_lds;
        for (int i = tid; i < Fmt<kIQ2_XXS>::kTableWords; i += kThreadsWG) words[i] = Fmt<kIQ2_XXS>::table_word(i, i < 1024 ? d_iq2xxs_grid_mm[i >> 2] : 0);
    }
    // ---- LoRA tiles go to A stage 0 / W buffer 0 (all lanes load): LA[rows, :r] and LB.  Every wave runs
    // this once, right after it has issued its first loads of the tile proper (A tile / packed weights),
    // so that the two memory round trips overlap.
    auto lora_tiles = [&]() __attribute__((always_inline)) {
        if (p.r_pad > 0) {
            const int chunks = p.r_pad >> 3;  // 16-byte chunks per row (r_pad % 16 == 0)
            for (int id = tid; id < kTM * 8; id += kThreadsWG) {
                const int r = id >> 3, ch = id & 7;
                uint4 v = zero4();
                if (r < c.rows_valid && ch < chunks) v = *(const uint4*)(p.la + (int64_t)(c.row_begin + r) * p.r_pad + ch * 8);
                *(uint4*)(c.as + r * kARowBytes + a_slot(r, ch) * 16) = v;
            }
            if (MODE == kModeNT) {
                // forward: the factor B is [columns][r_pad], the layout of the forward W tile
                const bf16_t* lb = p.lb + c.expert * p.lb_expert_elems + (int64_t)(c.seg_c * c.out_cols + c.col0) * p.r_pad;
                for (int id = tid; id < kTN * 8; id += kThreadsWG) {
                    const int cidx = id >> 3, ch = id & 7;
                    uint4 v = zero4();
                    if (c.col0 + cidx < c.out_cols && ch < chunks) v = *(const uint4*)(lb + (int64_t)cidx * p.r_pad + ch * 8);
                    *(uint4*)&c.bs[cidx * kLdsStride + ch * 8] = v;
                }
            } else {
                // grad-input: the factor A is [r][output columns], which is the layout of the grad-input W tile
                // ([contraction row][column]); rows r .. r_pad - 1 are zero
                const bf16_t* lb = p.lb + c.expert * p.lb_expert_elems + c.col0;
                const bool vec = (c.out_cols & 7) == 0;
                for (int id = tid; id < p.r_pad * (kTN / 8); id += kThreadsWG) {
                    const int j = id / (kTN / 8), ch = id - j * (kTN / 8);
                    const int col = c.col0 + ch * 8;
                    uint4 v = zero4();
                    if (j < p.lora_rank) {
                        const bf16_t* src = lb + (int64_t)j * c.out_cols + ch * 8;
                        v = vec && col + 8 <= c.out_cols ? *(const uint4*)src : load8_slow(src, c.out_cols - col);
                    }
                    *(uint4*)&c.bs[j * kNnPitch + nn_chunk(j, ch) * 8] = v;
                }
            }
        }
        if (EPI == kEpiAccumF32 && p.row_scale) {  // the factor that rescales the accumulator row before the addition
            for (int r = tid; r < kTM; r += kThreadsWG) row_scale[r] = p.row_scale[c.row_begin + min(r, c.rows_valid - 1)];
        }
        __syncthreads();  // LoRA tiles, the codebook tables and the row values are visible
    };

    if (wave >= kCW) {
        if (QT == kQ4_K) produce_q4k<MODE>(p, c, tid - kProducerLanes, wave - kCW, lora_tiles);
        else if constexpr (SH == 1) produce_all<QT, MODE>(p, c, tid - kProducerLanes, lora_tiles);
        else if (wave < 12) produce<QT, MODE, 0>(p, c, tid & 255, wave & 3, lora_tiles);
        else produce<QT, MODE, 1>(p, c, tid & 255, wave & 3, lora_tiles);
    } else {
        const int cw = wave, wave_m = cw / kWavesN;
        // this wave's row blocks are tile rows 32*wave_m .. +31 and 32*(wave_m + kWavesM) .. +31; blocks fill up from row 0
        const int blocks = (c.rows_valid + 31) >> 5;
        const int live = (blocks > wave_m ? 1 : 0) + (blocks > wave_m + kWavesM ? 1 : 0);
        switch (live) {
            case 0: consume_idle<MODE>(p, c, lane, cw, lora_tiles); break;
            case 1: consume<QT, MODE, EPI, 1>(p, c, lane, cw, lora_tiles); break;
            default: consume<QT, MODE, EPI, 2>(p, c, lane, cw, lora_tiles); break;
        }
    }
}
};  // struct Tile

template <int QT, int MODE, int EPI, int SH>
__global__ __launch_bounds__(kThreads, 1) __attribute__((amdgpu_waves_per_eu(4, 4))) void mmq_tile_kernel(const MmqParams p) {
    Tile<SH>::template run<QT, MODE, EPI>(p);
}

// Grouped launch with both shapes in one grid: wide tiles for the row tiles of table `tiles`, tall tiles
// for those of `tiles2`.  A row tile with all its column tiles is the unit that must stay on one XCD (its
// A tile is shared); units go round-robin over the XCDs, wide (heavier) units first, so that every XCD
// gets an equal share of both kinds.
template <int QT, int MODE, int EPI>
__global__ __launch_bounds__(kThreads, 1) __attribute__((amdgpu_waves_per_eu(4, 4))) void mmq_mixed_kernel(const MmqParams p) {
    const int segs = MODE == kModeNT ? p.nseg : 1;
    const int cols_w = segs * p.col_tiles_per_seg, cols_t = segs * p.col_tiles_per_seg2;
    const int n_w = min(*p.num_tiles, p.max_row_tiles), n_t = min(*p.num_tiles2, p.max_row_tiles2);
    const int xcd = (int)(blockIdx.x & 7), slot = (int)(blockIdx.x >> 3);
    const int units_w = (n_w - xcd + 7) >> 3, units_t = (n_t - xcd + 7) >> 3;  // units xcd, xcd + 8, ...
    const int slots_w = units_w * cols_w;
    if (slot < slots_w) {
        const int unit = slot / cols_w;
        Tile<kShapeWide>::template run_tile<QT, MODE, EPI>(p, p.tiles, xcd + 8 * unit, slot - unit * cols_w, p.col_tiles_per_seg);
    } else if (slot - slots_w < units_t * cols_t) {
        const int s2 = slot - slots_w, unit = s2 / cols_t;
        Tile<kShapeTall>::template run_tile<QT, MODE, EPI>(p, p.tiles2, xcd + 8 * unit, s2 - unit * cols_t, p.col_tiles_per_seg2);
    }
}

}  // namespace ggq
