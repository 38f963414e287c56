// Rank-r LoRA side kernels (r <= 64) around the packed-weight tile kernel.  All are HBM-bound streams
// over the activations; they use the 16x16x32 bf16 MFMA so the arithmetic never shows.
//
//   skinny_nt      out[m, j]  = sum_c In[m, c] * F[e][j, c]          (x A^T,  dY B via B^T)
//   factor_grad    G[e][c, j] = s * sum_{m in group e} In[m, c] * S[m, j]   (dB, dA; fixed order, no atomics)
//   pad / transpose helpers that lay the factors out [cols][r_pad] for the tile kernel.
#include <algorithm>
#include "common.h"
#include "launch.h"
#include "mmq_host.h"

namespace ggq {

__device__ __forceinline__ uint4 load8g(const bf16_t* p, int valid, bool vec) {
    if (valid >= 8 && vec) return *(const uint4*)p;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (valid <= 0) return v;
    uint32_t e[8];
#pragma unroll
    for (int i = 0; i < 8; i++) e[i] = i < valid ? (uint32_t)p[i] : 0u;
    v.x = e[0] | (e[1] << 16), v.y = e[2] | (e[3] << 16), v.z = e[4] | (e[5] << 16), v.w = e[6] | (e[7] << 16);
    return v;
}

// ---- out[m, 0..r_pad) = In[m, :] . F[e][0..r, :]^T.  One workgroup per 16 rows; its four waves deal the
// contraction out in 128-wide trips (trip t to wave t % 4), so a 64-row tile keeps sixteen waves of loads
// in flight, and add their partial sums through LDS in wave order (fixed order: deterministic).
// In may be two column segments (pair): contraction runs over seg 0 then seg 1, F rows are [r][nseg*C].
template <int JB>  // JB = r_pad / 16
__global__ __launch_bounds__(256) void skinny_nt_kernel(SkinnyNtParams p) {
    __shared__ float red[3][JB][4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // Workgroup ids go round-robin over the eight XCDs; give every XCD a contiguous run of units, so the
    // workgroups that share one expert's factor rows share an L2 as well.
    const int units = 4 * (p.tiles ? *p.num_tiles : (int)(gridDim.x >> 2));
    const int per_xcd = (units + 7) >> 3;
    const int slot = blockIdx.x >> 3;
    if (slot >= per_xcd) return;
    const int unit = (blockIdx.x & 7) * per_xcd + slot;
    if (unit >= units) return;
    const int tile = unit >> 2, sub = unit & 3;
    int group = 0, row_begin, row_end;
    if (p.tiles) {
        const TileDesc t = p.tiles[tile];
        group = t.group, row_begin = t.row_begin, row_end = t.row_end;
    } else {
        row_begin = tile * 64;
        row_end = min(p.m, row_begin + 64);
    }
    const int64_t expert = p.expert_ids ? p.expert_ids[group] : 0;
    const int m0 = row_begin + sub * 16;
    if (m0 >= row_end) return;  // uniform over the workgroup
    const int li = lane & 15, lq = lane >> 4;
    const int row = m0 + li;
    const bool row_ok = row < row_end;
    const int src_row = row_ok ? p.in_rows.source(row) : 0;  // stored row of segment 0 (an index comes with one segment)
    const bf16_t* f = p.f + expert * p.f_expert_elems;  // [r][ldf]
    f32x4_t acc[JB];
#pragma unroll
    for (int jb = 0; jb < JB; jb++) acc[jb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    const bool fvec = ((p.ldf & 7) == 0) && ((p.c & 7) == 0) && (((uintptr_t)p.f & 15) == 0);
    bool vec = (p.ld_in & 7) == 0;
    for (int seg = 0; seg < p.nseg; seg++) vec = vec && (((uintptr_t)p.in[seg] & 15) == 0);
    // aligned operands: 128-wide trips, every load of a trip issued ahead of its MFMAs
    const int trips_per_seg = (vec && fvec) ? p.c / 128 : 0;
    for (int t = wave; t < trips_per_seg * p.nseg; t += 4) {
        const int seg = t / trips_per_seg, c0 = (t - seg * trips_per_seg) * 128;
        const bf16_t* in = p.in[seg] + (int64_t)src_row * p.ld_in;
        uint4 av[4], bv[JB][4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int cc = c0 + 32 * u + lq * 8;
            av[u] = row_ok ? *(const uint4*)(in + cc) : make_uint4(0, 0, 0, 0);
#pragma unroll
            for (int jb = 0; jb < JB; jb++) {
                const int j = jb * 16 + li;
                bv[jb][u] = j < p.r ? *(const uint4*)(f + (int64_t)j * p.ldf + seg * p.c + cc) : make_uint4(0, 0, 0, 0);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int jb = 0; jb < JB; jb++)
                acc[jb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av[u]), __builtin_bit_cast(bf16x8_t, bv[jb][u]), acc[jb], 0, 0, 0);
    }
    // what the trips leave (and everything, for unaligned operands): 32-wide steps dealt the same way
    int step = 0;
    for (int seg = 0; seg < p.nseg; seg++) {
        const bf16_t* in = p.in[seg] + (int64_t)src_row * p.ld_in;
        for (int c0 = trips_per_seg * 128; c0 < p.c; c0 += 32, step++) {
            if ((step & 3) != wave) continue;
            const int cc = c0 + lq * 8;
            const uint4 av = load8g(in + cc, row_ok ? p.c - cc : 0, vec);
            const bf16x8_t a = __builtin_bit_cast(bf16x8_t, av);
#pragma unroll
            for (int jb = 0; jb < JB; jb++) {
                const int j = jb * 16 + li;
                const uint4 bv = load8g(f + (int64_t)j * p.ldf + seg * p.c + cc, j < p.r ? p.c - cc : 0, fvec);
                acc[jb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8_t, bv), acc[jb], 0, 0, 0);
            }
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int jb = 0; jb < JB; jb++)
#pragma unroll
            for (int v = 0; v < 4; v++) red[wave - 1][jb][v][lane] = acc[jb][v];
    }
    __syncthreads();
    if (wave > 0) return;
    // acc[jb][v]: row = m0 + 4*lq + v, col = 16*jb + li
#pragma unroll
    for (int jb = 0; jb < JB; jb++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const float sum = ((acc[jb][v] + red[0][jb][v][lane]) + red[1][jb][v][lane]) + red[2][jb][v][lane];
            const int r = m0 + 4 * lq + v;
            if (r < row_end) p.out[(int64_t)r * (JB * 16) + jb * 16 + li] = to_bf16(sum);
        }
}

// ---- The same product for aligned operands with a contraction that is a multiple of 64: every byte
// goes global -> LDS directly in whole 128-byte row pieces (a lane-per-row register load of the MFMA
// operand layout costs the vector cache one access per lane; these loads cost one per 64 bytes), and the
// operands are read back from LDS.  One workgroup per 64-row tile; wave w owns rows 32*(w&1)..+31 and
// every second 64-wide contraction step (parity w>>1), with a two-stage ring of its own: no workgroup
// barrier inside the loop.  Rows keep their 16-byte chunks XOR-swizzled (a_slot) so both the 1 KB writes
// and the operand reads are bank-conflict free.
// FNAT: the factor is given as [contraction][r] (r a multiple of 8, the natural layout of B for dY . B): a
// 64-wide step of it is one contiguous run, copied as it is; the operand reads transpose it on the way out
// of LDS (ds_read_b64_tr_b16: within 16 lanes, lane L gets element L % 4 of the 8 bytes addressed by lanes
// L / 4 + 4 t, t = 0..3, so source lane s points at contraction row s / 4, factor columns 4 (s % 4) .. +3).
typedef short v4i16_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4i16_t* lds_v4i16_ptr;

template <int JB, bool FNAT>
__global__ __launch_bounds__(256) void skinny_nt_direct_kernel(SkinnyNtParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t sk_lds[];
    constexpr int kInBytes = 32 * 128, kFBytes = JB * 16 * 128, kStage = kInBytes + kFBytes;
    const int f_loads = FNAT ? p.r >> 3 : 2 * JB;  // 1 KB direct-to-LDS instructions per stage of the factor
    const int loads = 4 + f_loads;                 // ... and of the stage
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int units = p.tiles ? *p.num_tiles : (p.m + 63) / 64;
    const int per_xcd = (units + 7) >> 3;
    const int slot = blockIdx.x >> 3;
    if (slot >= per_xcd) return;
    const int unit = (blockIdx.x & 7) * per_xcd + slot;
    if (unit >= units) return;
    int group = 0, row_begin, row_end;
    if (p.tiles) {
        const TileDesc t = p.tiles[unit];
        group = t.group, row_begin = t.row_begin, row_end = t.row_end;
    } else {
        row_begin = unit * 64;
        row_end = min(p.m, row_begin + 64);
    }
    const int64_t expert = p.expert_ids ? p.expert_ids[group] : 0;
    const int half = wave & 1, parity = wave >> 1;
    const int r0 = row_begin + 32 * half;
    const int rows_valid = row_end - r0;  // <= 0: this wave only joins the final barrier
    const bf16_t* f = p.f + expert * p.f_expert_elems;  // [r][ldf], or [nseg*C][r] (FNAT)
    uint8_t* my = sk_lds + wave * 2 * kStage;
    const uint32_t my_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)my;
    // lane's 16 bytes in each 8-row load: row lane/8 of the load, the chunk that belongs in slot lane%8
    uint32_t in_off[4], f_off[2 * JB];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int rl = 8 * q + (lane >> 3);
        int row = min(rl, rows_valid - 1);  // rows past the tile are copies of its last row, never stored
        if (p.in_rows.on()) row = rows_valid > 0 ? p.in_rows.source(r0 + row) : 0;  // the whole stored row (matrix under 4 GiB)
        in_off[q] = ((uint32_t)row * (uint32_t)p.ld_in + (uint32_t)(a_slot(rl, lane & 7) * 8)) * 2u;
    }
#pragma unroll
    for (int q = 0; q < 2 * JB; q++) {
        if (FNAT) {
            f_off[q] = (uint32_t)(q * 64 + lane) * 16u;  // a straight copy
        } else {
            const int jl = 8 * q + (lane >> 3);
            const int j = min(jl, p.r - 1);  // factor rows past the rank are masked when the operand is read
            f_off[q] = ((uint32_t)j * (uint32_t)p.ldf + (uint32_t)(a_slot(jl, lane & 7) * 8)) * 2u;
        }
    }
    const int steps_per_seg = p.c / 64, steps = steps_per_seg * p.nseg;
    auto issue = [&](int step, int stage) {
        const int seg = step / steps_per_seg, c0 = (step - seg * steps_per_seg) * 64;
        const bf16_t* in_base = p.in[seg] + (p.in_rows.on() ? 0 : (int64_t)r0 * p.ld_in) + c0;
        const bf16_t* f_base = FNAT ? f + ((int64_t)seg * p.c + c0) * p.r : f + seg * p.c + c0;
        const uint32_t lds = my_lds + stage * kStage;
#pragma unroll
        for (int q = 0; q < 4; q++) load16_to_lds(lds + q * 1024, in_off[q], in_base);
#pragma unroll
        for (int q = 0; q < 2 * JB; q++)
            if (q < f_loads) load16_to_lds(lds + kInBytes + q * 1024, f_off[q], f_base);
    };
    const int li = lane & 15, lq = lane >> 4;
    f32x4_t acc[2][JB];
#pragma unroll
    for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int jb = 0; jb < JB; jb++) acc[rb][jb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    if (rows_valid > 0) {
        if (parity < steps) issue(parity, 0);
        int stage = 0;
        for (int step = parity; step < steps; step += 2, stage ^= 1) {
            if (step + 2 < steps) {
                issue(step + 2, stage ^ 1);
                wait_loads_at_most(loads);
            } else {
                wait_loads_at_most(0);
            }
            const uint8_t* st = my + stage * kStage;
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                uint4 b[JB];
#pragma unroll
                for (int jb = 0; jb < JB; jb++) {
                    const int j = jb * 16 + li;
                    if (FNAT) {
                        const uint8_t* src = st + kInBytes + (kk * 32 + 8 * lq + (li >> 2)) * (p.r * 2) + jb * 32 + (li & 3) * 8;
                        const v4i16_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)src);
                        const v4i16_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(src + 4 * (p.r * 2)));
                        b[jb] = __builtin_bit_cast(uint4, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                    } else {
                        b[jb] = *(const uint4*)(st + kInBytes + j * 128 + a_slot(j, kk * 4 + lq) * 16);
                    }
                    if (j >= p.r) b[jb] = make_uint4(0, 0, 0, 0);
                }
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
                    const int rl = rb * 16 + li;
                    const uint4 a = *(const uint4*)(st + rl * 128 + a_slot(rl, kk * 4 + lq) * 16);
#pragma unroll
                    for (int jb = 0; jb < JB; jb++)
                        acc[rb][jb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b[jb]), acc[rb][jb], 0, 0, 0);
                }
            }
            // the next trip's loads overwrite the other stage only; this stage is rewritten one trip later,
            // after these reads have returned (the MFMAs above waited for them)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
    }
    // the odd-parity waves hand their sums to the even ones through the (now idle) ring
    __syncthreads();
    float* red = (float*)(sk_lds + (wave & 1) * 2 * kStage);  // the ring of wave (w&1): its loads are done
    if (parity == 1) {
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
            for (int jb = 0; jb < JB; jb++)
#pragma unroll
                for (int v = 0; v < 4; v++) red[((rb * JB + jb) * 4 + v) * 64 + lane] = acc[rb][jb][v];
    }
    __syncthreads();
    if (parity == 1) return;
    // acc[rb][jb][v]: row = r0 + 16*rb + 4*lq + v, col = 16*jb + li
#pragma unroll
    for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int jb = 0; jb < JB; jb++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float sum = acc[rb][jb][v] + red[((rb * JB + jb) * 4 + v) * 64 + lane];
                const int r = r0 + 16 * rb + 4 * lq + v;
                if (r < row_end) p.out[(int64_t)r * (JB * 16) + jb * 16 + li] = to_bf16(sum);
            }
}

// ---- G[e][c, j] = s * sum_m In[m, c] * S[m, j] over the rows of expert e.  One workgroup per
// (expert, 64 * CB columns); each wave owns CB blocks of 16 columns; rows are consumed 32 at a time
// through LDS, where the operands of the contraction over m are read with transposing loads.  The loads
// of four 32-row slices are issued together and the slices then go through two alternating LDS buffers,
// one barrier each.  Experts without rows get zeros.
template <int JB, int CB>
__global__ __launch_bounds__(256) void factor_grad_kernel(FactorGradParams p) {
    // rows are contraction rows m; the operands are read with transposing 8-byte LDS reads (lane L of a
    // 16-lane group gets element L % 4 of the 8 bytes addressed by lanes L / 4 + 4 t), so the tiles stay as
    // loaded; the row pitches keep four consecutive rows' 32-byte pieces on distinct banks
    constexpr int kCols = 64 * CB, kPitch = kCols + 32, kSPitch = JB * 16 + 8;
    __shared__ __attribute__((aligned(16))) bf16_t in_t[2][32][kPitch];
    __shared__ __attribute__((aligned(16))) bf16_t s_t[2][32][kSPitch];
    __shared__ __attribute__((aligned(16))) bf16_t g_t[4][16][JB * 16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int blocks_per_seg = (p.c + kCols - 1) / kCols;
    const int col_blocks = p.nseg * blocks_per_seg;
    // contiguous runs of (expert, column block) units per XCD: one L2 sees whole rows of an expert
    const int per_xcd = ((int)gridDim.x + 7) >> 3;
    const int unit = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per_xcd || unit >= p.units) return;
    const int splits = p.row_splits > 1 ? p.row_splits : 1;
    const int split = unit % splits, ucb = unit / splits;
    const int e = ucb / col_blocks, cblk = ucb - e * col_blocks;
    const int seg = cblk / blocks_per_seg;
    const int c0 = (cblk - seg * blocks_per_seg) * kCols;
    int row_begin = 0, row_end = p.m;
    if (p.ranges) {
        row_begin = p.ranges[2 * e];
        row_end = p.ranges[2 * e + 1];
    } else if (splits > 1) {  // this workgroup's share of the rows, in whole 32-row slices
        const int share = (((p.m + splits - 1) / splits) + 31) & ~31;
        row_begin = min(p.m, split * share);
        row_end = min(p.m, row_begin + share);
    }
    const bf16_t* in = p.in[seg];
    const bool vec = ((p.ld_in & 7) == 0) && (((uintptr_t)in & 15) == 0);
    const int li = lane & 15, lq = lane >> 4;
    f32x4_t acc[CB][JB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++)
#pragma unroll
        for (int jb = 0; jb < JB; jb++) acc[cb][jb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    constexpr int rp = JB * 16;
    const int tr = threadIdx.x >> 3, tch = threadIdx.x & 7;           // In slice: 32 rows x CB x 8 chunks of 8
    const int sr = threadIdx.x / (rp / 8), sch = threadIdx.x % (rp / 8);  // S slice: 32 rows x rp/8 chunks
    int buf = 0;
    for (int m0 = row_begin; m0 < row_end; m0 += 128) {
        uint4 vin[4][CB], vs[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int r = m0 + 32 * u + tr;
            const int src = r < row_end ? p.in_rows.source(r) : 0;
#pragma unroll
            for (int cb = 0; cb < CB; cb++) {
                const int tcc = c0 + cb * 64 + tch * 8;
                vin[u][cb] = load8g(in + (int64_t)src * p.ld_in + tcc, r < row_end ? p.c - tcc : 0, vec);
            }
            vs[u] = make_uint4(0, 0, 0, 0);
            if (sr < 32 && m0 + 32 * u + sr < row_end) {
                const int64_t row = m0 + 32 * u + sr;
                vs[u] = *(const uint4*)(p.s + row * rp + sch * 8);
                if (p.s_weights) {
                    const int64_t wi = p.s_weight_index[row];
                    // (routing weights act at bf16 precision everywhere on the path)
                    const float w = p.s_weights_are_bf16 ? bf16_to_f32(((const bf16_t*)p.s_weights)[wi]) : bf16_to_f32(to_bf16(((const float*)p.s_weights)[wi]));
                    vs[u] = make_uint4(pack_bf16(bf16_lo(vs[u].x) * w, bf16_hi(vs[u].x) * w), pack_bf16(bf16_lo(vs[u].y) * w, bf16_hi(vs[u].y) * w),
                                       pack_bf16(bf16_lo(vs[u].z) * w, bf16_hi(vs[u].z) * w), pack_bf16(bf16_lo(vs[u].w) * w, bf16_hi(vs[u].w) * w));
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (m0 + 32 * u >= row_end) break;  // uniform over the workgroup
#pragma unroll
            for (int cb = 0; cb < CB; cb++) *(uint4*)&in_t[buf][tr][cb * 64 + tch * 8] = vin[u][cb];
            if (sr < 32) *(uint4*)&s_t[buf][sr][sch * 8] = vs[u];
            // one barrier per slice: the slice after the next reuses this buffer, and every wave passes the
            // next barrier only after its reads of this one
            __syncthreads();
            // B operand (n = factor column j, contraction m): source lane s = li points at contraction row
            // 8*lq + s/4 (+4 for the second read), factor columns 4*(s%4) .. +3 of the block's 16
            bf16x8_t b[JB];
#pragma unroll
            for (int jb = 0; jb < JB; jb++) {
                const bf16_t* b_src = &s_t[buf][8 * lq + (li >> 2)][jb * 16 + (li & 3) * 4];
                const v4i16_t b_lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)b_src);
                const v4i16_t b_hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(b_src + 4 * kSPitch));
                b[jb] = __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(b_lo, b_hi, 0, 1, 2, 3, 4, 5, 6, 7));
            }
            // A operand (row = column c, contraction m): the same pattern over the wave's 16 columns of block cb
#pragma unroll
            for (int cb = 0; cb < CB; cb++) {
                const bf16_t* a_src = &in_t[buf][8 * lq + (li >> 2)][cb * 64 + wave * 16 + (li & 3) * 4];
                const v4i16_t a_lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)a_src);
                const v4i16_t a_hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(a_src + 4 * kPitch));
                const bf16x8_t a = __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(a_lo, a_hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
                for (int jb = 0; jb < JB; jb++) acc[cb][jb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[jb], acc[cb][jb], 0, 0, 0);
            }
            buf ^= 1;
        }
    }
    // acc[cb][jb][v]: c = c0 + 64*cb + wave*16 + 4*lq + v, j = 16*jb + li
    const int64_t ctot = (int64_t)p.nseg * p.c;
    if (splits > 1) {  // unscaled fp32 partial sums [split][column][r_pad]; factor_reduce_kernel finishes
        float* part = p.partials + (int64_t)split * ctot * rp;
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
#pragma unroll
            for (int jb = 0; jb < JB; jb++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int c = c0 + 64 * cb + wave * 16 + 4 * lq + v;
                    if (c < p.c) part[((int64_t)seg * p.c + c) * rp + jb * 16 + li] = acc[cb][jb][v];
                }
        return;
    }
    bf16_t* out = p.out + (int64_t)e * p.out_expert_elems;
    const bool vec4 = (ctot & 3) == 0 && (((uintptr_t)out & 7) == 0);
    const bool vec8 = (p.r & 7) == 0 && (((uintptr_t)out & 15) == 0);
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        const int cw0 = c0 + 64 * cb + wave * 16;  // first column of this wave's block
        if (p.out_j_major) {
            // [r][columns]: a lane holds four consecutive columns of factor row j: one 8-byte store
#pragma unroll
            for (int jb = 0; jb < JB; jb++) {
                const int j = jb * 16 + li, c = cw0 + 4 * lq;
                if (j >= p.r) continue;
                bf16_t* dst = out + (int64_t)j * ctot + (int64_t)seg * p.c + c;
                if (vec4 && c + 3 < p.c) {
                    *(uint2*)dst = make_uint2(pack_bf16(acc[cb][jb][0] * p.scale, acc[cb][jb][1] * p.scale), pack_bf16(acc[cb][jb][2] * p.scale, acc[cb][jb][3] * p.scale));
                } else {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                        if (c + v < p.c) dst[v] = to_bf16(acc[cb][jb][v] * p.scale);
                }
            }
        } else if (vec8) {
            // [columns][r]: the wave's 16 columns x r are one contiguous run; transpose through LDS (each wave
            // reads back only what it wrote; LDS serves a wave in order) and store 16 bytes per lane
#pragma unroll
            for (int jb = 0; jb < JB; jb++)
#pragma unroll
                for (int v = 0; v < 4; v++) g_t[wave][4 * lq + v][jb * 16 + li] = to_bf16(acc[cb][jb][v] * p.scale);
            const int chunks_per_row = p.r >> 3;
            bf16_t* dst = out + ((int64_t)seg * p.c + cw0) * p.r;
            for (int id = lane; id < 16 * chunks_per_row; id += 64) {
                const int row = id / chunks_per_row, ch = id - row * chunks_per_row;
                const uint4 piece = *(const uint4*)&g_t[wave][row][ch * 8];
                if (cw0 + row < p.c) *(uint4*)(dst + (int64_t)id * 8) = piece;
            }
        } else {
#pragma unroll
            for (int jb = 0; jb < JB; jb++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int c = cw0 + 4 * lq + v, j = jb * 16 + li;
                    if (c < p.c && j < p.r) out[((int64_t)seg * p.c + c) * p.r + j] = to_bf16(acc[cb][jb][v] * p.scale);
                }
        }
    }
}

// out = bf16(scale * sum over the row splits, in split order) of the partial sums of a split factor_grad launch.
// One lane per (column, j < r_pad); lanes of a wave run along j, then columns: contiguous reads.
__global__ __launch_bounds__(256) void factor_reduce_kernel(const float* partials, bf16_t* out, int64_t ctot, int r, int r_pad, int splits, int out_j_major,
                                                            float scale) {
    const int64_t total = ctot * r_pad;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t c = i / r_pad;
        const int j = (int)(i - c * r_pad);
        if (j >= r) continue;
        float sum = 0.f;
        for (int sp = 0; sp < splits; sp++) sum += partials[(int64_t)sp * total + i];
        out[out_j_major ? (int64_t)j * ctot + c : c * r + j] = to_bf16(sum * scale);
    }
}

// dst[e][c][0..r_pad) = src[e][c][0..r) zero padded   (transpose = false, src [E][C][r])
// dst[e][c][0..r_pad) = src[e][0..r)[c] zero padded   (transpose = true,  src [E][r][C])
// One lane per (e, c): its r_pad outputs are contiguous (16-byte stores); with transpose the reads of a
// wave are 64 consecutive columns of one factor row.
__global__ __launch_bounds__(256) void pad_factor_kernel(const bf16_t* src, bf16_t* dst, int64_t experts, int c, int r, int r_pad, int transpose) {
    const int64_t total = experts * c;
    for (int64_t ec = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; ec < total; ec += (int64_t)gridDim.x * blockDim.x) {
        const int cc = (int)(ec % c);
        const int64_t e = ec / c;
        for (int j0 = 0; j0 < r_pad; j0 += 8) {
            uint32_t v[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int j = j0 + i;
                v[i] = j < r ? (uint32_t)(transpose ? src[(e * r + j) * c + cc] : src[ec * r + j]) : 0u;
            }
            *(uint4*)(dst + ec * r_pad + j0) = make_uint4(v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16));
        }
    }
}

// dst[e][j][c] = src[e][c][j]  for j < r  (B [E][C][r] -> B^T [E][r][C]).  One lane per (e, c): it reads
// its r contiguous inputs and a wave writes 64 consecutive columns of each output row.
__global__ __launch_bounds__(256) void transpose_factor_kernel(const bf16_t* src, bf16_t* dst, int64_t experts, int c, int r) {
    const int64_t total = experts * c;
    const bool vec = (r & 7) == 0 && (((uintptr_t)src & 15) == 0);
    for (int64_t ec = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; ec < total; ec += (int64_t)gridDim.x * blockDim.x) {
        const int cc = (int)(ec % c);
        const int64_t e = ec / c;
        for (int j0 = 0; j0 < r; j0 += 8) {
            uint32_t w[4] = {0u, 0u, 0u, 0u};
            if (vec) {
                const uint4 q = *(const uint4*)(src + ec * r + j0);
                w[0] = q.x, w[1] = q.y, w[2] = q.z, w[3] = q.w;
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    if (j0 + i < r) w[i >> 1] |= (uint32_t)src[ec * r + j0 + i] << (16 * (i & 1));
            }
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (j0 + i < r) dst[(e * r + j0 + i) * c + cc] = (bf16_t)(w[i >> 1] >> (16 * (i & 1)));
        }
    }
}

static inline unsigned grid_for(int64_t total, int block) {
    int64_t g = (total + block - 1) / block;
    return (unsigned)(g < 1 ? 1 : (g > 65535 * 16 ? 65535 * 16 : g));
}

int pad_factor(const bf16_t* src, bf16_t* dst, int64_t experts, int c, int r, int r_pad, bool transpose, hipStream_t s) {
    const int64_t total = experts * c;
    if (total == 0) return 0;
    hipLaunchKernelGGL(pad_factor_kernel, dim3(grid_for(total, 256)), dim3(256), 0, s, src, dst, experts, c, r, r_pad, transpose ? 1 : 0);
    return check_launch("pad_factor");
}

int transpose_factor(const bf16_t* src, bf16_t* dst, int64_t experts, int c, int r, hipStream_t s) {
    const int64_t total = experts * c;
    if (total == 0) return 0;
    hipLaunchKernelGGL(transpose_factor_kernel, dim3(grid_for(total, 256)), dim3(256), 0, s, src, dst, experts, c, r);
    return check_launch("transpose_factor");
}

template <int JB, bool FNAT>
static int launch_skinny_direct(const SkinnyNtParams& p, int grid_tiles, hipStream_t s) {
    constexpr int kSmem = 4 * 2 * (32 * 128 + JB * 16 * 128);
    static LdsLimit lds_limit;  // per instantiation
    if (int rc = raise_lds_limit(lds_limit, (const void*)skinny_nt_direct_kernel<JB, FNAT>, kSmem, "skinny_nt")) return rc;
    hipLaunchKernelGGL((skinny_nt_direct_kernel<JB, FNAT>), dim3(((unsigned)grid_tiles + 7u) & ~7u), dim3(256), kSmem, s, p);
    return check_launch("skinny_nt_direct");
}

// The factor may be handed over as [contraction][r] (f_natural) when this holds; otherwise the caller
// passes it transposed, [r][contraction].
bool skinny_nt_takes_natural_factor(const SkinnyNtParams& p) {
    bool ok = (p.r & 7) == 0 && (p.ld_in & 7) == 0 && (p.c & 63) == 0 && ((uintptr_t)p.f & 15) == 0 && (p.f_expert_elems & 7) == 0 &&
              (uint64_t)64 * (uint64_t)p.ld_in * 2 < (1ull << 31);
    for (int seg = 0; seg < p.nseg; seg++) ok = ok && ((uintptr_t)p.in[seg] & 15) == 0;
    return ok;
}

int skinny_nt(const SkinnyNtParams& p, int r_pad, int grid_tiles, hipStream_t s) {
    if (grid_tiles <= 0) return 0;
    bool direct = (p.ld_in & 7) == 0 && (p.ldf & 7) == 0 && (p.c & 63) == 0 && ((uintptr_t)p.f & 15) == 0 && (p.f_expert_elems & 7) == 0 &&
                  (uint64_t)64 * (uint64_t)p.ld_in * 2 < (1ull << 31) && (uint64_t)64 * (uint64_t)p.ldf * 2 < (1ull << 31);
    for (int seg = 0; seg < p.nseg; seg++) direct = direct && ((uintptr_t)p.in[seg] & 15) == 0;
    if (p.in_rows.on()) {
        if (p.nseg != 1 || p.in_rows.index_div <= 0 || p.in_rows.index_rows <= 0) return set_error(GGQ_ERR_SHAPE, "skinny_nt: a row index needs one segment and a positive divisor and row count");
        direct = direct && (uint64_t)p.in_rows.index_rows * (uint64_t)p.ld_in * 2 < (1ull << 32);
    }
    if (p.f_natural) {
        if (!skinny_nt_takes_natural_factor(p)) return set_error(GGQ_ERR_SHAPE, "skinny_nt: this shape needs the factor transposed");
        switch (r_pad / 16) {
            case 1: return launch_skinny_direct<1, true>(p, grid_tiles, s);
            case 2: return launch_skinny_direct<2, true>(p, grid_tiles, s);
            case 3: return launch_skinny_direct<3, true>(p, grid_tiles, s);
            case 4: return launch_skinny_direct<4, true>(p, grid_tiles, s);
            default: return set_error(GGQ_ERR_SHAPE, "LoRA rank must be between 1 and 64");
        }
    }
    if (direct) {
        switch (r_pad / 16) {
            case 1: return launch_skinny_direct<1, false>(p, grid_tiles, s);
            case 2: return launch_skinny_direct<2, false>(p, grid_tiles, s);
            case 3: return launch_skinny_direct<3, false>(p, grid_tiles, s);
            case 4: return launch_skinny_direct<4, false>(p, grid_tiles, s);
            default: return set_error(GGQ_ERR_SHAPE, "LoRA rank must be between 1 and 64");
        }
    }
    switch (r_pad / 16) {
        case 1: hipLaunchKernelGGL(skinny_nt_kernel<1>, dim3((4u * (unsigned)grid_tiles + 7u) & ~7u), dim3(256), 0, s, p); break;
        case 2: hipLaunchKernelGGL(skinny_nt_kernel<2>, dim3((4u * (unsigned)grid_tiles + 7u) & ~7u), dim3(256), 0, s, p); break;
        case 3: hipLaunchKernelGGL(skinny_nt_kernel<3>, dim3((4u * (unsigned)grid_tiles + 7u) & ~7u), dim3(256), 0, s, p); break;
        case 4: hipLaunchKernelGGL(skinny_nt_kernel<4>, dim3((4u * (unsigned)grid_tiles + 7u) & ~7u), dim3(256), 0, s, p); break;
        default: return set_error(GGQ_ERR_SHAPE, "LoRA rank must be between 1 and 64");
    }
    return check_launch("skinny_nt");
}

template <int CB>
static int launch_factor_grad(const FactorGradParams& p_in, int r_pad, int64_t experts, hipStream_t s) {
    const int col_blocks = p_in.nseg * ((p_in.c + 64 * CB - 1) / (64 * CB));
    FactorGradParams p = p_in;
    // One row range for everything (a dense layer) leaves only the column blocks to spread over the compute units: deal
    // the rows out as well, enough to give every unit a workgroup, in shares of at least 128 rows.
    p.row_splits = 1;
    if (!p.ranges && experts == 1 && p.partials && col_blocks < 256 && p.m >= 256) {
        const int64_t want = (256 + col_blocks - 1) / col_blocks;
        const int64_t fit = p.partials_bytes / ((int64_t)p.nseg * p.c * r_pad * 4);
        p.row_splits = (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want, p.m / 128), std::min<int64_t>(fit, 64)));
    }
    const int64_t units = experts * col_blocks * p.row_splits;
    if (units <= 0) return 0;
    if (units > 0x7FFFFFF0) return set_error(GGQ_ERR_SHAPE, "factor_grad: grid too large");
    const int64_t grid = (units + 7) / 8 * 8;
    p.units = (int)units;
    switch (r_pad / 16) {
        case 1: hipLaunchKernelGGL((factor_grad_kernel<1, CB>), dim3((unsigned)grid), dim3(256), 0, s, p); break;
        case 2: hipLaunchKernelGGL((factor_grad_kernel<2, CB>), dim3((unsigned)grid), dim3(256), 0, s, p); break;
        case 3: hipLaunchKernelGGL((factor_grad_kernel<3, CB>), dim3((unsigned)grid), dim3(256), 0, s, p); break;
        case 4: hipLaunchKernelGGL((factor_grad_kernel<4, CB>), dim3((unsigned)grid), dim3(256), 0, s, p); break;
        default: return set_error(GGQ_ERR_SHAPE, "LoRA rank must be between 1 and 64");
    }
    if (int rc = check_launch("factor_grad")) return rc;
    if (p.row_splits > 1) {
        const int64_t ctot = (int64_t)p.nseg * p.c;
        const unsigned blocks = (unsigned)std::min<int64_t>((ctot * r_pad + 255) / 256, 4096);
        hipLaunchKernelGGL(factor_reduce_kernel, dim3(blocks), dim3(256), 0, s, p.partials, p.out, ctot, p.r, r_pad, p.row_splits, p.out_j_major, p.scale);
        return check_launch("factor_reduce");
    }
    return 0;
}

int factor_grad(const FactorGradParams& p, int r_pad, int64_t experts, hipStream_t s) {
    // wide column blocks (256 contiguous bytes per row and workgroup) when they divide the segment
    return p.c % 128 == 0 ? launch_factor_grad<2>(p, r_pad, experts, s) : launch_factor_grad<1>(p, r_pad, experts, s);
}

}  // namespace ggq
