// Tile kernel for matmuls against packed GGUF weights on gfx950 (MI355X, 64-wide waves, bf16 MFMA).
//
//   NT ("forward")    C[m, n] = sum_k A[m, k] * W[n, k]      A = activations [M, K]
//   NN ("grad input") C[m, k] = sum_n A[m, n] * W[n, k]      A = output cotangents [M, N]
//
// with W [N, K] stored as packed blocks, optionally two weight segments ("pair": gate and up), optional
// expert groups (row ranges of A/C that use different experts' W), and an optional rank-r LoRA term
// s * LA[m, :] . LB[col, :] folded in as extra contraction steps ahead of the main loop.
//
// One workgroup = 256 lanes (4 waves) computes a 128 x 256 tile of C.  Per contraction step of 64:
//   * the A tile (128 x 64 bf16) goes global -> registers -> LDS with 128-bit accesses;
//   * each lane loads the packed bytes of one 64-element segment of one W row into registers, unpacks
//     scales/mins/codebook in registers (blocks.h) and writes bf16 into the LDS W tile laid out
//     [output column][contraction]; in NN mode that write is the transposition (2-byte stores, 64 lanes
//     = 64 consecutive n);
//   * the four waves (2 x 2) each run 2 x 4 MFMA 32x32x16 blocks over the step (fp32 accumulators).
// Global loads for step i+1 are issued before the MFMAs of step i.  Rows past the end of a group and
// MFMA row blocks with no valid row are skipped, so ragged expert groups waste little.
#pragma once
#include "blocks.h"
#include "iq2xxs_grid.h"
#include "mmq_host.h"

namespace ggq {

static __device__ const uint64_t d_iq2xxs_grid_mm[256] = GGQ_IQ2XXS_GRID_INIT;

__device__ __forceinline__ uint4 zero4() { return make_uint4(0, 0, 0, 0); }

// 8 consecutive bf16 from a row, zero-filled past `valid` elements; `vec` = 16-byte access is legal.
__device__ __forceinline__ uint4 load8(const bf16_t* p, int valid, bool vec) {
    if (valid >= 8 && vec) return *(const uint4*)p;
    uint4 v = zero4();
    if (valid <= 0) return v;
    uint32_t e[8];
#pragma unroll
    for (int i = 0; i < 8; i++) e[i] = i < valid ? (uint32_t)p[i] : 0u;
    v.x = e[0] | (e[1] << 16), v.y = e[2] | (e[3] << 16), v.z = e[4] | (e[5] << 16), v.w = e[6] | (e[7] << 16);
    return v;
}

template <int QT, int MODE, int EPI>
__global__ __launch_bounds__(kThreads, 2) void mmq_tile_kernel(const MmqParams p) {
    using F = Fmt<QT>;
    __shared__ __attribute__((aligned(16))) bf16_t As[kBM * kLdsStride];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[kBN * kLdsStride];
    __shared__ uint2 grid_lds[QT == kIQ2_XXS ? 256 : 1];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const int lane_c = lane & 31, lane_h = lane >> 5;

    // ---- tile assignment.  Hardware deals consecutive workgroup ids round-robin over the 8 XCDs; remap
    // so that consecutive logical tiles (which share an A tile) land on one XCD and hit its L2.
    const int col_tiles = (MODE == kModeNT ? p.nseg : 1) * p.col_tiles_per_seg;
    const int grid_n = gridDim.x;
    const int per_xcd = (grid_n + 7) >> 3;
    const int logical = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    const int row_tile = logical / col_tiles, col_tile = logical - row_tile * col_tiles;
    int group = 0, row_begin, row_end;
    if (p.tiles) {
        if (row_tile >= p.max_row_tiles || row_tile >= *p.num_tiles) return;
        const TileDesc t = p.tiles[row_tile];
        group = t.group, row_begin = t.row_begin, row_end = t.row_end;
    } else {
        if (row_tile >= p.max_row_tiles) return;
        row_begin = row_tile * kBM;
        row_end = min(p.m, row_begin + kBM);
    }
    const int rows_valid = row_end - row_begin;  // 1..128
    const int64_t expert = p.expert_ids ? p.expert_ids[group] : 0;

    // column tile -> (segment, first output column inside the segment)
    const int seg_c = MODE == kModeNT ? col_tile / p.col_tiles_per_seg : 0;
    const int col0 = (col_tile - seg_c * p.col_tiles_per_seg) * kBN;
    const int out_cols = MODE == kModeNT ? p.n : p.k;       // output columns per segment
    const int contraction = MODE == kModeNT ? p.k : p.n;    // contraction length per segment

    if (QT == kIQ2_XXS) {
        const uint64_t g = d_iq2xxs_grid_mm[tid];
        grid_lds[tid] = make_uint2((uint32_t)g, (uint32_t)(g >> 32));
    }

    f32x16_t acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    const bool rb_live[2] = {wave_m * 64 < rows_valid, wave_m * 64 + 32 < rows_valid};

    auto mfma_step = [&](int ksub_count) {
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            if (kk < ksub_count) {
                const int koff = kk * 16 + lane_h * 8;
                bf16x8_t a[2], b[4];
#pragma unroll
                for (int rb = 0; rb < 2; rb++)
                    a[rb] = *(const bf16x8_t*)&As[(wave_m * 64 + rb * 32 + lane_c) * kLdsStride + koff];
#pragma unroll
                for (int cb = 0; cb < 4; cb++)
                    b[cb] = *(const bf16x8_t*)&Bs[(wave_n * 128 + cb * 32 + lane_c) * kLdsStride + koff];
#pragma unroll
                for (int rb = 0; rb < 2; rb++)
                    if (rb_live[rb]) {
#pragma unroll
                        for (int cb = 0; cb < 4; cb++)
                            acc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[rb], b[cb], acc[rb][cb], 0, 0, 0);
                    }
            }
        }
    };

    // ---- LoRA term first: acc = s * LA[rows, :r] . LB[cols, :r]^T, as r_pad/16 MFMA sub-steps.
    if (p.r_pad > 0) {
        const int chunks = p.r_pad >> 3;  // 16-byte chunks per row (r_pad % 16 == 0)
        for (int id = tid; id < kBM * 8; id += kThreads) {
            const int r = id >> 3, ch = id & 7;
            uint4 v = zero4();
            if (r < rows_valid && ch < chunks) v = *(const uint4*)(p.la + (int64_t)(row_begin + r) * p.r_pad + ch * 8);
            *(uint4*)&As[r * kLdsStride + ch * 8] = v;
        }
        const bf16_t* lb = p.lb + expert * p.lb_expert_elems + (int64_t)(seg_c * out_cols + col0) * p.r_pad;
        for (int id = tid; id < kBN * 8; id += kThreads) {
            const int cidx = id >> 3, ch = id & 7;
            uint4 v = zero4();
            if (col0 + cidx < out_cols && ch < chunks) v = *(const uint4*)(lb + (int64_t)cidx * p.r_pad + ch * 8);
            *(uint4*)&Bs[cidx * kLdsStride + ch * 8] = v;
        }
        __syncthreads();
        mfma_step(p.r_pad >> 4);
        const float s = p.lora_scale;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][j][e] *= s;
        __syncthreads();
    } else if (QT == kIQ2_XXS) {
        __syncthreads();  // codebook visible
    }

    // ---- main loop over the contraction, 64 per step
    const int total_steps = (MODE == kModeNN ? p.nseg : 1) * p.steps_per_seg;
    const bool a_vec = ((p.lda & 7) == 0) && ((((uintptr_t)p.a[0]) | ((uintptr_t)p.a[MODE == kModeNN && p.nseg > 1 ? 1 : 0])) & 15) == 0;

    uint4 a_reg[4];
    typename F::Raw w_reg;
    bool w_live = false;

    auto prefetch = [&](int step) {
        // which segment / contraction offset this step covers
        const int seg_k = MODE == kModeNN ? step / p.steps_per_seg : 0;
        const int kc0 = (step - seg_k * p.steps_per_seg) * kBK;
        const bf16_t* abase = p.a[MODE == kModeNN ? seg_k : 0];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int id = tid + i * kThreads;
            const int r = id >> 3, ch = id & 7;
            const int valid = r < rows_valid ? contraction - (kc0 + ch * 8) : 0;
            a_reg[i] = load8(abase + (int64_t)(row_begin + r) * p.lda + kc0 + ch * 8, valid, a_vec);
        }
        // weight segment owned by this lane
        int wrow, kseg;
        if (MODE == kModeNT) {
            wrow = col0 + tid;  // output column n
            kseg = step;
            w_live = wrow < p.n;
        } else {
            wrow = kc0 + lane;  // contraction row n
            kseg = (col0 >> 6) + wave;
            w_live = wrow < p.n && kseg * 64 < p.k;
        }
        if (w_live) {
            const int seg = MODE == kModeNT ? seg_c : seg_k;
            const uint8_t* row = p.w[seg] + expert * p.w_expert_bytes + (int64_t)wrow * p.w_row_bytes;
            F::load(w_reg, row, kseg);
        }
    };

    auto stage = [&](int step) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int id = tid + i * kThreads;
            *(uint4*)&As[(id >> 3) * kLdsStride + (id & 7) * 8] = a_reg[i];
        }
        uint32_t wv[32];
        if (w_live) {
            const int kseg = MODE == kModeNT ? step : (col0 >> 6) + wave;
            F::decode(w_reg, kseg, wv, grid_lds);
        } else {
#pragma unroll
            for (int i = 0; i < 32; i++) wv[i] = 0u;
        }
        if (MODE == kModeNT) {
#pragma unroll
            for (int i = 0; i < 8; i++)
                *(uint4*)&Bs[tid * kLdsStride + i * 8] = make_uint4(wv[4 * i], wv[4 * i + 1], wv[4 * i + 2], wv[4 * i + 3]);
        } else {
            // transpose: element e of this lane's row n is output column 64*wave + e, contraction index lane
#pragma unroll
            for (int e2 = 0; e2 < 32; e2++) {
                Bs[(wave * 64 + 2 * e2) * kLdsStride + lane] = (bf16_t)(wv[e2] & 0xFFFFu);
                Bs[(wave * 64 + 2 * e2 + 1) * kLdsStride + lane] = (bf16_t)(wv[e2] >> 16);
            }
        }
    };

    if (total_steps > 0) prefetch(0);
    for (int step = 0; step < total_steps; step++) {
        stage(step);
        __syncthreads();
        if (step + 1 < total_steps) prefetch(step + 1);
        mfma_step(4);
        __syncthreads();
    }

    // ---- epilogue.  acc[rb][cb][i]: row = 64*wave_m + 32*rb + 8*(i/4) + 4*lane_h + (i%4),
    //                                 col = 128*wave_n + 32*cb + lane_c
    const int col_base = col0 + wave_n * 128 + lane_c;
    if (EPI == kEpiStore || EPI == kEpiAccumF32 || EPI == kEpiCeGrad) {
#pragma unroll
        for (int rb = 0; rb < 2; rb++) {
            if (!rb_live[rb]) continue;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int r = wave_m * 64 + rb * 32 + (i >> 2) * 8 + lane_h * 4 + (i & 3);
                if (r >= rows_valid) continue;
                const int64_t grow = row_begin + r;
                float lse = 0.f, rs = 0.f;
                int64_t label = -1;
                if (EPI == kEpiCeGrad) {
                    lse = p.lse[grow];
                    rs = p.row_scale[grow];
                    label = p.labels[grow];
                }
#pragma unroll
                for (int cb = 0; cb < 4; cb++) {
                    const int col = col_base + cb * 32;
                    if (col >= out_cols) continue;
                    const float v = acc[rb][cb][i];
                    if (EPI == kEpiStore) {
                        ((bf16_t*)p.c[seg_c])[grow * p.ldc + col] = to_bf16(v);
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
        for (int rb = 0; rb < 2; rb++) {
            if (!rb_live[rb]) continue;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int r = wave_m * 64 + rb * 32 + (i >> 2) * 8 + lane_h * 4 + (i & 3);
                const bool row_ok = r < rows_valid;
                const int64_t grow = row_begin + (row_ok ? r : 0);
                const int64_t label = row_ok ? p.labels[grow] : -1;
                float v[4];
                float mx = -INFINITY;
#pragma unroll
                for (int cb = 0; cb < 4; cb++) {
                    const int col = col_base + cb * 32;
                    v[cb] = col < out_cols ? bf16_to_f32(to_bf16(acc[rb][cb][i])) : -INFINITY;
                    mx = fmaxf(mx, v[cb]);
                    if (row_ok && col < out_cols && (int64_t)(col + p.ce_col_offset) == label) p.ce_target_logit[grow] = v[cb];
                }
                // reduce over the 32 lanes that share this row (lanes with equal lane_h)
#pragma unroll
                for (int off = 16; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
                float sum = 0.f;
#pragma unroll
                for (int cb = 0; cb < 4; cb++) sum += v[cb] == -INFINITY ? 0.f : __expf(v[cb] - mx);
#pragma unroll
                for (int off = 16; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, 64);
                if (row_ok && lane_c == 0)
                    p.ce_partials[grow * p.ce_partials_ld + p.ce_partial_offset + col_tile * 2 + wave_n] = make_float2(mx, sum);
            }
        }
    }
}

}  // namespace ggq
