// Rank-r LoRA side kernels (r <= 64) around the packed-weight tile kernel.  All are HBM-bound streams
// over the activations; they use the 16x16x32 bf16 MFMA so the arithmetic never shows.
//
//   skinny_nt      out[m, j]  = sum_c In[m, c] * F[e][j, c]          (x A^T,  dY B via B^T)
//   factor_grad    G[e][c, j] = s * sum_{m in group e} In[m, c] * S[m, j]   (dB, dA; fixed order, no atomics)
//   pad / transpose helpers that lay the factors out [cols][r_pad] for the tile kernel.
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

// ---- out[m, 0..r_pad) = In[m, :] . F[e][0..r, :]^T ; one wave per 16 rows, 64-row tiles per workgroup.
// In may be two column segments (pair): contraction runs over seg 0 then seg 1, F rows are [r][nseg*C].
template <int JB>  // JB = r_pad / 16
__global__ __launch_bounds__(256) void skinny_nt_kernel(SkinnyNtParams p) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int group = 0, row_begin, row_end;
    if (p.tiles) {
        if ((int)blockIdx.x >= *p.num_tiles) return;
        const TileDesc t = p.tiles[blockIdx.x];
        group = t.group, row_begin = t.row_begin, row_end = t.row_end;
    } else {
        row_begin = blockIdx.x * 64;
        row_end = min(p.m, row_begin + 64);
    }
    const int64_t expert = p.expert_ids ? p.expert_ids[group] : 0;
    const int m0 = row_begin + wave * 16;
    if (m0 >= row_end) return;
    const int li = lane & 15, lq = lane >> 4;
    const int row = m0 + li;
    const bool row_ok = row < row_end;
    const bf16_t* f = p.f + expert * p.f_expert_elems;  // [r][ldf]
    f32x4_t acc[JB];
#pragma unroll
    for (int jb = 0; jb < JB; jb++) acc[jb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    for (int seg = 0; seg < p.nseg; seg++) {
        const bf16_t* in = p.in[seg] + (int64_t)row * p.ld_in;
        const bool vec = ((p.ld_in & 7) == 0) && (((uintptr_t)p.in[seg] & 15) == 0);
        const bool fvec = ((p.ldf & 7) == 0) && ((p.c & 7) == 0) && (((uintptr_t)p.f & 15) == 0);
        int c0 = 0;
        if (vec && fvec) {
            // aligned operands: four sub-steps per trip with every load issued ahead of the MFMAs (the
            // stream is latency-bound otherwise: one wave owns 16 rows)
            for (; c0 + 128 <= p.c; c0 += 128) {
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
        }
        for (; c0 < p.c; c0 += 32) {
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
    // acc[jb][v]: row = m0 + 4*lq + v, col = 16*jb + li
#pragma unroll
    for (int jb = 0; jb < JB; jb++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int r = m0 + 4 * lq + v;
            if (r < row_end) p.out[(int64_t)r * (JB * 16) + jb * 16 + li] = to_bf16(acc[jb][v]);
        }
}

// ---- G[e][c, j] = s * sum_m In[m, c] * S[m, j] over the rows of expert e.  One workgroup per
// (expert, 64 columns); each wave owns 16 columns; rows are consumed 32 at a time through LDS so the
// strided operands of the contraction over m become LDS gathers.  Experts without rows get zeros.
template <int JB>
__global__ __launch_bounds__(256) void factor_grad_kernel(FactorGradParams p) {
    __shared__ bf16_t in_t[32][64 + 2];
    __shared__ bf16_t s_t[32][JB * 16 + 2];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int blocks_per_seg = (p.c + 63) / 64;
    const int col_blocks = p.nseg * blocks_per_seg;
    const int e = blockIdx.x / col_blocks, cblk = blockIdx.x - e * col_blocks;
    const int seg = cblk / blocks_per_seg;
    const int c0 = (cblk - seg * blocks_per_seg) * 64;
    int row_begin = 0, row_end = p.m;
    if (p.ranges) {
        row_begin = p.ranges[2 * e];
        row_end = p.ranges[2 * e + 1];
    }
    const bf16_t* in = p.in[seg];
    const bool vec = ((p.ld_in & 7) == 0) && (((uintptr_t)in & 15) == 0);
    const int li = lane & 15, lq = lane >> 4;
    f32x4_t acc[JB];
#pragma unroll
    for (int jb = 0; jb < JB; jb++) acc[jb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    const int rp = JB * 16;
    for (int m0 = row_begin; m0 < row_end; m0 += 32) {
        {   // In tile: 32 rows x 64 cols = 256 chunks of 8
            const int r = threadIdx.x >> 3, ch = threadIdx.x & 7;
            const int cc = c0 + ch * 8;
            const uint4 v = load8g(in + (int64_t)(m0 + r) * p.ld_in + cc, m0 + r < row_end ? p.c - cc : 0, vec);
            uint32_t* d = (uint32_t*)&in_t[r][ch * 8];
            d[0] = v.x, d[1] = v.y, d[2] = v.z, d[3] = v.w;
        }
        for (int id = threadIdx.x; id < 32 * (rp / 8); id += 256) {
            const int r = id / (rp / 8), ch = id - r * (rp / 8);
            uint4 v = make_uint4(0, 0, 0, 0);
            if (m0 + r < row_end) v = *(const uint4*)(p.s + (int64_t)(m0 + r) * rp + ch * 8);
            uint32_t* d = (uint32_t*)&s_t[r][ch * 8];
            d[0] = v.x, d[1] = v.y, d[2] = v.z, d[3] = v.w;
        }
        __syncthreads();
        // A operand: row = column c (wave*16 + li), contraction m = 8*lq .. 8*lq+7
        uint32_t aw[4];
#pragma unroll
        for (int h = 0; h < 4; h++)
            aw[h] = (uint32_t)in_t[8 * lq + 2 * h][wave * 16 + li] | ((uint32_t)in_t[8 * lq + 2 * h + 1][wave * 16 + li] << 16);
        const bf16x8_t a = __builtin_bit_cast(bf16x8_t, make_uint4(aw[0], aw[1], aw[2], aw[3]));
#pragma unroll
        for (int jb = 0; jb < JB; jb++) {
            uint32_t bw[4];
#pragma unroll
            for (int h = 0; h < 4; h++)
                bw[h] = (uint32_t)s_t[8 * lq + 2 * h][jb * 16 + li] | ((uint32_t)s_t[8 * lq + 2 * h + 1][jb * 16 + li] << 16);
            acc[jb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8_t, make_uint4(bw[0], bw[1], bw[2], bw[3])), acc[jb], 0, 0, 0);
        }
        __syncthreads();
    }
    // acc[jb][v]: c = c0 + wave*16 + 4*lq + v, j = 16*jb + li
    bf16_t* out = p.out + (int64_t)e * p.out_expert_elems;
#pragma unroll
    for (int jb = 0; jb < JB; jb++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int c = c0 + wave * 16 + 4 * lq + v, j = jb * 16 + li;
            if (c < p.c && j < p.r) {
                const bf16_t val = to_bf16(acc[jb][v] * p.scale);
                const int64_t cg = (int64_t)seg * p.c + c;
                if (p.out_j_major) out[(int64_t)j * (p.nseg * p.c) + cg] = val;
                else out[cg * p.r + j] = val;
            }
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

int skinny_nt(const SkinnyNtParams& p, int r_pad, int grid_tiles, hipStream_t s) {
    if (grid_tiles <= 0) return 0;
    switch (r_pad / 16) {
        case 1: hipLaunchKernelGGL(skinny_nt_kernel<1>, dim3(grid_tiles), dim3(256), 0, s, p); break;
        case 2: hipLaunchKernelGGL(skinny_nt_kernel<2>, dim3(grid_tiles), dim3(256), 0, s, p); break;
        case 3: hipLaunchKernelGGL(skinny_nt_kernel<3>, dim3(grid_tiles), dim3(256), 0, s, p); break;
        case 4: hipLaunchKernelGGL(skinny_nt_kernel<4>, dim3(grid_tiles), dim3(256), 0, s, p); break;
        default: return set_error(GGQ_ERR_SHAPE, "LoRA rank must be between 1 and 64");
    }
    return check_launch("skinny_nt");
}

int factor_grad(const FactorGradParams& p, int r_pad, int64_t experts, hipStream_t s) {
    const int col_blocks = p.nseg * ((p.c + 63) / 64);
    const int64_t grid = experts * col_blocks;
    if (grid <= 0) return 0;
    if (grid > 0x7FFFFFFF) return set_error(GGQ_ERR_SHAPE, "factor_grad: grid too large");
    switch (r_pad / 16) {
        case 1: hipLaunchKernelGGL(factor_grad_kernel<1>, dim3((unsigned)grid), dim3(256), 0, s, p); break;
        case 2: hipLaunchKernelGGL(factor_grad_kernel<2>, dim3((unsigned)grid), dim3(256), 0, s, p); break;
        case 3: hipLaunchKernelGGL(factor_grad_kernel<3>, dim3((unsigned)grid), dim3(256), 0, s, p); break;
        case 4: hipLaunchKernelGGL(factor_grad_kernel<4>, dim3((unsigned)grid), dim3(256), 0, s, p); break;
        default: return set_error(GGQ_ERR_SHAPE, "LoRA rank must be between 1 and 64");
    }
    return check_launch("factor_grad");
}

}  // namespace ggq
