// Grouped bf16 (or fp16) matrix products over row groups, with no packed weight involved: what the reference takes from AITER's
// gmm / ptgmm (fast_moe_lora.py:22, 42-87) for its LoRA factors and for expert weights that have no packed kernel.
//
//   gmm:    out[i, :]  = lhs[i, :] . rhs[e]            for the rows i of group e   (rhs[e] is [k, n], either index contiguous)
//   ptgmm:  out[e]     = lhs[rows of e, :]^T . dy[rows of e, :]                    ([k, n] per group; empty groups give zeros)
//
// One kernel body serves both: a workgroup of four waves computes a 128 x 128 output tile, 32 contraction elements per
// step, each wave a 64 x 64 quarter as 4 x 4 MFMA 16x16x32 blocks with fp32 accumulators, one rounding to bf16 at the end.
// An operand whose contraction index is contiguous in memory is staged in LDS as [128][32] and read with 16-byte reads; one
// whose contraction index is the slow one is staged as loaded, [32][128], and transposed on the way out of LDS
// (ds_read_b64_tr_b16: within 16 lanes, lane L gets element L % 4 of the 8 bytes addressed by lanes L / 4 + 4 t).
// The next step's global loads are in flight while the current step's MFMAs run; two LDS buffers, one barrier per step.
// The column-side operand goes in as the MFMA's first operand, so a lane ends with four consecutive columns of one row
// (8-byte stores).  Any k and n; 16-byte loads when the leading dimensions and base addresses allow, element loads otherwise.
#include "common.h"
#include "launch.h"
#include "mmq_host.h"

namespace ggq {

namespace {

typedef short v4i16_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

// the two 16-bit element types of the entry points (the reference's wrapper admits both, fast_moe_lora.py:116-119)
template <bool F16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    if (F16) {
        const f16x2_t v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    return pack_bf16(lo, hi);
}
typedef __attribute__((address_space(3))) v4i16_t* lds_v4i16_ptr;

constexpr int kT = 128;          // output tile edge
constexpr int kStep = 32;        // contraction elements per step
constexpr int kPlainPitch = 40;  // [128][32] tile: 80-byte rows
constexpr int kTrPitch = 160;    // [32][128] tile: 320-byte rows (four consecutive rows' 32-byte pieces on distinct banks)
constexpr int kTileElems = 128 * kPlainPitch;  // = 32 * kTrPitch

__device__ __forceinline__ uint4 load8(const bf16_t* p, int valid, bool vec) {
    if (valid >= 8 && vec) return *(const uint4*)p;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (valid <= 0) return v;
    uint32_t e[8];
#pragma unroll
    for (int i = 0; i < 8; i++) e[i] = i < valid ? (uint32_t)p[i] : 0u;
    v.x = e[0] | (e[1] << 16), v.y = e[2] | (e[3] << 16), v.z = e[4] | (e[5] << 16), v.w = e[6] | (e[7] << 16);
    return v;
}

// One operand of the tile product: `outer` indexes the output (row or column of the tile), `t` the contraction.
struct Operand {
    const bf16_t* base;  // element (outer 0 of the tile, t 0 of the contraction range)
    int64_t ld;          // TR: elements between consecutive t; plain: between consecutive outer indices
    int outer_valid;     // outer indices of this tile that exist (<= 128)
    bool vec;
};

template <bool TR>
__device__ __forceinline__ void fetch(const Operand& o, int t0, int t_end, uint4 (&regs)[2]) {
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int id = threadIdx.x + 256 * u;
        if (TR) {
            const int t = id >> 4, ch = id & 15;
            const bool ok = t0 + t < t_end;
            regs[u] = load8(o.base + (int64_t)(ok ? t0 + t : 0) * o.ld + ch * 8, ok ? o.outer_valid - ch * 8 : 0, o.vec);
        } else {
            const int row = id >> 2, ch = id & 3;
            const bool ok = row < o.outer_valid;
            regs[u] = load8(o.base + (int64_t)(ok ? row : 0) * o.ld + t0 + ch * 8, ok ? t_end - (t0 + ch * 8) : 0, o.vec);
        }
    }
}

template <bool TR>
__device__ __forceinline__ void stage(bf16_t* tile, const uint4 (&regs)[2]) {
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int id = threadIdx.x + 256 * u;
        if (TR) *(uint4*)(tile + (id >> 4) * kTrPitch + (id & 15) * 8) = regs[u];
        else *(uint4*)(tile + (id >> 2) * kPlainPitch + (id & 3) * 8) = regs[u];
    }
}

// The MFMA operand of the 16 outer indices at `first`: lane (li, lq) gets contraction elements 8 lq .. 8 lq + 7 of outer index first + li.
template <bool TR>
__device__ __forceinline__ bf16x8_t operand(const bf16_t* tile, int first, int li, int lq) {
    if (TR) {
        const bf16_t* src = tile + (8 * lq + (li >> 2)) * kTrPitch + first + (li & 3) * 4;
        const v4i16_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)src);
        const v4i16_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(src + 4 * kTrPitch));
        return __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }
    return *(const bf16x8_t*)(tile + (first + li) * kPlainPitch + lq * 8);
}

// out[i, j] = sum over t in [0, t_len) of R(i, t) * C(j, t) for the tile's rows i < rows.outer_valid and columns j < cols.outer_valid.
template <bool ROWS_TR, bool COLS_TR, bool F16>
__device__ __forceinline__ void tile_product(const Operand& rows, const Operand& cols, int t_len, bf16_t* out, int64_t ld_out) {
    __shared__ __attribute__((aligned(16))) bf16_t r_t[2][kTileElems];
    __shared__ __attribute__((aligned(16))) bf16_t c_t[2][kTileElems];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int li = lane & 15, lq = lane >> 4;
    const int wi = wave >> 1, wj = wave & 1;
    f32x4_t acc[4][4];
#pragma unroll
    for (int ib = 0; ib < 4; ib++)
#pragma unroll
        for (int jb = 0; jb < 4; jb++) acc[ib][jb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    uint4 rr[2], cr[2];
    if (t_len > 0) {
        fetch<ROWS_TR>(rows, 0, t_len, rr);
        fetch<COLS_TR>(cols, 0, t_len, cr);
    }
    int buf = 0;
    for (int t0 = 0; t0 < t_len; t0 += kStep) {
        stage<ROWS_TR>(r_t[buf], rr);
        stage<COLS_TR>(c_t[buf], cr);
        // one barrier per step: the step after the next reuses this buffer, and a wave passes the next barrier only
        // after its reads of this one
        __syncthreads();
        if (t0 + kStep < t_len) {
            fetch<ROWS_TR>(rows, t0 + kStep, t_len, rr);
            fetch<COLS_TR>(cols, t0 + kStep, t_len, cr);
        }
        bf16x8_t c_op[4];
#pragma unroll
        for (int jb = 0; jb < 4; jb++) c_op[jb] = operand<COLS_TR>(c_t[buf], wj * 64 + jb * 16, li, lq);
#pragma unroll
        for (int ib = 0; ib < 4; ib++) {
            const bf16x8_t r_op = operand<ROWS_TR>(r_t[buf], wi * 64 + ib * 16, li, lq);
#pragma unroll
            for (int jb = 0; jb < 4; jb++) {
                if (F16) acc[ib][jb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, c_op[jb]), __builtin_bit_cast(f16x8_t, r_op), acc[ib][jb], 0, 0, 0);
                else acc[ib][jb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(c_op[jb], r_op, acc[ib][jb], 0, 0, 0);
            }
        }
        buf ^= 1;
    }
    // acc[ib][jb][v]: tile row wi*64 + ib*16 + li, tile column wj*64 + jb*16 + 4*lq + v
    const bool vec4 = (ld_out & 3) == 0 && (((uintptr_t)out & 7) == 0);
#pragma unroll
    for (int ib = 0; ib < 4; ib++) {
        const int i = wi * 64 + ib * 16 + li;
        if (i >= rows.outer_valid) continue;
#pragma unroll
        for (int jb = 0; jb < 4; jb++) {
            const int j = wj * 64 + jb * 16 + 4 * lq;
            bf16_t* dst = out + (int64_t)i * ld_out + j;
            if (vec4 && j + 3 < cols.outer_valid) {
                *(uint2*)dst = make_uint2(pack2<F16>(acc[ib][jb][0], acc[ib][jb][1]), pack2<F16>(acc[ib][jb][2], acc[ib][jb][3]));
            } else {
#pragma unroll
                for (int v = 0; v < 4; v++)
                    if (j + v < cols.outer_valid) dst[v] = (bf16_t)(pack2<F16>(acc[ib][jb][v], 0.0f) & 0xFFFFu);
            }
        }
    }
}

struct GroupedGemmParams {
    const bf16_t* lhs;    // [m, k]
    const bf16_t* rhs;    // gmm: [E][k][n] or [E][n][k]; ptgmm: dy [m, n]
    bf16_t* out;          // gmm: [m, n]; ptgmm: [E][k][n]
    const int32_t* plan;  // row_offsets[E + 2] (the last group holds the rows past every expert's), then tile_prefix[E + 2]
    int m, k, n, experts;
};

// Cumulative row offsets of the groups (clipped to m; negative sizes count as zero) and cumulative counts of their
// 128-row tiles.  A last, expert-less group takes the rows no group covers: gmm writes zeros there.
__global__ __launch_bounds__(256) void grouped_gemm_plan_kernel(const int32_t* group_sizes, int experts, int m, int32_t* plan) {
    __shared__ int64_t part_rows[256];
    __shared__ int part_tiles[256];
    int32_t* row_offsets = plan;
    int32_t* tile_prefix = plan + experts + 2;
    const int per = (experts + 255) / 256;
    const int e0 = min(experts, (int)threadIdx.x * per), e1 = min(experts, e0 + per);
    int64_t rows = 0;
    for (int e = e0; e < e1; e++) rows += max(group_sizes[e], 0);
    part_rows[threadIdx.x] = rows;
    __syncthreads();
    if (threadIdx.x == 0) {
        int64_t run = 0;
        for (int i = 0; i < 256; i++) {
            const int64_t v = part_rows[i];
            part_rows[i] = run;
            run += v;
        }
    }
    __syncthreads();
    int64_t at = part_rows[threadIdx.x];
    int tiles = 0;
    for (int e = e0; e < e1; e++) {  // first pass: this thread's tile count
        const int64_t b = min(at, (int64_t)m);
        at += max(group_sizes[e], 0);
        tiles += (int)((min(at, (int64_t)m) - b + kT - 1) / kT);
    }
    part_tiles[threadIdx.x] = tiles;
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int i = 0; i < 256; i++) {
            const int v = part_tiles[i];
            part_tiles[i] = run;
            run += v;
        }
    }
    __syncthreads();
    at = part_rows[threadIdx.x];
    int tile_at = part_tiles[threadIdx.x];
    for (int e = e0; e < e1; e++) {
        const int64_t b = min(at, (int64_t)m);
        row_offsets[e] = (int32_t)b;
        tile_prefix[e] = tile_at;
        at += max(group_sizes[e], 0);
        tile_at += (int)((min(at, (int64_t)m) - b + kT - 1) / kT);
    }
    if (threadIdx.x == 255) {  // (e1 == experts here: this thread's run ends the list)
        const int64_t b = min(at, (int64_t)m);
        row_offsets[experts] = (int32_t)b;
        tile_prefix[experts] = tile_at;
        row_offsets[experts + 1] = m;
        tile_prefix[experts + 1] = tile_at + (int)((m - b + kT - 1) / kT);
    }
}

template <bool RHS_TR, bool F16>
__global__ __launch_bounds__(256) void gmm_kernel(GroupedGemmParams p) {
    const int col_tiles = (p.n + kT - 1) / kT;
    const int rt = (int)(blockIdx.x / col_tiles), ct = (int)(blockIdx.x % col_tiles);
    const int32_t* row_offsets = p.plan;
    const int32_t* tile_prefix = p.plan + p.experts + 2;
    if (rt >= tile_prefix[p.experts + 1]) return;
    int lo = 0, hi = p.experts + 1;  // the group g with tile_prefix[g] <= rt < tile_prefix[g + 1]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tile_prefix[mid] <= rt) lo = mid;
        else hi = mid;
    }
    const int g = lo;
    const int r0 = row_offsets[g] + (rt - tile_prefix[g]) * kT;
    const int row_end = row_offsets[g + 1];
    const int c0 = ct * kT;
    Operand rows, cols;
    rows.base = p.lhs + (int64_t)r0 * p.k;
    rows.ld = p.k;
    rows.outer_valid = min(kT, row_end - r0);
    rows.vec = (p.k & 7) == 0 && (((uintptr_t)p.lhs & 15) == 0);
    const bool no_expert = g == p.experts;  // rows no group covers: zeros
    const bf16_t* rhs = p.rhs + (int64_t)(no_expert ? 0 : g) * p.k * p.n;
    cols.outer_valid = min(kT, p.n - c0);
    if (RHS_TR) {  // [k][n]
        cols.base = rhs + c0;
        cols.ld = p.n;
        cols.vec = (p.n & 7) == 0 && (((uintptr_t)p.rhs & 15) == 0);
    } else {  // [n][k]
        cols.base = rhs + (int64_t)c0 * p.k;
        cols.ld = p.k;
        cols.vec = (p.k & 7) == 0 && (((uintptr_t)p.rhs & 15) == 0);
    }
    tile_product<false, RHS_TR, F16>(rows, cols, no_expert ? 0 : p.k, p.out + (int64_t)r0 * p.n + c0, p.n);
}

template <bool F16>
__global__ __launch_bounds__(256) void ptgmm_kernel(GroupedGemmParams p) {
    const int col_tiles = (p.n + kT - 1) / kT, row_tiles = (p.k + kT - 1) / kT;
    const int per_expert = col_tiles * row_tiles;
    const int e = (int)(blockIdx.x / per_expert), rem = (int)(blockIdx.x % per_expert);
    const int kt = rem / col_tiles, ct = rem % col_tiles;
    const int row_begin = p.plan[e], row_end = p.plan[e + 1];
    Operand rows, cols;
    rows.base = p.lhs + (int64_t)row_begin * p.k + kt * kT;
    rows.ld = p.k;
    rows.outer_valid = min(kT, p.k - kt * kT);
    rows.vec = (p.k & 7) == 0 && (((uintptr_t)p.lhs & 15) == 0);
    cols.base = p.rhs + (int64_t)row_begin * p.n + ct * kT;
    cols.ld = p.n;
    cols.outer_valid = min(kT, p.n - ct * kT);
    cols.vec = (p.n & 7) == 0 && (((uintptr_t)p.rhs & 15) == 0);
    tile_product<true, true, F16>(rows, cols, row_end - row_begin, p.out + ((int64_t)e * p.k + kt * kT) * p.n + ct * kT, p.n);
}

int check_common(const char* what, const void* lhs, const void* rhs, const int32_t* group_sizes, const void* out, int64_t m, int64_t k, int64_t n,
                 int64_t experts, int64_t rhs_elems, int64_t out_elems, const void* ws, int64_t ws_bytes) {
    if (m < 0 || k < 0 || n < 0 || experts < 1)
        return set_error(GGQ_ERR_SHAPE, "%s: negative size or no expert (m=%lld k=%lld n=%lld experts=%lld)", what, (long long)m, (long long)k, (long long)n, (long long)experts);
    if (m > INT32_MAX - 2 * kT || k > INT32_MAX - 2 * kT || n > INT32_MAX - 2 * kT || experts > (1 << 24))
        return set_error(GGQ_ERR_SHAPE, "%s: a size exceeds the 32-bit index range of the kernels", what);
    if (!group_sizes || !ws || (!lhs && m * k > 0) || (!rhs && rhs_elems > 0) || (!out && out_elems > 0)) return set_error(GGQ_ERR_NULL, "%s: null pointer", what);
    if (((uintptr_t)lhs | (uintptr_t)rhs | (uintptr_t)out) & 1) return set_error(GGQ_ERR_ALIGN, "%s: matrices must be 2-byte aligned", what);
    if (ws_bytes < grouped_gemm_workspace_bytes(experts))
        return set_error(GGQ_ERR_WORKSPACE, "%s: workspace of %lld bytes, %lld needed", what, (long long)ws_bytes, (long long)grouped_gemm_workspace_bytes(experts));
    if (((uintptr_t)ws | (uintptr_t)group_sizes) & 3) return set_error(GGQ_ERR_ALIGN, "%s: group sizes and workspace must be 4-byte aligned", what);
    return GGQ_OK;
}

}  // namespace

int64_t grouped_gemm_workspace_bytes(int64_t experts) { return experts < 1 ? -1 : (2 * experts + 4) * (int64_t)sizeof(int32_t); }

int grouped_gemm(const void* lhs, const void* rhs, const int32_t* group_sizes, void* out, int64_t m, int64_t k, int64_t n, int64_t experts, int rhs_k_contiguous,
                 int is_f16, void* ws, int64_t ws_bytes, hipStream_t stream) {
    if (int rc = check_common("gmm", lhs, rhs, group_sizes, out, m, k, n, experts, experts * k * n, m * n, ws, ws_bytes)) return rc;
    if (m == 0 || n == 0) return GGQ_OK;
    GroupedGemmParams p;
    p.lhs = (const bf16_t*)lhs, p.rhs = (const bf16_t*)rhs, p.out = (bf16_t*)out, p.plan = (const int32_t*)ws;
    p.m = (int)m, p.k = (int)k, p.n = (int)n, p.experts = (int)experts;
    hipLaunchKernelGGL(grouped_gemm_plan_kernel, dim3(1), dim3(256), 0, stream, group_sizes, (int)experts, (int)m, (int32_t*)ws);
    if (int rc = check_launch("grouped_gemm_plan")) return rc;
    const int64_t row_tiles = (m + kT - 1) / kT + experts + 1, col_tiles = (n + kT - 1) / kT;
    if (row_tiles * col_tiles > INT32_MAX) return set_error(GGQ_ERR_SHAPE, "gmm: %lld tiles exceed the grid limit", (long long)(row_tiles * col_tiles));
    const dim3 grid((unsigned)(row_tiles * col_tiles));
    if (rhs_k_contiguous && is_f16) hipLaunchKernelGGL((gmm_kernel<false, true>), grid, dim3(256), 0, stream, p);
    else if (rhs_k_contiguous) hipLaunchKernelGGL((gmm_kernel<false, false>), grid, dim3(256), 0, stream, p);
    else if (is_f16) hipLaunchKernelGGL((gmm_kernel<true, true>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((gmm_kernel<true, false>), grid, dim3(256), 0, stream, p);
    return check_launch("gmm");
}

int grouped_gemm_transposed(const void* lhs, const void* grad_out, const int32_t* group_sizes, void* out, int64_t m, int64_t k, int64_t n, int64_t experts,
                            int is_f16, void* ws, int64_t ws_bytes, hipStream_t stream) {
    if (int rc = check_common("ptgmm", lhs, grad_out, group_sizes, out, m, k, n, experts, m * n, experts * k * n, ws, ws_bytes)) return rc;
    if (k == 0 || n == 0) return GGQ_OK;
    GroupedGemmParams p;
    p.lhs = (const bf16_t*)lhs, p.rhs = (const bf16_t*)grad_out, p.out = (bf16_t*)out, p.plan = (const int32_t*)ws;
    p.m = (int)m, p.k = (int)k, p.n = (int)n, p.experts = (int)experts;
    hipLaunchKernelGGL(grouped_gemm_plan_kernel, dim3(1), dim3(256), 0, stream, group_sizes, (int)experts, (int)m, (int32_t*)ws);
    if (int rc = check_launch("grouped_gemm_plan")) return rc;
    const int64_t tiles = experts * ((k + kT - 1) / kT) * ((n + kT - 1) / kT);
    if (tiles > INT32_MAX) return set_error(GGQ_ERR_SHAPE, "ptgmm: %lld tiles exceed the grid limit", (long long)tiles);
    if (is_f16) hipLaunchKernelGGL(ptgmm_kernel<true>, dim3((unsigned)tiles), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(ptgmm_kernel<false>, dim3((unsigned)tiles), dim3(256), 0, stream, p);
    return check_launch("ptgmm");
}

}  // namespace ggq
