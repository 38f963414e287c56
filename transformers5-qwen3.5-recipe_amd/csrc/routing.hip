// Expert-sorted routing layout: stable counting sort of the flat top-k expert ids, per-expert offsets,
// row gather / weighted combine and their backward passes.  Pure integer and byte work, HBM-bound;
// everything is deterministic (no atomics) so a recomputed forward reproduces the same bits.
//
// Route r = token * k + rank.  permutation[s] = route at sorted position s; inverse[r] = s.
#include <mutex>

#include "common.h"
#include "launch.h"
#include "mmq_host.h"

namespace ggq {

constexpr int kChunk = 256;  // routes per workgroup in the sort

template <typename IdT>
__device__ __forceinline__ int load_id(const IdT* ids, int64_t i, int num_experts, int* bad) {
    int64_t v = (int64_t)ids[i];
    if (v < 0 || v >= num_experts) {
        *bad = 1;
        v = v < 0 ? 0 : num_experts - 1;
    }
    return (int)v;
}

// Pass 1: per chunk of 256 routes, the rank of every route among equal ids inside the chunk and the
// chunk's histogram.
template <typename IdT>
__global__ __launch_bounds__(kChunk) void route_rank_kernel(const IdT* ids, int64_t routes, int num_experts,
                                                            int* local_rank, int* chunk_hist, int* chunk_bad) {
    __shared__ int sid[kChunk];
    __shared__ int any_bad;
    const int tid = threadIdx.x;
    const int64_t i = (int64_t)blockIdx.x * kChunk + tid;
    int bad = 0;
    const int my = i < routes ? load_id(ids, i, num_experts, &bad) : -1;
    if (tid == 0) any_bad = 0;
    sid[tid] = my;
    __syncthreads();
    if (bad) any_bad = 1;  // benign race: every writer stores 1
    __syncthreads();
    if (tid == 0) chunk_bad[blockIdx.x] = any_bad;
    if (i < routes) {
        int rank = 0;
        for (int j = 0; j < tid; j++) rank += (sid[j] == my);
        local_rank[i] = rank;
    }
    for (int e = tid; e < num_experts; e += kChunk) {
        int c = 0;
        for (int j = 0; j < kChunk; j++) c += (sid[j] == e);
        chunk_hist[(int64_t)blockIdx.x * num_experts + e] = c;
    }
}

// Pass 1 for up to kWaveRankMaxExperts experts, in chunks of 1024 routes: the lanes of a wave that hold the same id find
// each other through one ballot per id bit (rank inside the wave = equal ids in lower lanes), the first of them leaves the
// wave's count in LDS, and a route's rank inside the chunk adds the counts of the waves before its own.  Same outputs as
// route_rank_kernel with four times fewer chunks for the scan pass to walk.
constexpr int kWaveChunk = 1024;
constexpr int kWaveRankMaxExperts = 1024;
template <typename IdT>
__global__ __launch_bounds__(kWaveChunk) void route_rank_wave_kernel(const IdT* ids, int64_t routes, int num_experts, int id_bits,
                                                                      int* local_rank, int* chunk_hist, int* chunk_bad) {
    extern __shared__ int wave_hist[];  // [16 waves][num_experts]
    __shared__ int any_bad;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < 16 * num_experts; i += kWaveChunk) wave_hist[i] = 0;
    if (tid == 0) any_bad = 0;
    __syncthreads();
    const int64_t i = (int64_t)blockIdx.x * kWaveChunk + tid;
    int bad = 0;
    const int my = i < routes ? load_id(ids, i, num_experts, &bad) : -1;  // (-1 has bit id_bits set: it matches no id)
    unsigned long long same = ~0ull;
    for (int b = 0; b <= id_bits; b++) {
        const int bit = (my >> b) & 1;
        const unsigned long long set = __ballot(bit);
        same &= bit ? set : ~set;
    }
    const int rank = __popcll(same & ((1ull << lane) - 1ull));
    if (my >= 0 && rank == 0) wave_hist[wave * num_experts + my] = __popcll(same);
    if (bad) any_bad = 1;  // benign race: every writer stores 1
    __syncthreads();
    if (i < routes) {
        int before = 0;
        for (int w = 0; w < wave; w++) before += wave_hist[w * num_experts + my];
        local_rank[i] = before + rank;
    }
    for (int e = tid; e < num_experts; e += kWaveChunk) {
        int c = 0;
#pragma unroll
        for (int w = 0; w < 16; w++) c += wave_hist[w * num_experts + e];
        chunk_hist[(int64_t)blockIdx.x * num_experts + e] = c;
    }
    if (tid == 0) chunk_bad[blockIdx.x] = any_bad;
}

// Pass 2 (one workgroup): turn chunk histograms into chunk bases, expert counts, cumulative end
// offsets and the compact list of active experts.
__global__ __launch_bounds__(256) void route_scan_kernel(int* chunk_hist, int chunks, int num_experts, int* counts,
                                                         int* end_offsets, int64_t* active_ids, int* active_end,
                                                         int* num_active, int* expert_base, const int* chunk_bad) {
    __shared__ int scan[256];
    __shared__ int totals[2][2][4];  // [round parity][rows / active][wave]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int carry_rows = 0, carry_active = 0;  // the same values in every thread
    int flip = 0;
    for (int e0 = 0; e0 < num_experts; e0 += 256) {
        const int e = e0 + tid;
        int total = 0;
        if (e < num_experts) {
            // sixty-four chunk counts are loaded together (one dependent load per chunk would cost a memory
            // round trip each); every count is replaced by the chunk's base inside the expert
            for (int c0 = 0; c0 < chunks; c0 += 64) {
                int v[64];
#pragma unroll
                for (int i = 0; i < 64; i++) v[i] = c0 + i < chunks ? chunk_hist[(int64_t)(c0 + i) * num_experts + e] : 0;
#pragma unroll
                for (int i = 0; i < 64; i++) {
                    if (c0 + i < chunks) chunk_hist[(int64_t)(c0 + i) * num_experts + e] = total;
                    total += v[i];
                }
            }
            counts[e] = total;
        }
        // prefix sums over the 256 experts of the round, rows and active flags together: a shuffle scan inside each
        // wave, the wave totals through LDS (one barrier; the next round writes the other half of `totals`)
        const int active = total > 0 ? 1 : 0;
        int rows_incl = total, act_incl = active;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int ur = __shfl_up(rows_incl, off, 64), ua = __shfl_up(act_incl, off, 64);
            if (lane >= off) rows_incl += ur, act_incl += ua;
        }
        if (lane == 63) totals[flip][0][wave] = rows_incl, totals[flip][1][wave] = act_incl;
        __syncthreads();
        int rows_before = 0, act_before = 0, round_rows = 0, round_active = 0;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const int tr = totals[flip][0][w], ta = totals[flip][1][w];
            if (w < wave) rows_before += tr, act_before += ta;
            round_rows += tr, round_active += ta;
        }
        if (e < num_experts) {
            const int end = carry_rows + rows_before + rows_incl;
            end_offsets[e] = end;
            expert_base[e] = end - total;
            if (active) {
                const int slot = carry_active + act_before + act_incl - 1;
                active_ids[slot] = e;
                active_end[slot] = end;
            }
        }
        carry_rows += round_rows, carry_active += round_active;
        flip ^= 1;
    }
    // status word pair: number of active experts, and whether any id was outside [0, num_experts)
    // (such ids are clamped so that no access leaves the buffers; the caller decides what to do).
    int bad = 0;
    for (int c = tid; c < chunks; c += 256) bad |= chunk_bad[c];
    const int wave_bad = __any(bad) ? 1 : 0;  // the vote is taken by all 64 lanes, outside any divergent branch
    if (lane == 0) scan[wave] = wave_bad;
    __syncthreads();
    if (tid == 0) {
        num_active[0] = carry_active;
        num_active[1] = scan[0] | scan[1] | scan[2] | scan[3];
    }
    // unused tail of the compact lists: repeat the total so that "offsets" stay monotone
    for (int s = carry_active + tid; s < num_experts; s += 256) {
        active_ids[s] = 0;
        active_end[s] = carry_rows;
    }
}

// Pass 3: scatter.
template <typename IdT>
__global__ __launch_bounds__(kWaveChunk) void route_scatter_kernel(const IdT* ids, int64_t routes, int num_experts,
                                                                   const int* local_rank, const int* chunk_base,
                                                                   const int* expert_base, int64_t* sorted_ids,
                                                                   int64_t* permutation, int64_t* inverse) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // a workgroup is one chunk of the rank pass
    if (i >= routes) return;
    int bad = 0;
    const int e = load_id(ids, i, num_experts, &bad);
    const int64_t pos = (int64_t)expert_base[e] + chunk_base[(int64_t)blockIdx.x * num_experts + e] + local_rank[i];
    sorted_ids[pos] = e;
    permutation[pos] = i;
    inverse[i] = pos;
}

// Passes 2 and 3 in one launch for the chunks of route_rank_wave_kernel (num_experts <= 1024 = one thread per expert):
// every workgroup sums the chunk histograms itself (one batch of loads per 64 chunks; the table is a few dozen KB and
// stays in L2) into the experts' totals and its own chunk's bases, scans the totals over the experts, and scatters its
// chunk; workgroup 0 also writes the counts, end offsets, active list and status words.  One dependent launch fewer than
// scan-then-scatter, and the scan no longer runs on a single compute unit while the others wait.
template <typename IdT>
__global__ __launch_bounds__(kWaveChunk) void route_scan_scatter_wave_kernel(const IdT* ids, int64_t routes, int num_experts, int chunks,
                                                                              const int* local_rank, const int* chunk_hist, const int* chunk_bad,
                                                                              int* counts, int* end_offsets, int64_t* active_ids, int* active_end,
                                                                              int* num_active, int64_t* sorted_ids, int64_t* permutation, int64_t* inverse) {
    __shared__ int base[kWaveRankMaxExperts];      // first sorted position of the expert, plus this chunk's base inside it
    __shared__ int wave_totals[2][16];
    __shared__ int any_bad;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int e = tid;
    int total = 0, before_chunk = 0;
    if (e < num_experts) {
        for (int c0 = 0; c0 < chunks; c0 += 64) {
            int v[64];
#pragma unroll
            for (int i = 0; i < 64; i++) v[i] = c0 + i < chunks ? chunk_hist[(int64_t)(c0 + i) * num_experts + e] : 0;
#pragma unroll
            for (int i = 0; i < 64; i++) {
                if (c0 + i < (int)blockIdx.x) before_chunk += v[i];
                total += v[i];
            }
        }
    }
    if (tid == 0) any_bad = 0;
    // inclusive scans over the experts (rows, and active flags for the compact list): shuffles inside a wave, wave totals through LDS
    const int active = total > 0 ? 1 : 0;
    int rows_incl = total, act_incl = active;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int ur = __shfl_up(rows_incl, off, 64), ua = __shfl_up(act_incl, off, 64);
        if (lane >= off) rows_incl += ur, act_incl += ua;
    }
    if (lane == 63) wave_totals[0][wave] = rows_incl, wave_totals[1][wave] = act_incl;
    __syncthreads();
    int rows_before = 0, act_before = 0, all_rows = 0, all_active = 0;
#pragma unroll
    for (int w = 0; w < 16; w++) {
        const int tr = wave_totals[0][w], ta = wave_totals[1][w];
        if (w < wave) rows_before += tr, act_before += ta;
        all_rows += tr, all_active += ta;
    }
    const int end = rows_before + rows_incl;
    if (e < num_experts) base[e] = end - total + before_chunk;
    if (blockIdx.x == 0) {
        if (e < num_experts) {
            counts[e] = total;
            end_offsets[e] = end;
            if (active) {
                const int slot = act_before + act_incl - 1;
                active_ids[slot] = e;
                active_end[slot] = end;
            }
        }
        int bad = 0;
        for (int c = tid; c < chunks; c += kWaveChunk) bad |= chunk_bad[c];
        if (bad) any_bad = 1;  // benign race: every writer stores 1
        // unused tail of the compact lists: repeat the total so that "offsets" stay monotone
        for (int sl = all_active + tid; sl < num_experts; sl += kWaveChunk) {
            active_ids[sl] = 0;
            active_end[sl] = all_rows;
        }
    }
    __syncthreads();
    if (blockIdx.x == 0 && tid == 0) {
        num_active[0] = all_active;
        num_active[1] = any_bad;
    }
    const int64_t i = (int64_t)blockIdx.x * kWaveChunk + tid;
    if (i >= routes) return;
    int bad = 0;
    const int id = load_id(ids, i, num_experts, &bad);
    const int64_t pos = (int64_t)base[id] + local_rank[i];
    sorted_ids[pos] = id;
    permutation[pos] = i;
    inverse[i] = pos;
}

int64_t route_plan_workspace_bytes(int64_t routes, int num_experts) {
    const int64_t chunks = (routes + kChunk - 1) / kChunk;
    return (routes + chunks * num_experts + num_experts + chunks + 4) * (int64_t)sizeof(int);
}

int route_plan(const void* topk_ids, int ids_are_int64, int64_t tokens, int top_k, int num_experts,
               int64_t* sorted_ids, int64_t* permutation, int64_t* inverse, int* counts, int* end_offsets,
               int64_t* active_ids, int* active_end, int* num_active, void* ws, int64_t ws_bytes, hipStream_t s) {
    const int64_t routes = tokens * top_k;
    if (tokens < 0 || top_k <= 0 || num_experts <= 0) return set_error(GGQ_ERR_SHAPE, "route_plan: bad shape");
    if (routes >= (int64_t)1 << 31) return set_error(GGQ_ERR_SHAPE, "route_plan: more than 2^31 routes");
    if (ws_bytes < route_plan_workspace_bytes(routes, num_experts)) return set_error(GGQ_ERR_WORKSPACE, "route_plan: workspace too small");
    // chunks of 1024 routes ranked by wave ballots when the per-wave counts fit in LDS, else chunks of 256 ranked by comparison
    const bool by_wave = num_experts <= kWaveRankMaxExperts;
    const int chunk = by_wave ? kWaveChunk : kChunk;
    const int chunks = (int)((routes + chunk - 1) / chunk);
    int* local_rank = (int*)ws;
    int* chunk_hist = local_rank + routes;
    int* expert_base = chunk_hist + (int64_t)chunks * num_experts;
    int* chunk_bad = expert_base + num_experts;
    if (chunks > 0 && by_wave) {
        int id_bits = 0;
        while ((1 << id_bits) < num_experts) id_bits++;
        const int lds = 16 * num_experts * (int)sizeof(int);
        static LdsLimit lim64, lim32;
        if (int rc = raise_lds_limit(ids_are_int64 ? lim64 : lim32, ids_are_int64 ? (const void*)route_rank_wave_kernel<int64_t> : (const void*)route_rank_wave_kernel<int32_t>, lds, "route_plan")) return rc;
        if (ids_are_int64)
            hipLaunchKernelGGL(route_rank_wave_kernel<int64_t>, dim3(chunks), dim3(kWaveChunk), lds, s, (const int64_t*)topk_ids, routes, num_experts, id_bits, local_rank, chunk_hist, chunk_bad);
        else
            hipLaunchKernelGGL(route_rank_wave_kernel<int32_t>, dim3(chunks), dim3(kWaveChunk), lds, s, (const int32_t*)topk_ids, routes, num_experts, id_bits, local_rank, chunk_hist, chunk_bad);
    } else if (chunks > 0) {
        if (ids_are_int64)
            hipLaunchKernelGGL(route_rank_kernel<int64_t>, dim3(chunks), dim3(kChunk), 0, s, (const int64_t*)topk_ids, routes, num_experts, local_rank, chunk_hist, chunk_bad);
        else
            hipLaunchKernelGGL(route_rank_kernel<int32_t>, dim3(chunks), dim3(kChunk), 0, s, (const int32_t*)topk_ids, routes, num_experts, local_rank, chunk_hist, chunk_bad);
    }
    if (chunks > 0 && by_wave) {
        if (ids_are_int64)
            hipLaunchKernelGGL(route_scan_scatter_wave_kernel<int64_t>, dim3(chunks), dim3(kWaveChunk), 0, s, (const int64_t*)topk_ids, routes, num_experts, chunks, local_rank,
                               chunk_hist, chunk_bad, counts, end_offsets, active_ids, active_end, num_active, sorted_ids, permutation, inverse);
        else
            hipLaunchKernelGGL(route_scan_scatter_wave_kernel<int32_t>, dim3(chunks), dim3(kWaveChunk), 0, s, (const int32_t*)topk_ids, routes, num_experts, chunks, local_rank,
                               chunk_hist, chunk_bad, counts, end_offsets, active_ids, active_end, num_active, sorted_ids, permutation, inverse);
        return check_launch("route_plan");
    }
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(256), 0, s, chunk_hist, chunks, num_experts, counts, end_offsets, active_ids, active_end, num_active, expert_base, chunk_bad);
    if (chunks > 0) {
        if (ids_are_int64)
            hipLaunchKernelGGL(route_scatter_kernel<int64_t>, dim3(chunks), dim3(chunk), 0, s, (const int64_t*)topk_ids, routes, num_experts, local_rank, chunk_hist, expert_base, sorted_ids, permutation, inverse);
        else
            hipLaunchKernelGGL(route_scatter_kernel<int32_t>, dim3(chunks), dim3(chunk), 0, s, (const int32_t*)topk_ids, routes, num_experts, local_rank, chunk_hist, expert_base, sorted_ids, permutation, inverse);
    }
    return check_launch("route_plan");
}

// ------------------------------------------------------------------------------------------------
// The same plan without a caller workspace: the sort's scratch (per-route ranks, per-chunk histograms, expert
// bases, per-chunk flags) lives in a file-scope device array.  Every GPU the library runs on holds its own copy
// of the array at its own address until the process ends; the address is looked up once per device.
constexpr int64_t kStaticPlanMaxRoutes = 1 << 18;  // 262144 routes (e.g. 32768 tokens x top-8)
constexpr int kStaticPlanMaxExperts = 256;
constexpr int64_t kStaticPlanInts =
    kStaticPlanMaxRoutes + (kStaticPlanMaxRoutes / kChunk) * kStaticPlanMaxExperts + kStaticPlanMaxExperts + kStaticPlanMaxRoutes / kChunk + 4;
static __device__ __align__(256) int scratch[kStaticPlanInts];  // 2.1 MB

constexpr int kMaxDevices = 64;
static int* scratch_ptr[kMaxDevices];  // device address of `scratch` on each device (null: not looked up yet)
static std::mutex scratch_lock;

// Device address of this device's copy of `scratch`.  The array's name is only a host-side handle: kernels and
// copies take the address returned here.
static int static_scratch(int** out) {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return set_error(GGQ_ERR_RUNTIME, "route_plan_static: no current device");
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (!scratch_ptr[device]) {
        int* p = nullptr;
        const hipError_t err = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess || !p) return set_error(GGQ_ERR_RUNTIME, "route_plan_static: hipGetSymbolAddress failed: %s", hipGetErrorString(err));
        scratch_ptr[device] = p;
    }
    *out = scratch_ptr[device];
    return GGQ_OK;
}

int route_plan_static(const void* topk_ids, int ids_are_int64, int64_t tokens, int top_k, int num_experts,
                      int64_t* sorted_ids, int64_t* permutation, int64_t* inverse, int* counts, int* end_offsets,
                      int64_t* active_ids, int* active_end, int* num_active, hipStream_t s) {
    if (tokens < 0 || top_k <= 0 || num_experts <= 0) return set_error(GGQ_ERR_SHAPE, "route_plan_static: bad shape");
    if (tokens > kStaticPlanMaxRoutes || tokens * top_k > kStaticPlanMaxRoutes || num_experts > kStaticPlanMaxExperts)
        return set_error(GGQ_ERR_SHAPE, "route_plan_static: at most %lld routes and %d experts fit the built-in scratch array, got %lld routes and %d experts (use route_plan with a workspace)",
                         (long long)kStaticPlanMaxRoutes, kStaticPlanMaxExperts, (long long)(tokens * top_k), num_experts);
    int* ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    // nothing in the scratch has to start at zero: every word the scan and scatter passes read is written by the
    // rank pass of the same call
    return route_plan(topk_ids, ids_are_int64, tokens, top_k, num_experts, sorted_ids, permutation, inverse, counts, end_offsets, active_ids,
                      active_end, num_active, ws, kStaticPlanInts * (int64_t)sizeof(int), s);
}

// ------------------------------------------------------------------------------------------------
// gather forward: selected[s, :] = hidden[permutation[s] / k, :]   (16-byte copies)
__global__ __launch_bounds__(256) void route_gather_fwd_kernel(const uint4* hidden, const int64_t* permutation, uint4* selected,
                                                               int64_t routes, int top_k, int chunks_per_row) {
    const int64_t total = routes * chunks_per_row;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t srow = i / chunks_per_row;
        const int ch = (int)(i - srow * chunks_per_row);
        const int64_t token = permutation[srow] / top_k;
        selected[i] = hidden[token * chunks_per_row + ch];
    }
}

// gather backward: grad_hidden[t] = sum over the token's routes, visited in ascending sorted position,
// with the running sum rounded to bf16 after every add.
template <int MAXK>
__global__ __launch_bounds__(256) void route_gather_bwd_kernel(const uint4* grad_selected, const int64_t* inverse, uint4* grad_hidden,
                                                               int64_t tokens, int top_k, int chunks_per_row) {
    const int64_t total = tokens * chunks_per_row;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / chunks_per_row;
        const int ch = (int)(i - t * chunks_per_row);
        int64_t pos[MAXK];
#pragma unroll
        for (int j = 0; j < MAXK; j++) pos[j] = j < top_k ? inverse[t * top_k + j] : INT64_MAX;
        // insertion sort (k is tiny)
#pragma unroll
        for (int a = 1; a < MAXK; a++)
#pragma unroll
            for (int b = a; b > 0; b--)
                if (pos[b] < pos[b - 1]) {
                    const int64_t tmp = pos[b];
                    pos[b] = pos[b - 1];
                    pos[b - 1] = tmp;
                }
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] = 0.f;
#pragma unroll
        for (int j = 0; j < MAXK; j++) {
            if (j < top_k) {
                const uint4 g = grad_selected[pos[j] * chunks_per_row + ch];
                const uint32_t w[4] = {g.x, g.y, g.z, g.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    acc[2 * e] = bf16_to_f32(to_bf16(acc[2 * e] + bf16_lo(w[e])));
                    acc[2 * e + 1] = bf16_to_f32(to_bf16(acc[2 * e + 1] + bf16_hi(w[e])));
                }
            }
        }
        uint4 o;
        o.x = pack_bf16(acc[0], acc[1]), o.y = pack_bf16(acc[2], acc[3]);
        o.z = pack_bf16(acc[4], acc[5]), o.w = pack_bf16(acc[6], acc[7]);
        grad_hidden[i] = o;
    }
}

__device__ __forceinline__ float load_weight(const void* w, int w_is_bf16, int64_t i) {
    const float v = w_is_bf16 ? bf16_to_f32(((const bf16_t*)w)[i]) : ((const float*)w)[i];
    return bf16_to_f32(to_bf16(v));  // the layout applies routing weights at bf16 precision
}

// combine forward: out[t] = bf16( sum_rank fp32(o[inverse[t*k+rank]]) * w[t, rank] ), ranks in order.
__global__ __launch_bounds__(256) void route_combine_fwd_kernel(const uint4* expert_out, const void* weights, int w_is_bf16,
                                                                const int64_t* inverse, uint4* out, int64_t tokens, int top_k,
                                                                int chunks_per_row) {
    const int64_t total = tokens * chunks_per_row;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / chunks_per_row;
        const int ch = (int)(i - t * chunks_per_row);
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] = 0.f;
        for (int rank = 0; rank < top_k; rank++) {
            const int64_t route = t * top_k + rank;
            const float w = load_weight(weights, w_is_bf16, route);
            const uint4 g = expert_out[inverse[route] * chunks_per_row + ch];
            const uint32_t v[4] = {g.x, g.y, g.z, g.w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                acc[2 * e] = fmaf(bf16_lo(v[e]), w, acc[2 * e]);
                acc[2 * e + 1] = fmaf(bf16_hi(v[e]), w, acc[2 * e + 1]);
            }
        }
        uint4 o;
        o.x = pack_bf16(acc[0], acc[1]), o.y = pack_bf16(acc[2], acc[3]);
        o.z = pack_bf16(acc[4], acc[5]), o.w = pack_bf16(acc[6], acc[7]);
        out[i] = o;
    }
}

// combine backward: one wave per sorted route.  dO[s] = bf16(g[t] * w); dW[route] = sum_h g * o in
// fp32 with a fixed lane-strided order and a butterfly reduction.
__global__ __launch_bounds__(256) void route_combine_bwd_kernel(const uint4* expert_out, const void* weights, int w_is_bf16,
                                                                const int64_t* permutation, const uint4* grad_out, uint4* grad_expert_out,
                                                                void* grad_weights, int64_t routes, int top_k, int chunks_per_row) {
    const int lane = threadIdx.x & 63;
    const int64_t s = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (s >= routes) return;
    const int64_t route = permutation[s];
    const int64_t t = route / top_k;
    const float w = load_weight(weights, w_is_bf16, route);
    float dot = 0.f;
    for (int ch = lane; ch < chunks_per_row; ch += 64) {
        const uint4 g = grad_out[t * chunks_per_row + ch];
        const uint4 o = expert_out[s * chunks_per_row + ch];
        const uint32_t gv[4] = {g.x, g.y, g.z, g.w}, ov[4] = {o.x, o.y, o.z, o.w};
        uint32_t r[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float g0 = bf16_lo(gv[e]), g1 = bf16_hi(gv[e]);
            r[e] = pack_bf16(g0 * w, g1 * w);
            dot = fmaf(g0, bf16_lo(ov[e]), dot);
            dot = fmaf(g1, bf16_hi(ov[e]), dot);
        }
        if (grad_expert_out) grad_expert_out[s * chunks_per_row + ch] = make_uint4(r[0], r[1], r[2], r[3]);
    }
    if (grad_weights) {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) dot += __shfl_xor(dot, off, 64);
        if (lane == 0) {
            if (w_is_bf16) ((bf16_t*)grad_weights)[route] = to_bf16(dot);
            else ((float*)grad_weights)[route] = dot;
        }
    }
}

static inline unsigned stream_grid(int64_t items) {
    int64_t g = (items + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 256 * 64 ? 256 * 64 : g));
}

static int check_rows(const void* a, const void* b, int hidden, const char* what) {
    if (hidden <= 0 || hidden % 8) return set_error(GGQ_ERR_SHAPE, "%s: hidden size must be a positive multiple of 8", what);
    if (((uintptr_t)a | (uintptr_t)b) & 15) return set_error(GGQ_ERR_ALIGN, "%s: row buffers must be 16-byte aligned", what);
    return GGQ_OK;
}

int route_gather_fwd(const void* hidden, const int64_t* permutation, void* selected, int64_t tokens, int top_k, int hidden_dim, hipStream_t s) {
    if (int rc = check_rows(hidden, selected, hidden_dim, "route_gather_forward")) return rc;
    const int64_t routes = tokens * top_k;
    if (routes == 0) return GGQ_OK;
    hipLaunchKernelGGL(route_gather_fwd_kernel, dim3(stream_grid(routes * (hidden_dim / 8))), dim3(256), 0, s, (const uint4*)hidden, permutation, (uint4*)selected, routes, top_k, hidden_dim / 8);
    return check_launch("route_gather_forward");
}

int route_gather_bwd(const void* grad_selected, const int64_t* inverse, void* grad_hidden, int64_t tokens, int top_k, int hidden_dim, hipStream_t s) {
    if (int rc = check_rows(grad_selected, grad_hidden, hidden_dim, "route_gather_backward")) return rc;
    if (tokens == 0) return GGQ_OK;
    const unsigned grid = stream_grid(tokens * (hidden_dim / 8));
    if (top_k <= 8)
        hipLaunchKernelGGL(route_gather_bwd_kernel<8>, dim3(grid), dim3(256), 0, s, (const uint4*)grad_selected, inverse, (uint4*)grad_hidden, tokens, top_k, hidden_dim / 8);
    else if (top_k <= 16)
        hipLaunchKernelGGL(route_gather_bwd_kernel<16>, dim3(grid), dim3(256), 0, s, (const uint4*)grad_selected, inverse, (uint4*)grad_hidden, tokens, top_k, hidden_dim / 8);
    else
        return set_error(GGQ_ERR_SHAPE, "route_gather_backward: top_k above 16 is not supported");
    return check_launch("route_gather_backward");
}

int route_combine_fwd(const void* expert_out, const void* weights, int w_is_bf16, const int64_t* inverse, void* out, int64_t tokens, int top_k, int hidden_dim, hipStream_t s) {
    if (int rc = check_rows(expert_out, out, hidden_dim, "route_combine_forward")) return rc;
    if (tokens == 0) return GGQ_OK;
    hipLaunchKernelGGL(route_combine_fwd_kernel, dim3(stream_grid(tokens * (hidden_dim / 8))), dim3(256), 0, s, (const uint4*)expert_out, weights, w_is_bf16, inverse, (uint4*)out, tokens, top_k, hidden_dim / 8);
    return check_launch("route_combine_forward");
}

int route_combine_bwd(const void* expert_out, const void* weights, int w_is_bf16, const int64_t* permutation, const void* grad_out, void* grad_expert_out, void* grad_weights, int64_t tokens, int top_k, int hidden_dim, hipStream_t s) {
    if (int rc = check_rows(expert_out, grad_out, hidden_dim, "route_combine_backward")) return rc;
    if (grad_expert_out && ((uintptr_t)grad_expert_out & 15)) return set_error(GGQ_ERR_ALIGN, "route_combine_backward: output must be 16-byte aligned");
    const int64_t routes = tokens * top_k;
    if (routes == 0) return GGQ_OK;
    const int64_t grid = (routes + 3) / 4;
    if (grid > 0x7FFFFFFF) return set_error(GGQ_ERR_SHAPE, "route_combine_backward: too many routes");
    hipLaunchKernelGGL(route_combine_bwd_kernel, dim3((unsigned)grid), dim3(256), 0, s, (const uint4*)expert_out, weights, w_is_bf16, permutation, (const uint4*)grad_out, (uint4*)grad_expert_out, grad_weights, routes, top_k, hidden_dim / 8);
    return check_launch("route_combine_backward");
}

// ------------------------------------------------------------------------------------------------
// SiLU-gated product of the expert FFN: h = silu(gate) * up, and its backward.
// limit > 0 selects the clamped form: the gate is cut off above `limit`, up is kept within [-limit, limit].
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const uint4* gate, const uint4* up, uint4* h, int64_t chunks, float limit) {
    const float hi = limit > 0.0f ? limit : INFINITY;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < chunks; i += (int64_t)gridDim.x * 256) {
        const uint4 g = gate[i], u = up[i];
        const uint32_t gv[4] = {g.x, g.y, g.z, g.w}, uv[4] = {u.x, u.y, u.z, u.w};
        uint32_t r[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float g0 = fminf(bf16_lo(gv[e]), hi), g1 = fminf(bf16_hi(gv[e]), hi);
            const float u0 = fminf(fmaxf(bf16_lo(uv[e]), -hi), hi), u1 = fminf(fmaxf(bf16_hi(uv[e]), -hi), hi);
            const float s0 = g0 / (1.0f + __expf(-g0)), s1 = g1 / (1.0f + __expf(-g1));
            r[e] = pack_bf16(s0 * u0, s1 * u1);
        }
        h[i] = make_uint4(r[0], r[1], r[2], r[3]);
    }
}

// (clamped form: no gradient flows into a gate above the limit or an up outside [-limit, limit])
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const uint4* gate, const uint4* up, const uint4* dh, uint4* dgate, uint4* dup, int64_t chunks, float limit) {
    const float hi = limit > 0.0f ? limit : INFINITY;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < chunks; i += (int64_t)gridDim.x * 256) {
        const uint4 g = gate[i], u = up[i], d = dh[i];
        const uint32_t gv[4] = {g.x, g.y, g.z, g.w}, uv[4] = {u.x, u.y, u.z, u.w}, dv[4] = {d.x, d.y, d.z, d.w};
        uint32_t rg[4], ru[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float og[2], ou[2];
#pragma unroll
            for (int hlf = 0; hlf < 2; hlf++) {
                const float xr = hlf ? bf16_hi(gv[e]) : bf16_lo(gv[e]);
                const float ur = hlf ? bf16_hi(uv[e]) : bf16_lo(uv[e]);
                const float dd = hlf ? bf16_hi(dv[e]) : bf16_lo(dv[e]);
                const float x = fminf(xr, hi), uu = fminf(fmaxf(ur, -hi), hi);
                const float sig = 1.0f / (1.0f + __expf(-x));
                og[hlf] = xr <= hi ? dd * uu * (sig * (1.0f + x * (1.0f - sig))) : 0.0f;
                ou[hlf] = (ur >= -hi && ur <= hi) ? dd * x * sig : 0.0f;
            }
            rg[e] = pack_bf16(og[0], og[1]);
            ru[e] = pack_bf16(ou[0], ou[1]);
        }
        dgate[i] = make_uint4(rg[0], rg[1], rg[2], rg[3]);
        dup[i] = make_uint4(ru[0], ru[1], ru[2], ru[3]);
    }
}

// Backward of h = silu(gate) * up for rows whose cotangent arrives without its routing weight: one wave per expert-sorted
// row s, route = permutation[s], w = weights[route].  With d = the unweighted cotangent row, the gradient of the weight is
// sum_j d[j] * h[j] (h recomputed exactly as the forward rounds it), accumulated in fp32 in a fixed lane-strided order and
// reduced by a butterfly, and dgate / dup are those of the cotangent w * d (the product is not rounded in between).
__global__ __launch_bounds__(256) void swiglu_bwd_routed_kernel(const uint4* gate, const uint4* up, const uint4* dh, const void* weights,
                                                                int w_is_bf16, const int64_t* permutation, uint4* dgate, uint4* dup,
                                                                void* grad_weights, int64_t routes, int chunks_per_row, float limit) {
    const float hi = limit > 0.0f ? limit : INFINITY;
    const int lane = threadIdx.x & 63;
    const int64_t s = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (s >= routes) return;
    // the row's first chunks are requested before the route's weight, which hangs on two dependent loads
    const bool first = lane < chunks_per_row;
    const int64_t i0 = s * chunks_per_row + (first ? lane : 0);
    uint4 g = gate[i0], u = up[i0], d = dh[i0];
    const int64_t route = permutation[s];
    const float w = load_weight(weights, w_is_bf16, route);
    float dot = 0.f;
    for (int ch = lane; ch < chunks_per_row; ch += 64) {
        const int64_t i = s * chunks_per_row + ch;
        if (ch != lane) g = gate[i], u = up[i], d = dh[i];
        const uint32_t gv[4] = {g.x, g.y, g.z, g.w}, uv[4] = {u.x, u.y, u.z, u.w}, dv[4] = {d.x, d.y, d.z, d.w};
        uint32_t rg[4], ru[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float og[2], ou[2], hh[2], dd[2];
#pragma unroll
            for (int hlf = 0; hlf < 2; hlf++) {
                const float xr = hlf ? bf16_hi(gv[e]) : bf16_lo(gv[e]);
                const float ur = hlf ? bf16_hi(uv[e]) : bf16_lo(uv[e]);
                dd[hlf] = hlf ? bf16_hi(dv[e]) : bf16_lo(dv[e]);
                const float x = fminf(xr, hi), uu = fminf(fmaxf(ur, -hi), hi);
                const float den = 1.0f + __expf(-x);
                hh[hlf] = (x / den) * uu;  // the forward's expression, rounded below as the forward stores it
                const float sig = 1.0f / den;
                const float dw = dd[hlf] * w;
                og[hlf] = xr <= hi ? dw * uu * (sig * (1.0f + x * (1.0f - sig))) : 0.0f;
                ou[hlf] = (ur >= -hi && ur <= hi) ? dw * x * sig : 0.0f;
            }
            const uint32_t hb = pack_bf16(hh[0], hh[1]);
            dot = fmaf(dd[0], bf16_lo(hb), dot);
            dot = fmaf(dd[1], bf16_hi(hb), dot);
            rg[e] = pack_bf16(og[0], og[1]);
            ru[e] = pack_bf16(ou[0], ou[1]);
        }
        dgate[i] = make_uint4(rg[0], rg[1], rg[2], rg[3]);
        dup[i] = make_uint4(ru[0], ru[1], ru[2], ru[3]);
    }
    if (grad_weights) {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) dot += __shfl_xor(dot, off, 64);
        if (lane == 0) {
            if (w_is_bf16) ((bf16_t*)grad_weights)[route] = to_bf16(dot);
            else ((float*)grad_weights)[route] = dot;
        }
    }
}

int swiglu_bwd_routed(const void* gate, const void* up, const void* dh, const void* weights, int w_is_bf16, const int64_t* permutation,
                      void* dgate, void* dup, void* grad_weights, int64_t routes, int inter, float limit, hipStream_t s) {
    if (inter <= 0 || inter % 8) return set_error(GGQ_ERR_SHAPE, "swiglu_backward_routed: row width must be a positive multiple of 8");
    if (((uintptr_t)gate | (uintptr_t)up | (uintptr_t)dh | (uintptr_t)dgate | (uintptr_t)dup) & 15) return set_error(GGQ_ERR_ALIGN, "swiglu_backward_routed: buffers must be 16-byte aligned");
    if (routes == 0) return GGQ_OK;
    const int64_t grid = (routes + 3) / 4;
    if (grid > 0x7FFFFFFF) return set_error(GGQ_ERR_SHAPE, "swiglu_backward_routed: too many routes");
    hipLaunchKernelGGL(swiglu_bwd_routed_kernel, dim3((unsigned)grid), dim3(256), 0, s, (const uint4*)gate, (const uint4*)up, (const uint4*)dh, weights,
                       w_is_bf16, permutation, (uint4*)dgate, (uint4*)dup, grad_weights, routes, inter / 8, limit);
    return check_launch("swiglu_backward_routed");
}

int swiglu_fwd(const void* gate, const void* up, void* h, int64_t elems, float limit, hipStream_t s) {
    if (elems % 8) return set_error(GGQ_ERR_SHAPE, "swiglu: element count must be a multiple of 8");
    if (((uintptr_t)gate | (uintptr_t)up | (uintptr_t)h) & 15) return set_error(GGQ_ERR_ALIGN, "swiglu: buffers must be 16-byte aligned");
    if (elems == 0) return GGQ_OK;
    hipLaunchKernelGGL(swiglu_fwd_kernel, dim3(stream_grid(elems / 8)), dim3(256), 0, s, (const uint4*)gate, (const uint4*)up, (uint4*)h, elems / 8, limit);
    return check_launch("swiglu_forward");
}

int swiglu_bwd(const void* gate, const void* up, const void* dh, void* dgate, void* dup, int64_t elems, float limit, hipStream_t s) {
    if (elems % 8) return set_error(GGQ_ERR_SHAPE, "swiglu: element count must be a multiple of 8");
    if (((uintptr_t)gate | (uintptr_t)up | (uintptr_t)dh | (uintptr_t)dgate | (uintptr_t)dup) & 15) return set_error(GGQ_ERR_ALIGN, "swiglu: buffers must be 16-byte aligned");
    if (elems == 0) return GGQ_OK;
    hipLaunchKernelGGL(swiglu_bwd_kernel, dim3(stream_grid(elems / 8)), dim3(256), 0, s, (const uint4*)gate, (const uint4*)up, (const uint4*)dh, (uint4*)dgate, (uint4*)dup, elems / 8, limit);
    return check_launch("swiglu_backward");
}

// ------------------------------------------------------------------------------------------------
// Router top-k: per token the top_k best of up to 256 expert scores, best first, equal scores in ascending
// expert index.  One wave per token; lane l holds experts 4l .. 4l+3.  The order is that of the packed key
// (monotone map of the fp32 score bits) << 16 | (256 - expert): the maximum of the keys is the best score and,
// among equal scores, the smallest index.  Score functions: 0 = the logit itself (bf16 logits compare as the
// fp32 values they are), 1 = sqrt(softplus(logit)) in fp32 plus an optional per-expert bias.
// Optional routing weights of the selected experts: 1 = softmax over the selected logits in fp32, stored in the
// logits' type; 2 = sqrt(softplus(logit)) (no bias) / (sum + 1e-20) * scale, stored as fp32.
__device__ __forceinline__ uint32_t float_order_key(float v) {
    const uint32_t b = __builtin_bit_cast(uint32_t, v);
    return b ^ ((b & 0x80000000u) ? 0xFFFFFFFFu : 0x80000000u);
}
__device__ __forceinline__ float sqrt_softplus(float x) { return sqrtf(fmaxf(x, 0.0f) + logf(1.0f + expf(-fabsf(x)))); }

template <bool BF16>
__global__ __launch_bounds__(256) void router_topk_kernel(const void* logits, int64_t tokens, int experts, int top_k, const float* bias,
                                                          int score_fn, int64_t* indices, void* weights, int weights_mode, float scale) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= tokens) return;
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) v[j] = 0.0f;
    const int e0 = 4 * lane;
    if (e0 < experts) {  // experts is a multiple of 4: a lane holds four experts or none
        if (BF16) {
            const uint2 r = *(const uint2*)((const bf16_t*)logits + row * experts + e0);
            v[0] = bf16_lo(r.x), v[1] = bf16_hi(r.x), v[2] = bf16_lo(r.y), v[3] = bf16_hi(r.y);
        } else {
            const float4 r = *(const float4*)((const float*)logits + row * experts + e0);
            v[0] = r.x, v[1] = r.y, v[2] = r.z, v[3] = r.w;
        }
    }
    uint64_t key[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float sc = v[j];
        if (score_fn == 1) {
            sc = sqrt_softplus(sc);
            if (bias && e0 < experts) sc += bias[e0 + j];
        }
        key[j] = e0 < experts ? ((uint64_t)float_order_key(sc) << 16) | (uint64_t)(256 - (e0 + j)) : 0ull;
    }
    float my_logit = 0.0f;  // lane t ends up with the logit of the rank-t expert
    for (int t = 0; t < top_k; t++) {
        uint64_t best = key[0];
#pragma unroll
        for (int j = 1; j < 4; j++) best = key[j] > best ? key[j] : best;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const uint32_t lo = __shfl_xor((uint32_t)best, off), hi = __shfl_xor((uint32_t)(best >> 32), off);
            const uint64_t other = ((uint64_t)hi << 32) | lo;
            best = other > best ? other : best;
        }
        const int expert = 256 - (int)(best & 0xFFFFu);
        float lg = 0.0f;  // the winner's logit, from the lane that holds it
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (key[j] == best && best != 0ull) lg = v[j], key[j] = 0ull;
        // (one lane at most had the key: packed keys are distinct)
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) lg += __shfl_xor(lg, off);
        if (lane == t) my_logit = lg;
        if (lane == 0) indices[row * top_k + t] = expert;
    }
    if (weights_mode == 0 || !weights) return;
    const bool in = lane < top_k;
    if (weights_mode == 1) {
        float m = in ? my_logit : -INFINITY;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
        const float ex = in ? expf(my_logit - m) : 0.0f;
        float sum = ex;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
        const float w = ex / sum;
        if (in) {
            if (BF16) ((bf16_t*)weights)[row * top_k + lane] = to_bf16(w);
            else ((float*)weights)[row * top_k + lane] = w;
        }
    } else {
        const float sc = in ? sqrt_softplus(my_logit) : 0.0f;
        float sum = sc;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
        if (in) ((float*)weights)[row * top_k + lane] = sc / (sum + 1e-20f) * scale;
    }
}

int router_topk(const void* logits, int logits_are_bf16, int64_t tokens, int num_experts, int top_k, const float* bias, int score_fn,
                int64_t* indices, void* weights, int weights_mode, float scale, hipStream_t s) {
    if (!logits || !indices) return set_error(GGQ_ERR_NULL, "router_topk: null logits or indices");
    if (tokens < 0 || num_experts <= 0 || num_experts > 256 || (num_experts & 3) || top_k <= 0 || top_k > 8 || top_k > num_experts)
        return set_error(GGQ_ERR_SHAPE, "router_topk: supports up to 256 experts (a multiple of 4) and top_k <= 8, got experts=%d top_k=%d", num_experts, top_k);
    if (score_fn < 0 || score_fn > 1 || weights_mode < 0 || weights_mode > 2) return set_error(GGQ_ERR_SHAPE, "router_topk: unknown score function or weights mode");
    if (bias && score_fn != 1) return set_error(GGQ_ERR_SHAPE, "router_topk: a correction bias needs sqrt-softplus scoring");
    if (((uintptr_t)logits & 15) != 0) return set_error(GGQ_ERR_ALIGN, "router_topk: logits must be 16-byte aligned");
    if (tokens == 0) return GGQ_OK;
    const unsigned grid = (unsigned)((tokens + 3) / 4);
    if (logits_are_bf16) hipLaunchKernelGGL(router_topk_kernel<true>, dim3(grid), dim3(256), 0, s, logits, tokens, num_experts, top_k, bias, score_fn, indices, weights, weights_mode, scale);
    else hipLaunchKernelGGL(router_topk_kernel<false>, dim3(grid), dim3(256), 0, s, logits, tokens, num_experts, top_k, bias, score_fn, indices, weights, weights_mode, scale);
    return check_launch("router_topk");
}

}  // namespace ggq
