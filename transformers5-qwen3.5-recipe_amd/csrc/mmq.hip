// Host launchers for the packed-weight tile kernel, the expert row-tile table and the error state.
#include "mmq_tile.h"
#include "mmq_direct8.h"
#include "mmq_direct8_nn.h"
#include "mmq_small_iq2.h"
#include "launch.h"

#include <stdarg.h>
#include <stdio.h>

namespace ggq {

// ------------------------------------------------------------------------------------------------
static thread_local char g_last_error[512] = "";

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}
const char* last_error() { return g_last_error; }

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return set_error(GGQ_ERR_RUNTIME, "%s: %s", what, hipGetErrorString(e));
    return GGQ_OK;
}

// ------------------------------------------------------------------------------------------------
// Inclusive prefix sum over the 256 threads of the workgroup: a shuffle scan inside each wave, then the wave totals
// through LDS (one barrier; `totals` must not be reused before the next barrier of the caller).
__device__ __forceinline__ int block_scan_inclusive(int v, int tid, int* totals) {
    const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int u = __shfl_up(v, off, 64);
        if (lane >= off) v += u;
    }
    if (lane == 63) totals[wave] = v;
    __syncthreads();
    int before = 0;
#pragma unroll
    for (int w = 0; w < 3; w++) before += w < wave ? totals[w] : 0;
    return v + before;
}

// Row-tile tables.  One workgroup per table; groups are walked 256 at a time with a prefix sum, so
// a table is in group order and identical from run to run.  Table t keeps the groups with
// min_rows[t] < rows <= max_rows[t] and cuts them into tiles of bm[t] rows.
__global__ __launch_bounds__(256) void build_row_tiles_kernel(const int64_t* expert_ids, const int32_t* end_offsets,
                                                              int groups, RowTileTables tb, int* expert_ranges,
                                                              int num_experts) {
    __shared__ int totals[2][4];
    const int tid = threadIdx.x, t = blockIdx.x;
    const int bm = tb.bm[t], min_rows = tb.min_rows[t], max_rows = tb.max_rows[t];
    TileDesc* tiles = tb.tiles[t];
    if (expert_ranges && t == 0) {
        for (int e = tid; e < num_experts; e += 256) expert_ranges[2 * e] = expert_ranges[2 * e + 1] = 0;
        __syncthreads();  // (the ranges of the listed groups are written below, by other threads)
    }
    int base = 0;  // tiles of the groups walked so far (the same value in every thread)
    int flip = 0;
    for (int g0 = 0; g0 < groups; g0 += 256) {
        const int g = g0 + tid;
        int r0 = 0, r1 = 0, count = 0, expert = 0;
        if (g < groups) {
            expert = expert_ids ? (int)expert_ids[g] : g;
            r0 = g == 0 ? 0 : end_offsets[g - 1];
            r1 = end_offsets[g];
            count = (r1 - r0 > min_rows && r1 - r0 <= max_rows) ? (r1 - r0 + bm - 1) / bm : 0;
            if (expert_ranges && t == 0) {
                const int64_t e = expert_ids ? expert_ids[g] : g;
                if (e >= 0 && e < num_experts) expert_ranges[2 * e] = r0, expert_ranges[2 * e + 1] = r1;
            }
        }
        const int incl = block_scan_inclusive(count, tid, totals[flip]);
        const int first = base + incl - count;
        for (int i = 0; i < count; i++) {
            TileDesc d;
            d.group = g, d.row_begin = r0 + i * bm, d.row_end = min(r1, r0 + (i + 1) * bm), d.expert = expert;
            tiles[first + i] = d;
        }
        base += totals[flip][0] + totals[flip][1] + totals[flip][2] + totals[flip][3];
        flip ^= 1;  // the next round's totals go to the other row: no barrier needed between the rounds
    }
    if (tid == 0) *tb.num_tiles[t] = base;
    TileDesc* by_size = tb.by_size[t];
    if (!by_size) return;
    // Stable bucket sort by the number of 32-row blocks, largest first: thread i takes the i-th contiguous share of the
    // table; the per-thread bucket counts are scanned over the threads, bucket after bucket.
    __syncthreads();  // the table written above is visible to the whole workgroup
    constexpr int kBuckets = 8;  // tiles of up to 256 rows
    __shared__ int bucket_totals[kBuckets][4];
    const int total = base;
    const int share = (total + 255) / 256, i0 = min(total, tid * share), i1 = min(total, i0 + share);
    int mine[kBuckets];
#pragma unroll
    for (int b = 0; b < kBuckets; b++) mine[b] = 0;
    for (int i = i0; i < i1; i++) {
        const int bucket = kBuckets - min(kBuckets, max(1, (tiles[i].row_end - tiles[i].row_begin + 31) >> 5));
#pragma unroll
        for (int b = 0; b < kBuckets; b++) mine[b] += bucket == b;
    }
    int at[kBuckets];  // position of this thread's first tile of bucket b
    int run = 0;
#pragma unroll
    for (int b = 0; b < kBuckets; b++) {
        const int incl = block_scan_inclusive(mine[b], tid, bucket_totals[b]);
        at[b] = run + incl - mine[b];
        run += bucket_totals[b][0] + bucket_totals[b][1] + bucket_totals[b][2] + bucket_totals[b][3];
    }
    for (int i = i0; i < i1; i++) {
        const TileDesc d = tiles[i];
        const int bucket = kBuckets - min(kBuckets, max(1, (d.row_end - d.row_begin + 31) >> 5));
        int pos = 0;
#pragma unroll
        for (int b = 0; b < kBuckets; b++) {
            if (bucket == b) pos = at[b];
            at[b] += bucket == b;
        }
        by_size[pos] = d;
    }
}

int build_row_tile_tables(const int64_t* expert_ids, const int32_t* end_offsets, int groups, const RowTileTables& tb,
                          int* expert_ranges, int num_experts, hipStream_t s) {
    if (tb.count <= 0) return GGQ_OK;
    hipLaunchKernelGGL(build_row_tiles_kernel, dim3(tb.count), dim3(256), 0, s, expert_ids, end_offsets, groups, tb,
                       expert_ranges, num_experts);
    return check_launch("build_row_tiles");
}

int build_row_tiles(const int64_t* expert_ids, const int32_t* end_offsets, int groups, int bm, TileDesc* tiles,
                    int* num_tiles, int* expert_ranges, int num_experts, hipStream_t s, int min_rows, int max_rows) {
    RowTileTables tb{};
    tb.add(bm, min_rows, max_rows, tiles, num_tiles);
    return build_row_tile_tables(expert_ids, end_offsets, groups, tb, expert_ranges, num_experts, s);
}

// ------------------------------------------------------------------------------------------------
// Optional per-launch timing of the tile kernel with HIP events on the launch stream (off by default).
struct TimedLaunch {
    hipEvent_t start, stop;
    int qt, mode, epi, shape;
};
static TimedLaunch g_timed[kMaxTimedLaunches];
static int g_timed_count = 0;
static bool g_timing = false;

int profile_begin() {
    g_timed_count = 0;
    g_timing = true;
    return GGQ_OK;
}

int profile_end(float* ms, int* qt, int* mode, int* epi, int* shape, int capacity) {
    g_timing = false;
    int n = 0;
    for (int i = 0; i < g_timed_count; i++) {
        float t = 0.f;
        if (hipEventSynchronize(g_timed[i].stop) != hipSuccess || hipEventElapsedTime(&t, g_timed[i].start, g_timed[i].stop) != hipSuccess)
            return set_error(GGQ_ERR_RUNTIME, "profile_end: event query failed");
        if (n < capacity) {
            ms[n] = t, qt[n] = g_timed[i].qt, mode[n] = g_timed[i].mode, epi[n] = g_timed[i].epi;
            if (shape) shape[n] = g_timed[i].shape;
            n++;
        }
        (void)hipEventDestroy(g_timed[i].start);
        (void)hipEventDestroy(g_timed[i].stop);
    }
    g_timed_count = 0;
    return n;
}

template <int QT, int MODE, int EPI, int SH>
static int launch_one(const MmqParams& p, hipStream_t s) {
    const int col_tiles = (MODE == kModeNT ? p.nseg : 1) * p.col_tiles_per_seg;
    const int64_t total = (int64_t)p.max_row_tiles * col_tiles;
    if (total <= 0) return GGQ_OK;
    const int64_t grid = (total + 7) / 8 * 8;  // the XCD remap inside the kernel needs a multiple of 8
    if (grid > 0x7FFFFFF0) return set_error(GGQ_ERR_SHAPE, "mmq: too many tiles for one launch");
    TimedLaunch* t = nullptr;
    if (g_timing && g_timed_count < kMaxTimedLaunches) {
        t = &g_timed[g_timed_count];
        if (hipEventCreate(&t->start) != hipSuccess || hipEventCreate(&t->stop) != hipSuccess) return set_error(GGQ_ERR_RUNTIME, "mmq: event creation failed");
        t->qt = QT, t->mode = MODE, t->epi = EPI, t->shape = SH;
        g_timed_count++;
        (void)hipEventRecord(t->start, s);
    }
    constexpr int kSmemBytes = Tile<SH>::kTileLdsBytes + (QT == kIQ2_XXS ? Fmt<kIQ2_XXS>::kTableWords * 4 : 0) +
                               (EPI != kEpiStore ? Tile<SH>::kTM * 16 : 0);
    static LdsLimit lds_limit;  // per instantiation
    if (int rc = raise_lds_limit(lds_limit, (const void*)mmq_tile_kernel<QT, MODE, EPI, SH>, kSmemBytes, "mmq")) return rc;
    hipLaunchKernelGGL((mmq_tile_kernel<QT, MODE, EPI, SH>), dim3((unsigned)grid), dim3(kThreads), kSmemBytes, s, p);
    if (t) (void)hipEventRecord(t->stop, s);
    return check_launch("mmq_tile_kernel");
}

// Q4_K, store epilogue, direct shape: forward or grad-input.
template <int MODE>
static int launch_direct(const MmqParams& p, hipStream_t s) {
    const int col_tiles = (MODE == kModeNT ? p.nseg : 1) * p.col_tiles_per_seg;
    if (p.col_tiles_per_wg < 1) return set_error(GGQ_ERR_SHAPE, "mmq: column tiles per workgroup must be at least 1");
    // row tiles are dealt round-robin over the eight XCDs; each XCD walks its row tiles' column-tile runs
    const int64_t total = (int64_t)((p.max_row_tiles + 7) / 8) * ((col_tiles + p.col_tiles_per_wg - 1) / p.col_tiles_per_wg);
    if (total <= 0) return GGQ_OK;
    const int64_t grid = total * 8;
    if (grid > 0x7FFFFFF0) return set_error(GGQ_ERR_SHAPE, "mmq: too many tiles for one launch");
    if (MODE == kModeNN && ((p.n & 63) || ((p.nseg * p.steps_per_seg) & 1) || p.nseg * p.steps_per_seg < 4))
        return set_error(GGQ_ERR_SHAPE, "mmq: the direct grad-input kernel needs an even number, four or more, of whole 64-row steps");
    TimedLaunch* t = nullptr;
    if (g_timing && g_timed_count < kMaxTimedLaunches) {
        t = &g_timed[g_timed_count];
        if (hipEventCreate(&t->start) != hipSuccess || hipEventCreate(&t->stop) != hipSuccess) return set_error(GGQ_ERR_RUNTIME, "mmq: event creation failed");
        t->qt = kQ4_K, t->mode = MODE, t->epi = kEpiStore, t->shape = kShapeDirect;
        g_timed_count++;
        (void)hipEventRecord(t->start, s);
    }
    constexpr int kSmemBytes = MODE == kModeNT ? Direct8::kLdsBytes : Direct8NN::kLdsBytes;
    const void* fn = MODE == kModeNT ? (const void*)mmq_direct8_q4k_kernel : (const void*)mmq_direct8_nn_q4k_kernel;
    static LdsLimit lds_limit;  // per instantiation
    if (int rc = raise_lds_limit(lds_limit, fn, kSmemBytes, "mmq")) return rc;
    if (MODE == kModeNT) hipLaunchKernelGGL(mmq_direct8_q4k_kernel, dim3((unsigned)grid), dim3(Direct8::kThreadsWG), kSmemBytes, s, p);
    else hipLaunchKernelGGL(mmq_direct8_nn_q4k_kernel, dim3((unsigned)grid), dim3(Direct8NN::kThreadsWG), kSmemBytes, s, p);
    if (t) (void)hipEventRecord(t->stop, s);
    return check_launch(MODE == kModeNT ? "mmq_direct8_q4k_kernel" : "mmq_direct8_nn_q4k_kernel");
}

template <int QT, int MODE>
static int launch_mixed_mode(const MmqParams& p, hipStream_t s) {
    const int segs = MODE == kModeNT ? p.nseg : 1;
    // per XCD: ceil(wide units / 8) * wide column tiles + ceil(tall units / 8) * tall column tiles slots
    const int64_t slots = (int64_t)((p.max_row_tiles + 7) / 8) * segs * p.col_tiles_per_seg +
                          (int64_t)((p.max_row_tiles2 + 7) / 8) * segs * p.col_tiles_per_seg2;
    if (slots <= 0) return GGQ_OK;
    const int64_t grid = slots * 8;
    if (grid > 0x7FFFFFF0) return set_error(GGQ_ERR_SHAPE, "mmq: too many tiles for one launch");
    TimedLaunch* t = nullptr;
    if (g_timing && g_timed_count < kMaxTimedLaunches) {
        t = &g_timed[g_timed_count];
        if (hipEventCreate(&t->start) != hipSuccess || hipEventCreate(&t->stop) != hipSuccess) return set_error(GGQ_ERR_RUNTIME, "mmq: event creation failed");
        t->qt = QT, t->mode = MODE, t->epi = kEpiStore, t->shape = kShapeMixed;
        g_timed_count++;
        (void)hipEventRecord(t->start, s);
    }
    constexpr int kSmemBytes = (Tile<kShapeWide>::kTileLdsBytes > Tile<kShapeTall>::kTileLdsBytes ? Tile<kShapeWide>::kTileLdsBytes : Tile<kShapeTall>::kTileLdsBytes) +
                               (QT == kIQ2_XXS ? Fmt<kIQ2_XXS>::kTableWords * 4 : 0);
    static LdsLimit lds_limit;  // per instantiation
    if (int rc = raise_lds_limit(lds_limit, (const void*)mmq_mixed_kernel<QT, MODE, kEpiStore>, kSmemBytes, "mmq")) return rc;
    hipLaunchKernelGGL((mmq_mixed_kernel<QT, MODE, kEpiStore>), dim3((unsigned)grid), dim3(kThreads), kSmemBytes, s, p);
    if (t) (void)hipEventRecord(t->stop, s);
    return check_launch("mmq_mixed_kernel");
}

// IQ2_XXS, forward, store epilogue: tiles of up to kSmallBM rows (p.tiles) on the decoding-wave kernel.
int launch_mmq_small(const MmqParams& p, hipStream_t s) {
    const int col_tiles = p.nseg * p.col_tiles_per_seg;
    if (p.col_tiles_per_wg < 1) return set_error(GGQ_ERR_SHAPE, "mmq: column tiles per workgroup must be at least 1");
    if (p.steps_per_seg & 3) return set_error(GGQ_ERR_SHAPE, "mmq: the small-group kernel needs a contraction of whole 256-wide blocks");
    // row tiles are dealt round-robin over the eight XCDs; each XCD walks its row tiles' column-tile runs
    const int64_t total = (int64_t)((p.max_row_tiles + 7) / 8) * ((col_tiles + p.col_tiles_per_wg - 1) / p.col_tiles_per_wg);
    if (total <= 0) return GGQ_OK;
    const int64_t grid = total * 8;
    if (grid > 0x7FFFFFF0) return set_error(GGQ_ERR_SHAPE, "mmq: too many tiles for one launch");
    TimedLaunch* t = nullptr;
    if (g_timing && g_timed_count < kMaxTimedLaunches) {
        t = &g_timed[g_timed_count];
        if (hipEventCreate(&t->start) != hipSuccess || hipEventCreate(&t->stop) != hipSuccess) return set_error(GGQ_ERR_RUNTIME, "mmq: event creation failed");
        t->qt = kIQ2_XXS, t->mode = kModeNT, t->epi = kEpiStore, t->shape = kShapeSmall;
        g_timed_count++;
        (void)hipEventRecord(t->start, s);
    }
    static LdsLimit lds_limit;
    if (int rc = raise_lds_limit(lds_limit, (const void*)mmq_small_iq2xxs_kernel, SmallIq2::kLdsBytes, "mmq")) return rc;
    hipLaunchKernelGGL(mmq_small_iq2xxs_kernel, dim3((unsigned)grid), dim3(SmallIq2::kThreadsWG), SmallIq2::kLdsBytes, s, p);
    if (t) (void)hipEventRecord(t->stop, s);
    return check_launch("mmq_small_iq2xxs_kernel");
}

int launch_mmq_mixed(int qt, int mode, const MmqParams& p, hipStream_t s) {
#define GGQ_MIXED(QT) return mode == kModeNT ? launch_mixed_mode<QT, kModeNT>(p, s) : launch_mixed_mode<QT, kModeNN>(p, s)
    switch (qt) {
        case kQ8_0: GGQ_MIXED(kQ8_0);
        case kQ2_K: GGQ_MIXED(kQ2_K);
        case kQ3_K: GGQ_MIXED(kQ3_K);
        case kQ4_K: GGQ_MIXED(kQ4_K);
        case kQ5_K: GGQ_MIXED(kQ5_K);
        case kQ6_K: GGQ_MIXED(kQ6_K);
        case kIQ2_XXS: GGQ_MIXED(kIQ2_XXS);
    }
#undef GGQ_MIXED
    return set_error(GGQ_ERR_QTYPE, "unsupported GGML type id %d", qt);
}

template <int QT>
static int launch_qt(int mode, int epi, const MmqParams& p, hipStream_t s) {
    if (mode == kModeNT) {
        switch (epi) {
            case kEpiStore:
                if (QT == kQ4_K && p.shape == kShapeDirect) return launch_direct<kModeNT>(p, s);
                if (p.shape == kShapeWide) return launch_one<QT, kModeNT, kEpiStore, 1>(p, s);
                return launch_one<QT, kModeNT, kEpiStore, 0>(p, s);
        }
    } else {
        switch (epi) {
            case kEpiStore:
                if (QT == kQ4_K && p.shape == kShapeDirect) return launch_direct<kModeNN>(p, s);
                if (p.shape == kShapeWide) return launch_one<QT, kModeNN, kEpiStore, 1>(p, s);
                return launch_one<QT, kModeNN, kEpiStore, 0>(p, s);
            case kEpiAccumF32: return launch_one<QT, kModeNN, kEpiAccumF32, 0>(p, s);
        }
    }
    return set_error(GGQ_ERR_SHAPE, "mmq: unsupported mode/epilogue combination");
}

int launch_mmq(int qt, int mode, int epi, const MmqParams& p, hipStream_t s) {
    switch (qt) {
        case kQ8_0: return launch_qt<kQ8_0>(mode, epi, p, s);
        case kQ2_K: return launch_qt<kQ2_K>(mode, epi, p, s);
        case kQ3_K: return launch_qt<kQ3_K>(mode, epi, p, s);
        case kQ4_K: return launch_qt<kQ4_K>(mode, epi, p, s);
        case kQ5_K: return launch_qt<kQ5_K>(mode, epi, p, s);
        case kQ6_K: return launch_qt<kQ6_K>(mode, epi, p, s);
        case kIQ2_XXS: return launch_qt<kIQ2_XXS>(mode, epi, p, s);
    }
    return set_error(GGQ_ERR_QTYPE, "unsupported GGML type id %d (supported: 8 Q8_0, 10 Q2_K, 11 Q3_K, 12 Q4_K, 13 Q5_K, 14 Q6_K, 16 IQ2_XXS)", qt);
}

// Fills the shape-derived fields of a parameter block.  n, k describe one weight segment [n, k].
int init_params(MmqParams& p, int qt, int mode, int m, int n, int k, int nseg, int shape) {
    if (m < 0 || n <= 0 || k <= 0) return set_error(GGQ_ERR_SHAPE, "mmq: bad shape m=%d n=%d k=%d", m, n, k);
    if (packed_row_bytes(qt, k) < 0) return set_error(GGQ_ERR_QTYPE, "unsupported GGML type id %d", qt);
    if (!block_multiple(qt, k)) return set_error(GGQ_ERR_SHAPE, "mmq: K=%d is not a multiple of the block size of type %d", k, qt);
    if (k % 64) return set_error(GGQ_ERR_SHAPE, "mmq: K=%d must be a multiple of 64", k);
    p = MmqParams{};
    p.m = m, p.n = n, p.k = k, p.nseg = nseg;
    p.w_row_bytes = packed_row_bytes(qt, k);
    p.w_expert_bytes = p.w_row_bytes * n;
    if (shape == kShapeDirect && qt != kQ4_K) shape = kShapeTall;  // the decoding-wave kernels exist for Q4_K only
    const int bm = shape == kShapeDirect ? kDirectBM : shape == kShapeTall ? kBM : kWideBM;
    const int bn = shape == kShapeDirect ? kDirectBN : shape == kShapeWide ? kWideBN : kBN;
    p.shape = shape;
    if (mode == kModeNT) {
        p.col_tiles_per_seg = (n + bn - 1) / bn;
        p.steps_per_seg = k / kBK;
    } else {
        p.col_tiles_per_seg = (k + bn - 1) / bn;
        p.steps_per_seg = (n + kBK - 1) / kBK;
    }
    p.max_row_tiles = (m + bm - 1) / bm;
    p.col_tiles_per_wg = 1;
    return GGQ_OK;
}


}  // namespace ggq
