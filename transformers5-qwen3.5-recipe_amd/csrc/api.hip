// extern "C" surface of libggml_mmq_gfx950.so.  Declarations and the reference interface each entry
// point replaces are in include/ggml_mmq_gfx950.h.  Plain device pointers and sizes only.
#include "../../include/ggml_mmq_gfx950.h"

#include <algorithm>
#include <mutex>

#include "launch.h"
#include "mmq_host.h"

using namespace ggq;

namespace {

inline hipStream_t as_stream(void* s) { return (hipStream_t)s; }
inline int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }
inline int rank_pad(int r) { return (r + 15) / 16 * 16; }

struct Bump {  // carve 256-byte aligned pieces out of the caller's workspace
    char* base;
    int64_t size, used;
    void* take(int64_t bytes) {
        const int64_t at = used;
        used += align256(bytes);
        return used <= size ? base + at : nullptr;
    }
};

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

std::atomic<int> g_shape_override{-1};  // ggq_debug_force_grouped_shape (a test aid): -1 = the automatic choice

// ---------------------------------------------------------------------------------------------------
// The factor gradients dA / dB of a backward call depend on nothing the grad-input launch writes, are HBM-bound and
// small, while the grad-input launch is MFMA-bound and leaves compute units idle at its tail: they run on a second
// stream of the library's own, forked from the caller's stream behind the rank-sized product they read and joined back
// into it before the call returns, so that to the caller the call is still one ordered piece of work on its stream.
// Under stream capture the fork and the join become graph edges.  One side stream and event pair per device (default
// priority); the lock is held while a call enqueues its forked section, so calls from several threads do not mix their
// event records.  A stream that is being captured when the side stream does not exist yet runs the call unforked
// (nothing is created during a capture).
std::atomic<int> g_overlap_enabled{1};
constexpr int kMaxDevices = 64;
struct SideStream {
    hipStream_t stream = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    bool tried = false;
};
SideStream g_side[kMaxDevices];
std::mutex g_side_lock;

class Forked {  // fork on construction (when allowed), join in done() or on destruction
public:
    explicit Forked(hipStream_t main_stream) : main_(main_stream), lock_(g_side_lock, std::defer_lock) {
        if (!g_overlap_enabled.load(std::memory_order_relaxed)) return;
        int device = -1;
        if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return;
        lock_.lock();
        SideStream& st = g_side[device];
        if (!st.stream) {
            hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
            if (st.tried || hipStreamIsCapturing(main_, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
                (void)hipGetLastError();
                lock_.unlock();
                return;
            }
            st.tried = true;
            if (hipStreamCreateWithFlags(&st.stream, hipStreamNonBlocking) != hipSuccess || hipEventCreateWithFlags(&st.fork, hipEventDisableTiming) != hipSuccess ||
                hipEventCreateWithFlags(&st.join, hipEventDisableTiming) != hipSuccess) {
                (void)hipGetLastError();
                st.stream = nullptr;
                lock_.unlock();
                return;
            }
        }
        if (hipEventRecord(st.fork, main_) != hipSuccess || hipStreamWaitEvent(st.stream, st.fork, 0) != hipSuccess) {
            (void)hipGetLastError();
            lock_.unlock();
            return;
        }
        side_ = &st;
    }
    hipStream_t stream() const { return side_ ? side_->stream : main_; }  // the forked stream, or the caller's own
    int done() {
        if (!side_) return GGQ_OK;
        const bool ok = hipEventRecord(side_->join, side_->stream) == hipSuccess && hipStreamWaitEvent(main_, side_->join, 0) == hipSuccess;
        side_ = nullptr;
        lock_.unlock();
        return ok ? GGQ_OK : set_error(GGQ_ERR_RUNTIME, "could not join the library's side stream");
    }
    ~Forked() { (void)done(); }

private:
    hipStream_t main_;
    std::unique_lock<std::mutex> lock_;
    SideStream* side_ = nullptr;
};

int check_weights(const char* what, int qt, const void* w, int64_t k) {
    if (!w) return set_error(GGQ_ERR_NULL, "%s: packed weight pointer is null", what);
    if (packed_row_bytes(qt, k) < 0) return set_error(GGQ_ERR_QTYPE, "%s: unsupported GGML type id %d (supported: 8, 10, 11, 12, 13, 14, 16)", what, qt);
    if (!aligned16(w)) return set_error(GGQ_ERR_ALIGN, "%s: packed weights must be 16-byte aligned", what);
    return GGQ_OK;
}

int check_lora(const char* what, const void* a, const void* b, int r) {
    if ((a == nullptr) != (b == nullptr)) return set_error(GGQ_ERR_NULL, "%s: LoRA factors must both be given or both be null", what);
    if (a && (r < 1 || r > 64)) return set_error(GGQ_ERR_SHAPE, "%s: LoRA rank %d outside 1..64", what, r);
    if (a && (!aligned16(a) || !aligned16(b))) return set_error(GGQ_ERR_ALIGN, "%s: LoRA factors must be 16-byte aligned", what);
    return GGQ_OK;
}

}  // namespace

extern "C" {

const char* ggq_last_error(void) { return last_error(); }

int ggq_profile_begin(void) { return profile_begin(); }

int ggq_profile_end(float* ms, int* qt, int* mode, int* epilogue, int* shape, int capacity) {
    if (!ms || !qt || !mode || !epilogue) return set_error(GGQ_ERR_NULL, "profile_end: null pointer");
    return profile_end(ms, qt, mode, epilogue, shape, capacity);
}

int ggq_measure_mfma_ceiling(const void* a_samples, const void* b_samples, int64_t elems, int iters, void* sink, float* tflops_out, void* stream) {
    return measure_mfma_ceiling(a_samples, b_samples, elems, iters, sink, tflops_out, as_stream(stream));
}

int ggq_debug_force_grouped_shape(int shape) {
    if (shape != -1 && shape != kShapeTall && shape != kShapeWide && shape != kShapeDirect && shape != kShapeSmall) return set_error(GGQ_ERR_SHAPE, "debug_force_grouped_shape: unknown shape %d", shape);
    g_shape_override.store(shape);
    return GGQ_OK;
}

int ggq_set_factor_gradient_overlap(int enabled) {
    g_overlap_enabled.store(enabled ? 1 : 0, std::memory_order_relaxed);
    return GGQ_OK;
}

int ggq_supports_quant_type(int qt) { return packed_row_bytes(qt, 256) > 0 ? 1 : 0; }

int64_t ggq_row_bytes(int qt, int64_t k) { return block_multiple(qt, k) ? packed_row_bytes(qt, k) : -1; }

int ggq_dequantize(int qt, const void* packed, int64_t rows, int64_t k, void* out, int out_is_f32, void* stream) {
    if (!packed || !out) return set_error(GGQ_ERR_NULL, "dequantize: null pointer");
    return dequantize(qt, packed, rows, k, out, out_is_f32, as_stream(stream));
}

// ---------------------------------------------------------------------------------------------------
// A grouped call that runs its small groups in the wide shape puts the row tiles of its larger groups in a
// second table; one mixed launch covers both.
static int launch_wide_and_tall(int qt, int mode, MmqParams& p, int rows, int n, int k, int nseg, const TileDesc* tall,
                                const int* num_tall, int max_tall, hipStream_t s) {
    MmqParams sizes;
    if (int rc = init_params(sizes, qt, mode, rows, n, k, nseg, kShapeTall)) return rc;
    p.tiles2 = tall, p.num_tiles2 = num_tall, p.max_row_tiles2 = max_tall, p.col_tiles_per_seg2 = sizes.col_tiles_per_seg;
    return launch_mmq_mixed(qt, mode, p, s);
}

// Q4_K over expert groups that average at most 256 rows runs the direct kernels (the MFMA waves decode the weights
// themselves) when the operands allow (`direct_ok`); otherwise, and for every other block format, groups that average at
// most 192 rows run the tile kernel in its wide shape, mixed with tall tiles for their larger groups; everything else runs
// tall tiles.
static int pick_shape(int qt, int64_t rows, int64_t groups, bool direct_ok) {
    const int forced = g_shape_override.load();  // a test aid
    const bool q4k = qt == 12;            // GGML Q4_K: the only block format with decoding-wave kernels
    if (q4k && direct_ok && (forced == kShapeDirect || (forced < 0 && groups > 0 && rows <= 256 * groups))) return kShapeDirect;
    if (forced == kShapeTall || !(groups > 0 && rows <= 192 * groups)) return kShapeTall;
    return kShapeWide;
}

// Direct shape: a workgroup walks a run of column tiles of its row tile as one stream of steps, so that only the run's
// first tile waits for its first loads.  Measured on configs[2] by alternating captured steps on one box: tiles of 32
// steps and more want runs of two (one tile per workgroup is 0.9 % of the step slower per such launch, four 0.4 %
// slower still); shorter tiles want runs of four in the forward launch (two and eight are both slower) and of eight in
// the grad-input launch (four: + 0.4 %, two: + 1.3 %).  Fewer per run while that leaves compute units without work.
static int direct_tiles_per_wg(int64_t rows, int64_t groups, int col_tiles, int steps_per_tile, int mode) {
    const int64_t row_tiles = groups > 0 ? std::max<int64_t>(groups, rows / kDirectBM) : (rows + kDirectBM - 1) / kDirectBM;
    int per_wg = steps_per_tile >= 32 ? 2 : mode == kModeNN ? 8 : 4;
    while (per_wg > 1 && row_tiles * ((col_tiles + per_wg - 1) / per_wg) < 256) per_wg >>= 1;
    return per_wg;
}

// Small shape: a workgroup stages the decoder's tables and its row tile's LoRA rows once, so it walks up to four column
// tiles while that still leaves every compute unit eight workgroups.
static int small_tiles_per_wg(int64_t groups, int col_tiles) {
    int per_wg = 4;
    while (per_wg > 1 && groups * ((col_tiles + per_wg - 1) / per_wg) < 2048) per_wg >>= 1;
    return per_wg;
}

// A dense layer's factor gradients deal their rows to at most this many workgroups per column block (fp32 partial sums
// in the workspace).
constexpr int64_t kDenseFactorSplits = 32;

int64_t ggq_lora_workspace_bytes(int64_t rows, int64_t groups, int64_t experts, int64_t n_total, int64_t k, int r) {
    const int rp = rank_pad(r > 0 ? r : 1);
    if (experts < 1) experts = 1;
    const int64_t tiles = rows / 64 + groups + 2;
    return 5 * align256(tiles * (int64_t)sizeof(TileDesc)) + align256(16) + align256(experts * 2 * 4) +
           align256(experts * n_total * rp * 2) * 2 + align256(experts * k * rp * 2) + align256(rows * rp * 2) + 4096 +
           (groups == 0 ? align256(kDenseFactorSplits * std::max(n_total, k) * rp * 4) : 0);
}

int ggq_lora_mmq_forward(const void* x, const void* packed, int qt, int64_t m, int64_t n, int64_t k, const void* lora_a,
                         const void* lora_b, int r, float scale, void* xa_out, void* y, void* ws, int64_t ws_bytes,
                         void* stream) {
    return ggq_grouped_lora_mmq_forward(x, packed, nullptr, nullptr, nullptr, 0, 1, qt, m, n, k, lora_a, lora_b, r,
                                        scale, xa_out, y, nullptr, nullptr, ws, ws_bytes, stream);
}

int ggq_lora_mmq_backward(const void* dy, const void* packed, int qt, int64_t m, int64_t n, int64_t k, const void* x,
                          const void* xa, const void* lora_a, const void* lora_b, int r, float scale, void* dx,
                          void* d_lora_a, void* d_lora_b, void* ws, int64_t ws_bytes, void* stream) {
    return ggq_grouped_lora_mmq_backward(dy, nullptr, packed, nullptr, nullptr, nullptr, 0, 1, qt, m, n, k, x, xa, lora_a,
                                         lora_b, r, scale, dx, d_lora_a, d_lora_b, nullptr, ws, ws_bytes, stream);
}

int ggq_mmq(const void* x, const void* packed, int qt, int64_t m, int64_t n, int64_t k, void* y, void* stream) {
    return ggq_grouped_lora_mmq_forward(x, packed, nullptr, nullptr, nullptr, 0, 1, qt, m, n, k, nullptr, nullptr, 0, 0.f,
                                        nullptr, y, nullptr, nullptr, nullptr, 0, stream);
}

int ggq_mmq_grad_input(const void* dy, const void* packed, int qt, int64_t m, int64_t n, int64_t k, void* dx, void* stream) {
    return ggq_grouped_lora_mmq_backward(dy, nullptr, packed, nullptr, nullptr, nullptr, 0, 1, qt, m, n, k, nullptr, nullptr,
                                         nullptr, nullptr, 0, 0.f, dx, nullptr, nullptr, nullptr, nullptr, 0, stream);
}

// ---------------------------------------------------------------------------------------------------
// Fixed groups: x [rows, groups, k], one packed [n_group, k] matrix per group, y [rows, groups, n_group].  Group g is
// a dense matmul over the strided rows x[:, g, :]; it runs as that launch (same tiles, same arithmetic as ggq_mmq on a
// contiguous copy), so the results are bit-identical to the per-group dense calls.
static int fixed_grouped(const char* what, int mode, const void* in, const void* packed, int qt, int64_t rows, int groups, int64_t n_group,
                         int64_t k, void* out, hipStream_t s) {
    if (rows < 0 || groups <= 0 || n_group <= 0 || k <= 0 || rows >= (1ll << 31) || n_group >= (1ll << 30) || k >= (1ll << 30) ||
        (int64_t)groups * std::max(n_group, k) >= (1ll << 31))
        return set_error(GGQ_ERR_SHAPE, "%s: bad shape rows=%lld groups=%d n_group=%lld k=%lld", what, (long long)rows, groups, (long long)n_group, (long long)k);
    if (int rc = check_weights(what, qt, packed, k)) return rc;
    if (!in || !out) return set_error(GGQ_ERR_NULL, "%s: null activation or output pointer", what);
    if (rows == 0) return GGQ_OK;
    const int64_t in_cols = mode == kModeNT ? k : n_group, out_cols = mode == kModeNT ? n_group : k;
    for (int g = 0; g < groups; g++) {
        MmqParams p;
        if (int rc = init_params(p, qt, mode, (int)rows, (int)n_group, (int)k, 1, kShapeTall)) return rc;
        p.a[0] = (const bf16_t*)in + g * in_cols, p.lda = groups * in_cols;
        p.w[0] = (const uint8_t*)packed + g * p.w_expert_bytes;
        p.c[0] = (bf16_t*)out + g * out_cols, p.ldc = groups * out_cols;
        if (int rc = launch_mmq(qt, mode, kEpiStore, p, s)) return rc;
    }
    return GGQ_OK;
}

int ggq_fixed_grouped_mmq(const void* x, const void* packed_groups, int qt, int64_t rows, int groups, int64_t n_group, int64_t k, void* y,
                          void* stream) {
    return fixed_grouped("fixed_grouped_mmq", kModeNT, x, packed_groups, qt, rows, groups, n_group, k, y, as_stream(stream));
}

int ggq_fixed_grouped_mmq_grad_input(const void* dy, const void* packed_groups, int qt, int64_t rows, int groups, int64_t n_group, int64_t k,
                                     void* dx, void* stream) {
    return fixed_grouped("fixed_grouped_mmq_grad_input", kModeNN, dy, packed_groups, qt, rows, groups, n_group, k, dx, as_stream(stream));
}

// Row-tile tables of one grouping, built once (ggq_group_tables_build) and handed to the launches that share it: the
// main table in group order and sorted by size, the 64-row table of the LoRA side kernels, the two tile counts, the
// per-expert row ranges.  Only the decoding-wave kernels' tile height is covered; a launch of another shape builds its own.
struct GroupTablesView {
    TileDesc *t_main, *t_sorted, *t64;
    int* counts;
    int* ranges;
    int max_main, max64;
};
static int64_t group_tables_layout(void* base, int64_t rows, int64_t groups, int64_t experts, GroupTablesView& v) {
    Bump b{(char*)base, INT64_MAX, 0};
    v.max_main = (int)(rows / kDirectBM + groups), v.max64 = (int)(rows / 64 + groups);
    v.t_main = (TileDesc*)b.take((int64_t)v.max_main * sizeof(TileDesc));
    v.t_sorted = (TileDesc*)b.take((int64_t)v.max_main * sizeof(TileDesc));
    v.t64 = (TileDesc*)b.take((int64_t)v.max64 * sizeof(TileDesc));
    v.counts = (int*)b.take(16);
    v.ranges = (int*)b.take(experts * 2 * 4);
    return b.used;
}

int64_t ggq_group_tables_bytes(int64_t rows, int64_t groups, int64_t experts) {
    if (rows < 0 || groups < 1 || experts < 1 || rows >= (1ll << 31)) return -1;
    GroupTablesView v;
    return group_tables_layout(nullptr, rows, groups, experts, v);
}

int ggq_group_tables_build(const int64_t* expert_ids, const int32_t* end_offsets, int64_t groups, int64_t experts, int64_t rows, void* tables,
                           int64_t tables_bytes, void* stream) {
    if (!expert_ids || !end_offsets || !tables) return set_error(GGQ_ERR_NULL, "group_tables_build: null pointer");
    if (!aligned16(tables)) return set_error(GGQ_ERR_ALIGN, "group_tables_build: the table buffer must be 16-byte aligned");
    const int64_t need = ggq_group_tables_bytes(rows, groups, experts);
    if (need < 0) return set_error(GGQ_ERR_SHAPE, "group_tables_build: bad sizes rows=%lld groups=%lld experts=%lld", (long long)rows, (long long)groups, (long long)experts);
    if (tables_bytes < need) return set_error(GGQ_ERR_WORKSPACE, "group_tables_build: buffer of %lld bytes, %lld needed", (long long)tables_bytes, (long long)need);
    GroupTablesView v;
    group_tables_layout(tables, rows, groups, experts, v);
    RowTileTables tb{};
    tb.add(kDirectBM, 0, 0x7FFFFFFF, v.t_main, v.counts, v.t_sorted);
    tb.add(64, 0, 0x7FFFFFFF, v.t64, v.counts + 1);
    return build_row_tile_tables(expert_ids, end_offsets, (int)groups, tb, v.ranges, (int)experts, as_stream(stream));
}

// Forward of one projection (or a gate/up pair) over expert-sorted rows, optional LoRA fused.
// groups == 0 means dense: one group of all rows using expert 0.
// The forward launch reads its rows through an index when the source matrix stays under 4 GiB (the lane offsets of its
// loads are 32-bit).
static bool forward_reads_indexed_rows(int qt, int64_t rows, int64_t groups, int64_t x_rows, int64_t k) {
    (void)rows, (void)groups;
    return packed_row_bytes(qt, 256) > 0 && x_rows > 0 && k > 0 && (uint64_t)x_rows * (uint64_t)k * 2 < (1ull << 32);
}

int ggq_grouped_forward_reads_indexed_rows(int qt, int64_t rows, int64_t groups, int64_t x_rows, int64_t k) {
    return forward_reads_indexed_rows(qt, rows, groups, x_rows, k) ? 1 : 0;
}

static int grouped_forward(const char* what, const void* x, RowIndex x_index, const void* packed1, const void* packed2, const int64_t* expert_ids,
                           const int32_t* end_offsets, int64_t groups, int64_t experts, int qt, int64_t rows, int64_t n,
                           int64_t k, const void* lora_a, const void* lora_b, int r, float scale, void* xa_out, void* y1,
                           void* y2, const void* group_tables, void* ws, int64_t ws_bytes, void* stream) {
    hipStream_t s = as_stream(stream);
    if (group_tables && !aligned16(group_tables)) return set_error(GGQ_ERR_ALIGN, "%s: group tables must be 16-byte aligned", what);
    if (rows < 0 || n <= 0 || k <= 0 || rows >= (1ll << 31) || n >= (1ll << 30) || k >= (1ll << 30)) return set_error(GGQ_ERR_SHAPE, "%s: bad shape rows=%lld n=%lld k=%lld", what, (long long)rows, (long long)n, (long long)k);
    if (int rc = check_weights(what, qt, packed1, k)) return rc;
    if (packed2 && !aligned16(packed2)) return set_error(GGQ_ERR_ALIGN, "%s: packed weights must be 16-byte aligned", what);
    if (int rc = check_lora(what, lora_a, lora_b, r)) return rc;
    if (!x || !y1 || (packed2 && !y2)) return set_error(GGQ_ERR_NULL, "%s: null activation or output pointer", what);
    if (groups > 0 && (!expert_ids || !end_offsets)) return set_error(GGQ_ERR_NULL, "%s: expert ids / offsets are null", what);
    if (lora_a && !xa_out) return set_error(GGQ_ERR_NULL, "%s: xa_out is required with LoRA", what);
    if (rows == 0) return GGQ_OK;
    const int nseg = packed2 ? 2 : 1;
    const int rp = lora_a ? rank_pad(r) : 0;
    Bump bump{(char*)ws, ws_bytes, 0};

    MmqParams p;
    // the direct kernel moves A, LA and LB rows with aligned 16-byte accesses
    const bool direct_ok = aligned16(x) && k < (1 << 22) && (!lora_a || (aligned16(xa_out) && (rp != r || aligned16(lora_b))));
    if (int rc = init_params(p, qt, kModeNT, (int)rows, (int)n, (int)k, nseg, pick_shape(qt, rows, groups, direct_ok))) return rc;
    if (x_index.on() && (!forward_reads_indexed_rows(qt, rows, groups, x_index.index_rows, k) || x_index.index_div <= 0))
        return set_error(GGQ_ERR_SHAPE, "%s: this source matrix cannot be read through a row index (ask ggq_grouped_forward_reads_indexed_rows first)", what);
    p.a[0] = (const bf16_t*)x, p.lda = k, p.a_rows = x_index;
    p.w[0] = (const uint8_t*)packed1, p.w[1] = (const uint8_t*)packed2;
    p.c[0] = y1, p.c[1] = y2, p.ldc = n;
    if (p.shape == kShapeDirect) p.col_tiles_per_wg = direct_tiles_per_wg(rows, groups, nseg * p.col_tiles_per_seg, p.steps_per_seg, kModeNT);

    const TileDesc* tiles64 = nullptr;
    const int* num_tiles64 = nullptr;
    int max_tiles64 = (int)((rows + 63) / 64);
    TileDesc* t_tall = nullptr;
    const int* n_tall = nullptr;
    int max_tall = 0;
    TileDesc* t_small = nullptr;
    const int* n_small = nullptr;
    if (groups > 0 && group_tables && p.shape == kShapeDirect) {  // tables the caller built once for this grouping
        GroupTablesView v;
        group_tables_layout(const_cast<void*>(group_tables), rows, groups, experts, v);
        max_tiles64 = v.max64;
        p.expert_ids = expert_ids, p.tiles = v.t_sorted, p.num_tiles = v.counts, p.max_row_tiles = v.max_main;
        tiles64 = v.t64, num_tiles64 = v.counts + 1;
    } else if (groups > 0) {
        // Wide shape: groups of at most 128 rows take one wide tile each, larger groups go to a second,
        // tall launch (a second wide tile for a few dozen leftover rows would cost a whole decode pass).
        const bool wide = p.shape == kShapeWide;
        const int bm_main = p.shape == kShapeDirect ? kDirectBM : p.shape == kShapeTall ? kBM : kWideBM;
        const int max128 = wide ? (int)groups : (int)(rows / bm_main + groups);
        max_tall = wide ? (int)std::min<int64_t>(rows / kBM + groups, rows / (kWideBM + 1) + rows / kBM + 1) : 0;
        max_tiles64 = (int)(rows / 64 + groups);
        const bool direct = p.shape == kShapeDirect;  // its workgroups take the tiles with the most rows first
        TileDesc* t128 = (TileDesc*)bump.take((int64_t)max128 * sizeof(TileDesc));
        TileDesc* t_sorted = direct ? (TileDesc*)bump.take((int64_t)max128 * sizeof(TileDesc)) : nullptr;
        t_tall = wide ? (TileDesc*)bump.take((int64_t)max_tall * sizeof(TileDesc)) : nullptr;
        TileDesc* t64 = lora_a ? (TileDesc*)bump.take((int64_t)max_tiles64 * sizeof(TileDesc)) : nullptr;
        // IQ2_XXS: the groups of at most 128 rows leave the wide table for a launch of their own (decoding waves)
        // (its lanes address a weight plane with 32-bit offsets)
        const bool small = wide && qt == 16 /* GGML IQ2_XXS */ && direct_ok && p.w_expert_bytes < (1ll << 32) && g_shape_override.load() != kShapeWide;
        t_small = small ? (TileDesc*)bump.take((int64_t)groups * sizeof(TileDesc)) : nullptr;
        TileDesc* t_small_sorted = small ? (TileDesc*)bump.take((int64_t)groups * sizeof(TileDesc)) : nullptr;  // most row blocks first
        int* counts = (int*)bump.take(16);
        if (!t128 || !counts || (lora_a && !t64) || (wide && !t_tall) || (direct && !t_sorted) || (small && (!t_small || !t_small_sorted))) return set_error(GGQ_ERR_WORKSPACE, "%s: workspace too small", what);
        RowTileTables tb{};
        tb.add(bm_main, small ? kSmallBM : 0, wide ? kWideBM : 0x7FFFFFFF, t128, counts, t_sorted);
        if (direct) t128 = t_sorted;
        if (wide) tb.add(kBM, kWideBM, 0x7FFFFFFF, t_tall, counts + 2), n_tall = counts + 2;
        if (lora_a) tb.add(64, 0, 0x7FFFFFFF, t64, counts + 1);
        if (small) tb.add(kSmallBM, 0, kSmallBM, t_small, counts + 3, t_small_sorted), n_small = counts + 3, t_small = t_small_sorted;
        if (int rc = build_row_tile_tables(expert_ids, end_offsets, (int)groups, tb, nullptr, 0, s)) return rc;
        p.expert_ids = expert_ids, p.tiles = t128, p.num_tiles = counts, p.max_row_tiles = small ? 0 : max128;  // (small: the wide table stays empty)
        tiles64 = t64, num_tiles64 = counts + 1;
    }
    if (lora_a) {
        SkinnyNtParams sp{};
        sp.in[0] = (const bf16_t*)x, sp.ld_in = k, sp.in_rows = x_index;
        sp.f = (const bf16_t*)lora_a, sp.ldf = k, sp.f_expert_elems = (int64_t)r * k;
        sp.out = (bf16_t*)xa_out;
        sp.m = (int)rows, sp.c = (int)k, sp.r = r, sp.nseg = 1;
        sp.expert_ids = groups > 0 ? expert_ids : nullptr, sp.tiles = tiles64, sp.num_tiles = num_tiles64;
        if (int rc = skinny_nt(sp, rp, max_tiles64, s)) return rc;
        const bf16_t* lb = (const bf16_t*)lora_b;
        if (rp != r) {
            bf16_t* padded = (bf16_t*)bump.take(experts * nseg * n * rp * 2);
            if (!padded) return set_error(GGQ_ERR_WORKSPACE, "%s: workspace too small", what);
            if (int rc = pad_factor(lb, padded, experts, (int)(nseg * n), r, rp, false, s)) return rc;
            lb = padded;
        }
        p.la = (const bf16_t*)xa_out, p.lb = lb, p.lb_expert_elems = (int64_t)nseg * n * rp, p.r_pad = rp, p.lora_scale = scale;
    }
    if (t_small) {
        MmqParams ps = p;
        ps.tiles = t_small, ps.num_tiles = n_small, ps.max_row_tiles = (int)groups, ps.shape = kShapeSmall;
        ps.col_tiles_per_wg = small_tiles_per_wg(groups, nseg * p.col_tiles_per_seg);
        if (int rc = launch_mmq_small(ps, s)) return rc;
    }
    if (t_tall) return launch_wide_and_tall(qt, kModeNT, p, (int)rows, (int)n, (int)k, nseg, t_tall, n_tall, max_tall, s);
    return launch_mmq(qt, kModeNT, kEpiStore, p, s);
}

int ggq_grouped_lora_mmq_forward(const void* x, const void* packed1, const void* packed2, const int64_t* expert_ids,
                                 const int32_t* end_offsets, int64_t groups, int64_t experts, int qt, int64_t rows, int64_t n,
                                 int64_t k, const void* lora_a, const void* lora_b, int r, float scale, void* xa_out, void* y1,
                                 void* y2, const void* group_tables, void* ws, int64_t ws_bytes, void* stream) {
    return grouped_forward("grouped_lora_mmq_forward", x, RowIndex{}, packed1, packed2, expert_ids, end_offsets, groups, experts, qt, rows, n, k,
                           lora_a, lora_b, r, scale, xa_out, y1, y2, group_tables, ws, ws_bytes, stream);
}

// The same forward over rows that are not materialised: row i of the expert-sorted layout is row
// row_index[i] / index_div of x [x_rows, k].
int ggq_grouped_lora_mmq_forward_indexed(const void* x, int64_t x_rows, const int64_t* row_index, int index_div, const void* packed1,
                                         const void* packed2, const int64_t* expert_ids, const int32_t* end_offsets, int64_t groups,
                                         int64_t experts, int qt, int64_t rows, int64_t n, int64_t k, const void* lora_a,
                                         const void* lora_b, int r, float scale, void* xa_out, void* y1, void* y2, const void* group_tables,
                                         void* ws, int64_t ws_bytes, void* stream) {
    const char* what = "grouped_lora_mmq_forward_indexed";
    if (!row_index) return set_error(GGQ_ERR_NULL, "%s: null row index", what);
    if (x_rows <= 0 || x_rows >= (1ll << 31) || index_div <= 0) return set_error(GGQ_ERR_SHAPE, "%s: bad x_rows=%lld or index_div=%d", what, (long long)x_rows, index_div);
    return grouped_forward(what, x, RowIndex{row_index, index_div, (int)x_rows}, packed1, packed2, expert_ids, end_offsets, groups, experts, qt,
                           rows, n, k, lora_a, lora_b, r, scale, xa_out, y1, y2, group_tables, ws, ws_bytes, stream);
}

// Backward: dx = dy . W (+ LoRA term), and the factor gradients over all `experts` planes.
static int grouped_backward(const char* what, const void* dy1, const void* dy2, const void* packed1, const void* packed2,
                            const int64_t* expert_ids, const int32_t* end_offsets, int64_t groups, int64_t experts, int qt,
                            int64_t rows, int64_t n, int64_t k, const void* x, RowIndex x_index, const void* xa, const void* lora_a,
                            const void* lora_b, int r, float scale, void* dx, void* d_lora_a, void* d_lora_b, const void* group_tables,
                            void* ws, int64_t ws_bytes, void* stream, RowIndex dy_index = RowIndex{}, const void* row_weights = nullptr,
                            int row_weights_are_bf16 = 0) {
    // dy_index: row i of the launch is row dy_index.source(i) of dy1 (one cotangent matrix), and, with row_weights, stands
    // for weights[dy_index.row_index[i]] times that row: dx comes out WITHOUT that factor (the caller applies it), the
    // factor gradients with it (it is put on their small operand, dy.B or xa)
    hipStream_t s = as_stream(stream);
    if (group_tables && !aligned16(group_tables)) return set_error(GGQ_ERR_ALIGN, "%s: group tables must be 16-byte aligned", what);
    if (dy_index.on() && (dy2 || (uint64_t)dy_index.index_rows * (uint64_t)n * 2 >= (1ull << 32)))
        return set_error(GGQ_ERR_SHAPE, "%s: an indexed cotangent is one matrix under 4 GiB", what);
    if (rows < 0 || n <= 0 || k <= 0 || rows >= (1ll << 31) || n >= (1ll << 30) || k >= (1ll << 30)) return set_error(GGQ_ERR_SHAPE, "%s: bad shape rows=%lld n=%lld k=%lld", what, (long long)rows, (long long)n, (long long)k);
    if (int rc = check_weights(what, qt, packed1, k)) return rc;
    if (packed2 && !aligned16(packed2)) return set_error(GGQ_ERR_ALIGN, "%s: packed weights must be 16-byte aligned", what);
    if ((packed2 == nullptr) != (dy2 == nullptr)) return set_error(GGQ_ERR_NULL, "%s: a pair needs both cotangents and both weights", what);
    if (int rc = check_lora(what, lora_a, lora_b, r)) return rc;
    if (!dy1 || !dx) return set_error(GGQ_ERR_NULL, "%s: null cotangent or output pointer", what);
    if (groups > 0 && (!expert_ids || !end_offsets)) return set_error(GGQ_ERR_NULL, "%s: expert ids / offsets are null", what);
    if (lora_a && (!x || !xa)) return set_error(GGQ_ERR_NULL, "%s: x and xa are required with LoRA", what);
    if ((d_lora_a || d_lora_b) && !lora_a) return set_error(GGQ_ERR_NULL, "%s: factor gradients requested without factors", what);
    const int nseg = packed2 ? 2 : 1;
    const int rp = lora_a ? rank_pad(r) : 0;
    const int64_t ntot = nseg * n;
    Bump bump{(char*)ws, ws_bytes, 0};

    MmqParams p;
    // the direct kernel moves the cotangents with aligned 16-byte accesses and takes an even number, four or more, of whole
    // 64-row steps (the request of a tile's LoRA factor piece is certain to have landed behind the tile's third step)
    const bool direct_ok = aligned16(dy1) && (!dy2 || aligned16(dy2)) && n % 64 == 0 && (nseg * (n / 64)) % 2 == 0 && nseg * (n / 64) >= 4 && n < (1 << 22) &&
                           (!lora_a || aligned16(lora_a)) && k % 8 == 0;
    if (int rc = init_params(p, qt, kModeNN, (int)rows, (int)n, (int)k, nseg, pick_shape(qt, rows, groups, direct_ok))) return rc;
    p.a[0] = (const bf16_t*)dy1, p.a[1] = (const bf16_t*)dy2, p.lda = n, p.a_rows = dy_index;
    p.w[0] = (const uint8_t*)packed1, p.w[1] = (const uint8_t*)packed2;
    p.c[0] = dx, p.ldc = k;
    if (p.shape == kShapeDirect) p.col_tiles_per_wg = direct_tiles_per_wg(rows, groups, p.col_tiles_per_seg, nseg * p.steps_per_seg, kModeNN);

    const TileDesc* tiles64 = nullptr;
    const int* num_tiles64 = nullptr;
    const int* ranges = nullptr;
    int max_tiles64 = (int)((rows + 63) / 64);
    TileDesc* t_tall = nullptr;
    const int* n_tall = nullptr;
    int max_tall = 0;
    if (groups > 0 && group_tables && p.shape == kShapeDirect) {  // tables the caller built once for this grouping
        GroupTablesView v;
        group_tables_layout(const_cast<void*>(group_tables), rows, groups, experts, v);
        max_tiles64 = v.max64;
        p.expert_ids = expert_ids, p.tiles = v.t_sorted, p.num_tiles = v.counts, p.max_row_tiles = v.max_main;
        tiles64 = v.t64, num_tiles64 = v.counts + 1, ranges = v.ranges;
    } else if (groups > 0) {
        const bool wide = p.shape == kShapeWide;  // small groups: wide tiles; larger ones: a second, tall launch
        const int bm_main = p.shape == kShapeDirect ? kDirectBM : p.shape == kShapeTall ? kBM : kWideBM;
        const int max128 = wide ? (int)groups : (int)(rows / bm_main + groups);
        max_tall = wide ? (int)std::min<int64_t>(rows / kBM + groups, rows / (kWideBM + 1) + rows / kBM + 1) : 0;
        max_tiles64 = (int)(rows / 64 + groups);
        const bool direct = p.shape == kShapeDirect;  // its workgroups take the tiles with the most rows first
        TileDesc* t128 = (TileDesc*)bump.take((int64_t)max128 * sizeof(TileDesc));
        TileDesc* t_sorted = direct ? (TileDesc*)bump.take((int64_t)max128 * sizeof(TileDesc)) : nullptr;
        t_tall = wide ? (TileDesc*)bump.take((int64_t)max_tall * sizeof(TileDesc)) : nullptr;
        TileDesc* t64 = lora_a ? (TileDesc*)bump.take((int64_t)max_tiles64 * sizeof(TileDesc)) : nullptr;
        int* counts = (int*)bump.take(16);
        int* rg = lora_a ? (int*)bump.take(experts * 2 * 4) : nullptr;
        if (!t128 || !counts || (lora_a && (!t64 || !rg)) || (wide && !t_tall) || (direct && !t_sorted)) return set_error(GGQ_ERR_WORKSPACE, "%s: workspace too small", what);
        RowTileTables tb{};
        tb.add(bm_main, 0, wide ? kWideBM : 0x7FFFFFFF, t128, counts, t_sorted);
        if (direct) t128 = t_sorted;
        if (wide) tb.add(kBM, kWideBM, 0x7FFFFFFF, t_tall, counts + 2), n_tall = counts + 2;
        if (lora_a) tb.add(64, 0, 0x7FFFFFFF, t64, counts + 1);
        if (int rc = build_row_tile_tables(expert_ids, end_offsets, (int)groups, tb, rg, (int)experts, s)) return rc;
        p.expert_ids = expert_ids, p.tiles = t128, p.num_tiles = counts, p.max_row_tiles = max128;
        tiles64 = t64, num_tiles64 = counts + 1, ranges = rg;
    }
    if (lora_a) {
        // t = dy . B
        bf16_t* dyb = (bf16_t*)bump.take(rows * rp * 2);
        if (!dyb) return set_error(GGQ_ERR_WORKSPACE, "%s: workspace too small", what);
        if (rows > 0) {
            SkinnyNtParams sp{};
            sp.in[0] = (const bf16_t*)dy1, sp.in[1] = (const bf16_t*)dy2, sp.ld_in = n, sp.in_rows = dy_index;
            sp.f = (const bf16_t*)lora_b, sp.ldf = r, sp.f_expert_elems = (int64_t)r * ntot, sp.f_natural = 1;
            sp.out = dyb;
            sp.m = (int)rows, sp.c = (int)n, sp.r = r, sp.nseg = nseg;
            sp.expert_ids = groups > 0 ? expert_ids : nullptr, sp.tiles = tiles64, sp.num_tiles = num_tiles64;
            if (!skinny_nt_takes_natural_factor(sp)) {
                // B^T, so that both operands are contraction-contiguous
                bf16_t* bt = (bf16_t*)bump.take(experts * ntot * r * 2);
                if (!bt) return set_error(GGQ_ERR_WORKSPACE, "%s: workspace too small", what);
                if (int rc = transpose_factor((const bf16_t*)lora_b, bt, experts, (int)ntot, r, s)) return rc;
                sp.f = bt, sp.ldf = ntot, sp.f_natural = 0;
            }
            if (int rc = skinny_nt(sp, rp, max_tiles64, s)) return rc;
        }
        p.la = dyb, p.lb = (const bf16_t*)lora_a, p.lb_expert_elems = (int64_t)r * k, p.r_pad = rp, p.lora_rank = r, p.lora_scale = scale;
    }
    auto grad_input = [&]() -> int {
        if (rows == 0) return GGQ_OK;
        if (t_tall) return launch_wide_and_tall(qt, kModeNN, p, (int)rows, (int)n, (int)k, nseg, t_tall, n_tall, max_tall, s);
        return launch_mmq(qt, kModeNN, kEpiStore, p, s);
    };
    if (!lora_a || !(d_lora_a || d_lora_b)) return grad_input();
    float* partials = nullptr;
    int64_t partials_bytes = 0;
    if (groups == 0) {  // optional: without it the rows are not split
        partials_bytes = kDenseFactorSplits * std::max<int64_t>(ntot, k) * rp * 4;
        partials = (float*)bump.take(partials_bytes);
        if (!partials) partials_bytes = 0;
    }
    auto factor_gradients = [&](hipStream_t fs) -> int {
        if (d_lora_b) {
            FactorGradParams fp{};
            fp.partials = partials, fp.partials_bytes = partials_bytes;
            fp.in[0] = (const bf16_t*)dy1, fp.in[1] = (const bf16_t*)dy2, fp.ld_in = n, fp.in_rows = dy_index;
            fp.s = (const bf16_t*)xa, fp.out = (bf16_t*)d_lora_b, fp.out_expert_elems = ntot * r;
            fp.s_weights = row_weights, fp.s_weight_index = dy_index.row_index, fp.s_weights_are_bf16 = row_weights_are_bf16;
            fp.ranges = ranges, fp.m = (int)rows, fp.c = (int)n, fp.r = r, fp.nseg = nseg, fp.out_j_major = 0, fp.scale = scale;
            if (int rc = factor_grad(fp, rp, experts, fs)) return rc;
        }
        if (d_lora_a) {
            FactorGradParams fp{};
            fp.partials = partials, fp.partials_bytes = partials_bytes;
            fp.in[0] = (const bf16_t*)x, fp.ld_in = k, fp.in_rows = x_index;
            fp.s = (const bf16_t*)p.la, fp.out = (bf16_t*)d_lora_a, fp.out_expert_elems = (int64_t)r * k;
            fp.s_weights = row_weights, fp.s_weight_index = dy_index.row_index, fp.s_weights_are_bf16 = row_weights_are_bf16;
            fp.ranges = ranges, fp.m = (int)rows, fp.c = (int)k, fp.r = r, fp.nseg = 1, fp.out_j_major = 1, fp.scale = scale;
            if (int rc = factor_grad(fp, rp, experts, fs)) return rc;
        }
        return GGQ_OK;
    };
    if (rows > 0 && groups > 0) {
        // Expert groups: the factor gradients go out first, on the forked stream (they read dy, x, xa and dy . B, all complete
        // at the fork point, and write only dA / dB), then the grad-input launch on the caller's stream.  In that order the
        // short HBM-bound launches take their compute units at once and are done long before the join, and the grad-input
        // workgroups fill in behind them; the other way round the factor gradients trickle through whatever the grad-input
        // launch leaves free and the second of them runs exposed after it (0.943 against 0.931 ms per step on one box, 0.963
        // unforked).
        Forked side(s);
        if (side.stream() != s) {
            if (int rc = factor_gradients(side.stream())) return rc;
            if (int rc = grad_input()) return rc;
            return side.done();
        }
    }
    if (int rc = factor_gradients(s)) return rc;
    return grad_input();
}

int ggq_grouped_lora_mmq_backward(const void* dy1, const void* dy2, const void* packed1, const void* packed2,
                                  const int64_t* expert_ids, const int32_t* end_offsets, int64_t groups, int64_t experts, int qt,
                                  int64_t rows, int64_t n, int64_t k, const void* x, const void* xa, const void* lora_a,
                                  const void* lora_b, int r, float scale, void* dx, void* d_lora_a, void* d_lora_b,
                                  const void* group_tables, void* ws, int64_t ws_bytes, void* stream) {
    return grouped_backward("grouped_lora_mmq_backward", dy1, dy2, packed1, packed2, expert_ids, end_offsets, groups, experts, qt, rows, n, k, x,
                            RowIndex{}, xa, lora_a, lora_b, r, scale, dx, d_lora_a, d_lora_b, group_tables, ws, ws_bytes, stream);
}

// The backward of the indexed forward: x is the [x_rows, k] matrix the forward read through row_index (it is only
// read for the gradient of the factor A); dx comes out per expert-sorted row, [rows, k], as in the plain backward.
int ggq_grouped_lora_mmq_backward_indexed(const void* dy1, const void* dy2, const void* packed1, const void* packed2,
                                          const int64_t* expert_ids, const int32_t* end_offsets, int64_t groups, int64_t experts,
                                          int qt, int64_t rows, int64_t n, int64_t k, const void* x, int64_t x_rows,
                                          const int64_t* row_index, int index_div, const void* xa, const void* lora_a,
                                          const void* lora_b, int r, float scale, void* dx, void* d_lora_a, void* d_lora_b,
                                          const void* group_tables, void* ws, int64_t ws_bytes, void* stream) {
    const char* what = "grouped_lora_mmq_backward_indexed";
    if (!row_index) return set_error(GGQ_ERR_NULL, "%s: null row index", what);
    if (x_rows <= 0 || x_rows >= (1ll << 31) || index_div <= 0) return set_error(GGQ_ERR_SHAPE, "%s: bad x_rows=%lld or index_div=%d", what, (long long)x_rows, index_div);
    return grouped_backward(what, dy1, dy2, packed1, packed2, expert_ids, end_offsets, groups, experts, qt, rows, n, k, x,
                            RowIndex{row_index, index_div, (int)x_rows}, xa, lora_a, lora_b, r, scale, dx, d_lora_a, d_lora_b, group_tables, ws,
                            ws_bytes, stream);
}

// The backward of a projection whose output rows were scaled by routing weights and summed per token (the expert FFN's
// down projection followed by the combine): grad_out is the [tokens, n] cotangent of the COMBINED output; expert-sorted
// row i stands for weights[permutation[i]] * grad_out[permutation[i] / top_k].  dx_unscaled is dy . W (+ LoRA term) of
// the unweighted token rows; d_lora_a / d_lora_b carry the weights.
int ggq_grouped_lora_mmq_backward_routed_output(const void* grad_out, int64_t tokens, const int64_t* permutation, int top_k,
                                                const void* weights, int weights_are_bf16, const void* packed,
                                                const int64_t* expert_ids, const int32_t* end_offsets, int64_t groups, int64_t experts,
                                                int qt, int64_t rows, int64_t n, int64_t k, const void* x, const void* xa,
                                                const void* lora_a, const void* lora_b, int r, float scale, void* dx_unscaled,
                                                void* d_lora_a, void* d_lora_b, const void* group_tables, void* ws, int64_t ws_bytes,
                                                void* stream) {
    const char* what = "grouped_lora_mmq_backward_routed_output";
    if (!permutation || !weights) return set_error(GGQ_ERR_NULL, "%s: null permutation or weights", what);
    if (tokens <= 0 || tokens >= (1ll << 31) || top_k <= 0 || rows != tokens * top_k) return set_error(GGQ_ERR_SHAPE, "%s: rows must be tokens * top_k", what);
    return grouped_backward(what, grad_out, nullptr, packed, nullptr, expert_ids, end_offsets, groups, experts, qt, rows, n, k, x, RowIndex{}, xa,
                            lora_a, lora_b, r, scale, dx_unscaled, d_lora_a, d_lora_b, group_tables, ws, ws_bytes, stream,
                            RowIndex{permutation, top_k, (int)tokens}, weights, weights_are_bf16);
}

// ---------------------------------------------------------------------------------------------------
int64_t ggq_route_plan_workspace_bytes(int64_t tokens, int top_k, int num_experts) {
    return route_plan_workspace_bytes(tokens * top_k, num_experts) + 256;
}

int ggq_route_plan(const void* topk_ids, int ids_are_int64, int64_t tokens, int top_k, int num_experts, int64_t* sorted_ids,
                   int64_t* permutation, int64_t* inverse, int32_t* counts, int32_t* end_offsets, int64_t* active_ids,
                   int32_t* active_end_offsets, int32_t* status, void* ws, int64_t ws_bytes, void* stream) {
    if (!topk_ids || !sorted_ids || !permutation || !inverse || !counts || !end_offsets || !active_ids || !active_end_offsets || !status || !ws)
        return set_error(GGQ_ERR_NULL, "route_plan: null pointer");
    return route_plan(topk_ids, ids_are_int64, tokens, top_k, num_experts, sorted_ids, permutation, inverse, counts, end_offsets,
                      active_ids, active_end_offsets, status, ws, ws_bytes, as_stream(stream));
}

int ggq_route_plan_static(const void* topk_ids, int ids_are_int64, int64_t tokens, int top_k, int num_experts, int64_t* sorted_ids,
                          int64_t* permutation, int64_t* inverse, int32_t* counts, int32_t* end_offsets, int64_t* active_ids,
                          int32_t* active_end_offsets, int32_t* status, void* stream) {
    if (!topk_ids || !sorted_ids || !permutation || !inverse || !counts || !end_offsets || !active_ids || !active_end_offsets || !status)
        return set_error(GGQ_ERR_NULL, "route_plan_static: null pointer");
    return route_plan_static(topk_ids, ids_are_int64, tokens, top_k, num_experts, sorted_ids, permutation, inverse, counts, end_offsets,
                             active_ids, active_end_offsets, status, as_stream(stream));
}

int ggq_route_gather_forward(const void* hidden, const int64_t* permutation, void* selected, int64_t tokens, int top_k, int hidden_dim, void* stream) {
    if (!hidden || !permutation || !selected) return set_error(GGQ_ERR_NULL, "route_gather_forward: null pointer");
    return route_gather_fwd(hidden, permutation, selected, tokens, top_k, hidden_dim, as_stream(stream));
}

int ggq_route_gather_backward(const void* grad_selected, const int64_t* inverse, void* grad_hidden, int64_t tokens, int top_k, int hidden_dim, void* stream) {
    if (!grad_selected || !inverse || !grad_hidden) return set_error(GGQ_ERR_NULL, "route_gather_backward: null pointer");
    return route_gather_bwd(grad_selected, inverse, grad_hidden, tokens, top_k, hidden_dim, as_stream(stream));
}

int ggq_route_combine_forward(const void* expert_out, const void* weights, int weights_are_bf16, const int64_t* inverse, void* out, int64_t tokens, int top_k, int hidden_dim, void* stream) {
    if (!expert_out || !weights || !inverse || !out) return set_error(GGQ_ERR_NULL, "route_combine_forward: null pointer");
    return route_combine_fwd(expert_out, weights, weights_are_bf16, inverse, out, tokens, top_k, hidden_dim, as_stream(stream));
}

int ggq_route_combine_backward(const void* expert_out, const void* weights, int weights_are_bf16, const int64_t* permutation, const void* grad_out, void* grad_expert_out, void* grad_weights, int64_t tokens, int top_k, int hidden_dim, void* stream) {
    if (!expert_out || !weights || !permutation || !grad_out) return set_error(GGQ_ERR_NULL, "route_combine_backward: null pointer");
    return route_combine_bwd(expert_out, weights, weights_are_bf16, permutation, grad_out, grad_expert_out, grad_weights, tokens, top_k, hidden_dim, as_stream(stream));
}

int ggq_swiglu_forward(const void* gate, const void* up, void* h, int64_t elems, void* stream) {
    if (!gate || !up || !h) return set_error(GGQ_ERR_NULL, "swiglu_forward: null pointer");
    return swiglu_fwd(gate, up, h, elems, 0.0f, as_stream(stream));
}

int ggq_swiglu_clamped_forward(const void* gate, const void* up, void* h, int64_t elems, float limit, void* stream) {
    if (!gate || !up || !h) return set_error(GGQ_ERR_NULL, "swiglu_clamped_forward: null pointer");
    if (!(limit > 0.0f)) return set_error(GGQ_ERR_SHAPE, "swiglu_clamped_forward: the limit must be positive");
    return swiglu_fwd(gate, up, h, elems, limit, as_stream(stream));
}

int ggq_swiglu_backward(const void* gate, const void* up, const void* dh, void* dgate, void* dup, int64_t elems, void* stream) {
    if (!gate || !up || !dh || !dgate || !dup) return set_error(GGQ_ERR_NULL, "swiglu_backward: null pointer");
    return swiglu_bwd(gate, up, dh, dgate, dup, elems, 0.0f, as_stream(stream));
}

int ggq_swiglu_backward_routed(const void* gate, const void* up, const void* dh_unweighted, const void* weights, int weights_are_bf16,
                               const int64_t* permutation, void* dgate, void* dup, void* grad_weights, int64_t rows, int inter, float limit,
                               void* stream) {
    if (!gate || !up || !dh_unweighted || !weights || !permutation || !dgate || !dup) return set_error(GGQ_ERR_NULL, "swiglu_backward_routed: null pointer");
    return swiglu_bwd_routed(gate, up, dh_unweighted, weights, weights_are_bf16, permutation, dgate, dup, grad_weights, rows, inter, limit, as_stream(stream));
}

int ggq_swiglu_clamped_backward(const void* gate, const void* up, const void* dh, void* dgate, void* dup, int64_t elems, float limit, void* stream) {
    if (!gate || !up || !dh || !dgate || !dup) return set_error(GGQ_ERR_NULL, "swiglu_clamped_backward: null pointer");
    if (!(limit > 0.0f)) return set_error(GGQ_ERR_SHAPE, "swiglu_clamped_backward: the limit must be positive");
    return swiglu_bwd(gate, up, dh, dgate, dup, elems, limit, as_stream(stream));
}

int64_t ggq_gmm_workspace_bytes(int64_t experts) { return grouped_gemm_workspace_bytes(experts); }

int ggq_gmm(const void* lhs, const void* rhs, const int32_t* group_sizes, void* out, int64_t m, int64_t k, int64_t n, int64_t experts, int rhs_k_contiguous,
            int is_f16, void* ws, int64_t ws_bytes, void* stream) {
    return grouped_gemm(lhs, rhs, group_sizes, out, m, k, n, experts, rhs_k_contiguous, is_f16, ws, ws_bytes, as_stream(stream));
}

int ggq_ptgmm(const void* lhs, const void* grad_out, const int32_t* group_sizes, void* out, int64_t m, int64_t k, int64_t n, int64_t experts, int is_f16,
              void* ws, int64_t ws_bytes, void* stream) {
    return grouped_gemm_transposed(lhs, grad_out, group_sizes, out, m, k, n, experts, is_f16, ws, ws_bytes, as_stream(stream));
}

int ggq_router_topk(const void* logits, int logits_are_bf16, int64_t tokens, int num_experts, int top_k, const float* correction_bias,
                    int score_function, int64_t* indices, void* weights, int weights_mode, float routed_scaling, void* stream) {
    return router_topk(logits, logits_are_bf16, tokens, num_experts, top_k, correction_bias, score_function, indices, weights,
                       weights_mode, routed_scaling, as_stream(stream));
}

// ---------------------------------------------------------------------------------------------------
int64_t ggq_lmhead_ce_workspace_bytes(int64_t rows, int64_t vocab, int64_t hidden_dim, int64_t chunk) {
    return lmhead_ce_workspace_bytes(rows, vocab, hidden_dim, chunk);
}

int ggq_lmhead_cross_entropy(int qt, const void* hidden, const void* packed, const int64_t* labels, int64_t rows, int64_t vocab,
                             int64_t hidden_dim, int64_t chunk, int64_t ignore_index, int reduction_mean, float* loss_per_row,
                             void* grad_hidden, float* lse_out, int32_t* status_out, int64_t* predicted_tokens, float* token_correct, void* ws,
                             int64_t ws_bytes, void* stream) {
    if (int rc = check_weights("lmhead_cross_entropy", qt, packed, hidden_dim)) return rc;
    return lmhead_ce(qt, hidden, packed, labels, rows, vocab, hidden_dim, chunk, ignore_index, reduction_mean, loss_per_row,
                     grad_hidden, lse_out, status_out, predicted_tokens, token_correct, ws, ws_bytes, as_stream(stream));
}

}  // extern "C"
