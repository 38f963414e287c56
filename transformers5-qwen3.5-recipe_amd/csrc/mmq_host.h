// Parameter blocks and host launchers shared between the translation units of the library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ggq {

typedef uint16_t bf16_t;

struct TileDesc {  // one row tile of an expert group: rows [row_begin, row_end) of group `group`, whose weights are plane `expert`
    int group, row_begin, row_end, expert;
};

// Rows read through an index: logical row i of an operand is its stored row row_index[i] / index_div (clamped to
// index_rows - 1), so expert-sorted routes can read the token matrix in place: row_index = the sorted-position ->
// route permutation, index_div = routes per token.  A null row_index means stored row i.
struct RowIndex {
    const int64_t* row_index;
    int index_div, index_rows;
    __host__ __device__ bool on() const { return row_index != nullptr; }
#if defined(__HIPCC__)
    __device__ __forceinline__ int source(int i) const {
        return row_index ? min((int)((uint32_t)row_index[i] / (uint32_t)index_div), index_rows - 1) : i;
    }
#endif
};

struct SkinnyNtParams {
    const bf16_t* in[2];  // [m, c] per segment
    int64_t ld_in;
    RowIndex in_rows;     // segment 0 only (nseg == 1 when set)
    const bf16_t* f;      // per expert [r][ldf], contraction contiguous; or [nseg*c][r] when f_natural
    int64_t ldf, f_expert_elems;
    int f_natural;
    bf16_t* out;          // [m, r_pad]
    int m, c, r, nseg;
    const int64_t* expert_ids;
    const TileDesc* tiles;  // 64-row tiles (null: dense)
    const int* num_tiles;
};

struct FactorGradParams {
    const bf16_t* in[2];  // [m, c] per segment
    int64_t ld_in;
    RowIndex in_rows;     // segment 0 only (nseg == 1 when set)
    const bf16_t* s;      // [m, r_pad]
    // optional factor per row of s: row i is scaled by weights[index[i]] (fp32 or bf16 weights) and rounded to bf16 again
    const void* s_weights;
    const int64_t* s_weight_index;
    int s_weights_are_bf16;
    bf16_t* out;          // per expert: [nseg*c][r] (out_j_major = 0) or [r][nseg*c] (= 1)
    int64_t out_expert_elems;
    const int* ranges;    // per expert (row_begin, row_end); null: all m rows, one expert
    int m, c, r, nseg, out_j_major;
    float scale;
    int units;            // experts * column blocks * row splits (set by factor_grad)
    // one row range for all (ranges == null) and a scratch buffer: the rows are dealt to row_splits workgroups per column
    // block, whose fp32 partial sums [row_splits][nseg*c][r_pad] a second kernel adds in split order (set by factor_grad)
    float* partials;      // null: no splitting
    int64_t partials_bytes;
    int row_splits;
};

constexpr int kBM = 256, kBN = 128, kBK = 64;  // the tall tile shape (dense launches, large expert groups)
constexpr int kWideBM = 128, kWideBN = 256;    // the wide tile shape (Q4_K expert groups of about a hundred rows)
constexpr int kDirectBM = 192, kDirectBN = 256;  // the direct shape (Q4_K expert groups: the MFMA waves decode the weights themselves)
constexpr int kSmallBM = 128, kSmallBN = 256;   // the small shape (IQ2_XXS forward, expert groups of at most 128 rows: decoding waves)
constexpr int kShapeTall = 0, kShapeWide = 1, kShapeDirect = 3;
constexpr int kShapeSmall = 5;  // (a launch beside the wide and tall tiles of a call, never the shape of a whole call)
constexpr int kShapeMixed = 4;  // (profile records only: one launch of wide and tall tiles)
constexpr int kLdsStride = kBK + 8;  // bf16 elements per LDS row: 144 bytes keeps 128-bit reads conflict-free
constexpr int kThreads = 1024;  // waves 0..7 run the MFMAs, waves 8..15 load and decode

enum : int { kModeNT = 0, kModeNN = 1 };
enum : int {
    kEpiStore = 0,     // C (bf16) = acc
    kEpiAccumF32 = 1   // C32 (fp32) = C32 * row_scale[m] + acc  (row_scale null: += acc)
};

struct MmqParams {
    const bf16_t* a[2];   // activations; [1] only for a pair in NN mode
    int64_t lda;
    RowIndex a_rows;      // rows of a[0] read through an index (one segment only; the matrix stays under 4 GiB)
    int a_zero_padded;    // the rows of a hold zeros from the contraction length up to the next multiple of 64 (lda covers them):
                          // a contraction that ends inside a 64-wide step still takes the aligned 16-byte loads
    const uint8_t* w[2];  // packed weights; [1] only for a pair
    int64_t w_row_bytes, w_expert_bytes;
    void* c[2];           // outputs; [1] only for a pair in NT mode
    int64_t ldc;
    int m, n, k;          // W segment is [n, k]
    int nseg;             // 1, or 2 for a pair
    int col_tiles_per_seg;  // NT: ceil(n/256); NN: ceil(k/256) (nseg applies to contraction there)
    int steps_per_seg;      // NT: k/64; NN: ceil(n/64)
    // expert groups (null tiles => one dense group of m rows)
    const int64_t* expert_ids;
    const TileDesc* tiles;
    const int* num_tiles;
    int max_row_tiles;
    // second table of a mixed launch (tall tiles; `tiles` then holds the wide ones)
    const TileDesc* tiles2;
    const int* num_tiles2;
    int max_row_tiles2;
    int col_tiles_per_seg2;
    int col_tiles_per_wg;   // direct shape: column tiles one workgroup walks through (>= 1)
    int shape;  // kShapeTall / kShapeWide / kShapeDirect: which kernel the sizes above are for
    // LoRA
    const bf16_t* la;     // [rows, r_pad]  (x A^T in NT, dY B in NN)
    const bf16_t* lb;     // per expert: NT [cols_total, r_pad] (rows of B); NN [lora_rank, k] (the factor A as it is)
    int64_t lb_expert_elems;
    int r_pad;            // multiple of 16, <= 64; 0 = no LoRA
    int lora_rank;        // NN mode: rows of the factor A that exist (the tile's rows up to r_pad are zero)
    float lora_scale;
    const float* row_scale;    // accumulate epilogue: [m] factors of the old accumulator rows (null: 1)
};

constexpr int kMaxTimedLaunches = 8192;
int profile_begin();
int profile_end(float* ms, int* qt, int* mode, int* epi, int* shape, int capacity);
int measure_mfma_ceiling(const void* a_samples, const void* b_samples, int64_t elems, int iters, void* sink_buffer, float* tflops_out, hipStream_t s);
const char* last_error();
int launch_mmq(int qt, int mode, int epi, const MmqParams& p, hipStream_t s);
int launch_mmq_mixed(int qt, int mode, const MmqParams& p, hipStream_t s);  // Q4_K, store epilogue, tiles + tiles2
int launch_mmq_small(const MmqParams& p, hipStream_t s);  // IQ2_XXS forward, store epilogue, tiles of kSmallBM rows
int init_params(MmqParams& p, int qt, int mode, int m, int n, int k, int nseg, int shape = kShapeTall);

int pad_factor(const bf16_t* src, bf16_t* dst, int64_t experts, int c, int r, int r_pad, bool transpose, hipStream_t s);
int transpose_factor(const bf16_t* src, bf16_t* dst, int64_t experts, int c, int r, hipStream_t s);
int skinny_nt(const SkinnyNtParams& p, int r_pad, int grid_tiles, hipStream_t s);
bool skinny_nt_takes_natural_factor(const SkinnyNtParams& p);
int factor_grad(const FactorGradParams& p, int r_pad, int64_t experts, hipStream_t s);

// Builds the row-tile table of an expert-sorted layout on the device (no host sync):
// tiles[0..*num_tiles) in group order, tile height bm; optionally per-expert row ranges.
// Up to four row-tile tables built by one launch (one workgroup each).
struct RowTileTables {
    int count;
    int bm[4], min_rows[4], max_rows[4];
    TileDesc* tiles[4];
    int* num_tiles[4];
    // not null: the table also goes here ordered by descending number of 32-row blocks (ties in group order), so that
    // workgroups dispatched in table order take the most expensive tiles first
    TileDesc* by_size[4];
    void add(int bm_, int min_rows_, int max_rows_, TileDesc* tiles_, int* num_tiles_, TileDesc* by_size_ = nullptr) {
        bm[count] = bm_, min_rows[count] = min_rows_, max_rows[count] = max_rows_, tiles[count] = tiles_, num_tiles[count] = num_tiles_;
        by_size[count] = by_size_;
        count++;
    }
};
int build_row_tile_tables(const int64_t* expert_ids, const int32_t* end_offsets, int groups, const RowTileTables& tb,
                          int* expert_ranges, int num_experts, hipStream_t s);
int build_row_tiles(const int64_t* expert_ids, const int32_t* end_offsets, int groups, int bm, TileDesc* tiles,
                    int* num_tiles, int* expert_ranges, int num_experts, hipStream_t s, int min_rows = 0, int max_rows = 0x7FFFFFFF);

int64_t route_plan_workspace_bytes(int64_t routes, int num_experts);
int route_plan(const void* topk_ids, int ids_are_int64, int64_t tokens, int top_k, int num_experts,
               int64_t* sorted_ids, int64_t* permutation, int64_t* inverse, int* counts, int* end_offsets,
               int64_t* active_ids, int* active_end, int* num_active, void* ws, int64_t ws_bytes, hipStream_t s);
int route_plan_static(const void* topk_ids, int ids_are_int64, int64_t tokens, int top_k, int num_experts,
                      int64_t* sorted_ids, int64_t* permutation, int64_t* inverse, int* counts, int* end_offsets,
                      int64_t* active_ids, int* active_end, int* num_active, hipStream_t s);  // no workspace: a built-in scratch array
int route_gather_fwd(const void* hidden, const int64_t* permutation, void* selected, int64_t tokens, int top_k, int hidden_dim, hipStream_t s);
int route_gather_bwd(const void* grad_selected, const int64_t* inverse, void* grad_hidden, int64_t tokens, int top_k, int hidden_dim, hipStream_t s);
int route_combine_fwd(const void* expert_out, const void* weights, int w_is_bf16, const int64_t* inverse, void* out, int64_t tokens, int top_k, int hidden_dim, hipStream_t s);
int route_combine_bwd(const void* expert_out, const void* weights, int w_is_bf16, const int64_t* permutation, const void* grad_out, void* grad_expert_out, void* grad_weights, int64_t tokens, int top_k, int hidden_dim, hipStream_t s);
int router_topk(const void* logits, int logits_are_bf16, int64_t tokens, int num_experts, int top_k, const float* bias, int score_fn,
                int64_t* indices, void* weights, int weights_mode, float scale, hipStream_t s);
int swiglu_fwd(const void* gate, const void* up, void* h, int64_t elems, float limit, hipStream_t s);
int swiglu_bwd(const void* gate, const void* up, const void* dh, void* dgate, void* dup, int64_t elems, float limit, hipStream_t s);
int swiglu_bwd_routed(const void* gate, const void* up, const void* dh, const void* weights, int w_is_bf16, const int64_t* permutation,
                      void* dgate, void* dup, void* grad_weights, int64_t routes, int inter, float limit, hipStream_t s);

int64_t lmhead_ce_workspace_bytes(int64_t rows, int64_t vocab, int64_t hidden, int64_t chunk);
int lmhead_ce(int qt, const void* hidden, const void* packed, const int64_t* labels, int64_t rows, int64_t vocab,
              int64_t hidden_dim, int64_t chunk, int64_t ignore_index, int reduction_mean, float* loss_1d,
              void* grad_hidden, float* lse_out, int* n_valid_out, int64_t* predicted, float* correct, void* ws, int64_t ws_bytes, hipStream_t s);

int dequantize(int qt, const void* payload, int64_t rows, int64_t k, void* out, int out_f32, hipStream_t stream);

// Grouped bf16 / fp16 products without packed weights (grouped_gemm.hip): out[rows of e] = lhs[rows of e] . rhs[e] with rhs[e] stored
// [n][k] (rhs_k_contiguous) or [k][n]; and out[e] = lhs[rows of e]^T . grad_out[rows of e].
int64_t grouped_gemm_workspace_bytes(int64_t experts);
int grouped_gemm(const void* lhs, const void* rhs, const int32_t* group_sizes, void* out, int64_t m, int64_t k, int64_t n, int64_t experts, int rhs_k_contiguous,
                 int is_f16, void* ws, int64_t ws_bytes, hipStream_t stream);
int grouped_gemm_transposed(const void* lhs, const void* grad_out, const int32_t* group_sizes, void* out, int64_t m, int64_t k, int64_t n, int64_t experts,
                            int is_f16, void* ws, int64_t ws_bytes, hipStream_t stream);

}  // namespace ggq
