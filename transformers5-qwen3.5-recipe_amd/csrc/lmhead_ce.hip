// Chunked cross-entropy through a packed lm_head without ever holding [rows, vocab] logits.
//
// The caller's chunk is the memory contract, as in the reference, whose loop holds one [chunk, vocab] logits tensor at a time:
//  * chunk >= 4096 rows (or >= all rows): the logits of a chunk are kept.  Per chunk: one launch of the packed-weight tile
//    kernel writes its bf16 logits; one kernel, a workgroup per row, reads a row for its log-sum-exp, target logit and loss
//    and rewrites it as d(loss)/d(logits); one grad-input launch contracts the rows with the packed weights over the whole
//    vocabulary.  Two vocabulary-sized matmuls.
//  * smaller chunks: no logits are kept beyond a [rows, 8192] slab.  Per block of up to kGradRows rows the vocabulary is
//    swept once in blocks of kVocabBlock columns with a running (max, sum exp) per row: the tile kernel writes the block's
//    logits into the slab; a row kernel updates the running statistics and rewrites the slab as exp(logit - running max);
//    the grad-input form of the tile kernel adds slab . W_block to an fp32 accumulator that its epilogue first rescales
//    by exp(old max - new max).  At the end dH = (accumulator / sum - W[label]) * row_scale.  Two vocabulary-sized
//    matmuls here as well.
#include <algorithm>

#include "common.h"
#include "launch.h"
#include "mmq_host.h"

namespace ggq {

constexpr int kVocabBlock = 8192;
// The sweep takes up to this many rows at a time, whatever the caller's chunk (which stands for the reference's
// [chunk, vocab] logits): 4096 rows fill the chip with tiles of the [rows, hidden] grad-input output (a 1024-row chunk
// makes 64 tiles for 256 compute units) and cost a 64 MiB slab.
constexpr int64_t kGradRows = 4096;
// A chunk of at least this many rows is worth keeping the logits of: its grad-input launch fills the chip.
constexpr int64_t kKeptLogitsRows = 4096;

// row_scale[m] = 0 for ignored rows, else 1/n_valid (mean) or 1 (sum); n_valid = 0 gives all zeros.  A label outside
// [0, vocab) that is not ignore_index is treated as ignored (no loss, no gradient) and counted in status[1].
__device__ __forceinline__ bool label_counts(int64_t label, int64_t vocab, int64_t ignore_index) {
    return label != ignore_index && label >= 0 && label < vocab;
}
__global__ __launch_bounds__(1024) void ce_row_scale_kernel(const int64_t* labels, int64_t rows, int64_t vocab, int64_t ignore_index,
                                                             int mean, float* row_scale, int* status) {
    __shared__ int partial[1024], partial_bad[1024];
    int c = 0, bad = 0;
    for (int64_t i = threadIdx.x; i < rows; i += 1024) {
        const int64_t l = labels[i];
        c += label_counts(l, vocab, ignore_index);
        bad += l != ignore_index && (l < 0 || l >= vocab);
    }
    partial[threadIdx.x] = c, partial_bad[threadIdx.x] = bad;
    __syncthreads();
    for (int off = 512; off >= 1; off >>= 1) {
        if ((int)threadIdx.x < off) partial[threadIdx.x] += partial[threadIdx.x + off], partial_bad[threadIdx.x] += partial_bad[threadIdx.x + off];
        __syncthreads();
    }
    const int n = partial[0];
    const float scale = n == 0 ? 0.f : (mean ? 1.0f / (float)n : 1.0f);
    for (int64_t i = threadIdx.x; i < rows; i += 1024) row_scale[i] = label_counts(labels[i], vocab, ignore_index) ? scale : 0.f;
    if (threadIdx.x == 0 && status) status[0] = n, status[1] = partial_bad[0];
}

__global__ void fill_f32_kernel(float* p, int64_t n, float v) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = v;
}

static unsigned grid1d(int64_t n) {
    int64_t g = (n + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 16384 ? 16384 : g));
}

// One workgroup per row.  Pass 1: log-sum-exp of the row's logits (every lane keeps a running (max, sum) over its columns,
// merged in lane order inside a wave and in wave order across the workgroup: deterministic), the target logit, the loss
// (lse - target) * row_scale.  Pass 2: the row becomes (exp(logit - lse) - [column == label]) * row_scale in place, bf16;
// the padding columns [vocab, ld) become zero.  Eight columns per lane and trip (ld is a multiple of 64).
__device__ __forceinline__ void merge_max_sum(float& m, float& s, float m2, float s2) {
    const float mx = fmaxf(m, m2);
    s = (m == -INFINITY ? 0.f : s * __expf(m - mx)) + (m2 == -INFINITY ? 0.f : s2 * __expf(m2 - mx));
    m = mx;
}

// (value, column) of the better of two candidates: the larger value, and among equal values the smaller column (the first
// maximum of the row, the choice of an argmax that scans the columns in order)
__device__ __forceinline__ void merge_arg(float& v, int& i, float v2, int i2) {
    if (v2 > v || (v2 == v && i2 < i)) v = v2, i = i2;
}

__global__ __launch_bounds__(256) void ce_loss_and_grad_kernel(bf16_t* logits, int64_t ld, int64_t vocab, const int64_t* labels, const float* row_scale,
                                                               float* lse_out, float* loss_out, int64_t ignore_index, int64_t* predicted, float* correct) {
    __shared__ float wave_m[4], wave_s[4], wave_bv[4];
    __shared__ int wave_bi[4];
    const int64_t row = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint4* p = (uint4*)(logits + row * ld);
    const int64_t label = labels[row];
    const float rs = row_scale[row];
    float m = -INFINITY, sum = 0.f;
    float bv = -INFINITY;  // this lane's best logit and its column (its columns come in ascending order: strict > keeps the first)
    int bi = 0x7FFFFFFF;
    for (int64_t c8 = threadIdx.x; c8 < ld / 8; c8 += 256) {
        const uint4 v = p[c8];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        float x[8];
        float cm = -INFINITY;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            x[e] = c8 * 8 + e < vocab ? bf16_to_f32((bf16_t)((e & 1) ? w[e >> 1] >> 16 : w[e >> 1] & 0xFFFFu)) : -INFINITY;
            cm = fmaxf(cm, x[e]);
        }
        if (cm == -INFINITY) continue;  // padding only
        if (cm > bv) {
            bv = cm;
#pragma unroll
            for (int e = 7; e >= 0; e--)
                if (x[e] == cm) bi = (int)(c8 * 8 + e);
        }
        float cs = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) cs += x[e] == -INFINITY ? 0.f : __expf(x[e] - cm);
        merge_max_sum(m, sum, cm, cs);
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float m2 = __shfl_xor(m, off, 64), s2 = __shfl_xor(sum, off, 64);
        merge_max_sum(m, sum, m2, s2);
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float v2 = __shfl_xor(bv, off, 64);
        const int i2 = __shfl_xor(bi, off, 64);
        merge_arg(bv, bi, v2, i2);
    }
    if (lane == 0) wave_m[wave] = m, wave_s[wave] = sum, wave_bv[wave] = bv, wave_bi[wave] = bi;
    __syncthreads();
    m = wave_m[0], sum = wave_s[0];
#pragma unroll
    for (int w = 1; w < 4; w++) merge_max_sum(m, sum, wave_m[w], wave_s[w]);
    const float lse = m + __logf(sum);
    if (threadIdx.x == 0) {
        lse_out[row] = lse;
        const bool counts = label_counts(label, vocab, ignore_index);
        const float target = counts ? bf16_to_f32(logits[row * ld + label]) : 0.f;
        loss_out[row] = rs != 0.f ? (lse - target) * rs : 0.f;
        bv = wave_bv[0], bi = wave_bi[0];
#pragma unroll
        for (int w = 1; w < 4; w++) merge_arg(bv, bi, wave_bv[w], wave_bi[w]);
        if (predicted) predicted[row] = counts ? (int64_t)bi : -1;
        if (correct) correct[row] = counts && (int64_t)bi == label ? 1.0f : 0.0f;
    }
    __syncthreads();  // the target logit is read before the row is overwritten
    for (int64_t c8 = threadIdx.x; c8 < ld / 8; c8 += 256) {
        const uint4 v = p[c8];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        uint32_t o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float g[2];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int64_t col = c8 * 8 + 2 * e + h;
                const float logit = bf16_to_f32((bf16_t)(h ? w[e] >> 16 : w[e] & 0xFFFFu));
                float d = __expf(logit - lse);
                if (col == label && rs != 0.f) d -= 1.0f;
                g[h] = col < vocab ? d * rs : 0.0f;
            }
            o[e] = pack_bf16(g[0], g[1]);
        }
        p[c8] = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// ---- the form that keeps no logits: one sweep over the vocabulary in blocks of kVocabBlock columns with a running
// (max, sum exp) per row, as in a streaming softmax.  Per block and row: the block's logits (a [rows, kVocabBlock] slab
// written by the tile kernel) become p = exp(logit - running max) in place (bf16), alpha = exp(old max - new max) rescales
// what was accumulated so far, and the grad-input launch adds p . W_block to the fp32 accumulator it first multiplied by
// alpha.  At the end dH = ((acc / sum) - W[label]) * row_scale.  One workgroup per row.
__global__ __launch_bounds__(256) void ce_stream_block_kernel(bf16_t* slab, int64_t ld, int nb, int64_t v0, const int64_t* labels, float* run_max,
                                                              float* run_sum, float* target, float* alpha, int64_t* run_arg) {
    __shared__ float red[4];
    __shared__ int red_i[4];
    const int64_t row = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint4* p = (uint4*)(slab + row * ld);
    const int chunks = (nb + 63) / 64 * 8;  // the contraction of the grad-input launch runs to the next multiple of 64
    float bm = -INFINITY;
    for (int c8 = threadIdx.x; c8 < chunks; c8 += 256) {
        const uint4 v = p[c8];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 8; e++)
            if (c8 * 8 + e < nb) bm = fmaxf(bm, bf16_to_f32((bf16_t)((e & 1) ? w[e >> 1] >> 16 : w[e >> 1] & 0xFFFFu)));
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) bm = fmaxf(bm, __shfl_xor(bm, off, 64));
    if (lane == 0) red[wave] = bm;
    __syncthreads();
    bm = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    const float m_old = run_max[row];
    const float m_new = fmaxf(m_old, bm);
    const int64_t label = labels[row];
    if (threadIdx.x == 0 && label >= v0 && label < v0 + nb) target[row] = bf16_to_f32(slab[row * ld + (label - v0)]);  // (an ignore_index inside the range is masked by its zero row scale)
    __syncthreads();  // the target logit is read before the row is overwritten
    float sum = 0.f;
    int first = 0x7FFFFFFF;  // first column of the block that holds the block's maximum
    for (int c8 = threadIdx.x; c8 < chunks; c8 += 256) {
        const uint4 v = p[c8];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        uint32_t o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float g[2];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const float logit = bf16_to_f32((bf16_t)(h ? w[e] >> 16 : w[e] & 0xFFFFu));
                const int col = c8 * 8 + 2 * e + h;
                if (col < nb && logit == bm) first = min(first, col);
                g[h] = col < nb ? __expf(logit - m_new) : 0.0f;
            }
            o[e] = pack_bf16(g[0], g[1]);
            // the sum runs over the rounded values the accumulator receives, so that numerator and denominator agree
            sum += bf16_to_f32((bf16_t)(o[e] & 0xFFFFu)) + bf16_to_f32((bf16_t)(o[e] >> 16));
        }
        p[c8] = make_uint4(o[0], o[1], o[2], o[3]);
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) sum += __shfl_xor(sum, off, 64);
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) first = min(first, __shfl_xor(first, off, 64));
    if (lane == 0) red[wave] = sum, red_i[wave] = first;
    __syncthreads();
    if (threadIdx.x == 0) {
        // a later block takes the argmax over only with a strictly larger maximum: equal maxima keep the first column
        if (run_arg && bm > m_old) run_arg[row] = v0 + min(min(red_i[0], red_i[1]), min(red_i[2], red_i[3]));
        const float a = m_old == -INFINITY ? 0.f : __expf(m_old - m_new);
        alpha[row] = a;
        run_sum[row] = run_sum[row] * a + ((red[0] + red[1]) + (red[2] + red[3]));
        run_max[row] = m_new;
    }
}

// Packed rows of the labels (row 0 for ignored or out-of-range labels: their gradient is zero or undefined anyway).
__global__ __launch_bounds__(256) void gather_label_rows_kernel(const uint8_t* packed, int64_t row_bytes, const int64_t* labels, int64_t vocab, uint8_t* out) {
    const int64_t row = blockIdx.x;
    const int64_t label = labels[row];
    const uint16_t* src = (const uint16_t*)(packed + (label >= 0 && label < vocab ? label : 0) * row_bytes);
    uint16_t* dst = (uint16_t*)(out + row * row_bytes);
    for (int64_t i = threadIdx.x; i < row_bytes / 2; i += 256) dst[i] = src[i];
}

// lse, loss and dH = ((acc / sum) - W[label]) * row_scale, rounded to bf16.  One workgroup per row.
__global__ __launch_bounds__(256) void ce_stream_finish_kernel(const float* acc, const bf16_t* w_label, int64_t hidden, const int64_t* labels, int64_t vocab,
                                                               const float* run_max, const float* run_sum, const float* target, const float* row_scale,
                                                               float* lse_out, float* loss_out, bf16_t* grad_hidden, int64_t ignore_index,
                                                               const int64_t* run_arg, int64_t* predicted, float* correct) {
    const int64_t row = blockIdx.x;
    const float rs = row_scale[row], inv = 1.0f / run_sum[row];
    const int64_t label = labels[row];
    const bool has_target = label_counts(label, vocab, ignore_index);
    if (threadIdx.x == 0) {
        const float lse = run_max[row] + __logf(run_sum[row]);
        lse_out[row] = lse;
        loss_out[row] = rs != 0.f ? (lse - (has_target ? target[row] : 0.f)) * rs : 0.f;
        if (run_arg) {
            const int64_t arg = run_arg[row];
            if (correct) correct[row] = has_target && arg == label ? 1.0f : 0.0f;
            if (predicted) predicted[row] = has_target ? arg : -1;  // (may be the running storage itself: read first)
        }
    }
    for (int64_t c = threadIdx.x; c < hidden; c += 256) {
        const float wl = has_target ? bf16_to_f32(w_label[row * hidden + c]) : 0.f;
        grad_hidden[row * hidden + c] = to_bf16((acc[row * hidden + c] * inv - wl) * rs);
    }
}

static int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

static int64_t padded_vocab(int64_t vocab) { return (vocab + 63) / 64 * 64; }

static bool keeps_logits(int64_t rows, int64_t chunk) { return chunk >= rows || chunk >= kKeptLogitsRows; }

int64_t lmhead_ce_workspace_bytes(int64_t rows, int64_t vocab, int64_t hidden, int64_t chunk) {
    if (keeps_logits(rows, chunk)) return align256(rows * 4) * 2 + align256(std::min(rows, chunk) * padded_vocab(vocab) * 2) + 1024;
    const int64_t gr = std::min(rows, kGradRows);
    return align256(rows * 4) * 6 + align256(rows * 8) + align256(gr * kVocabBlock * 2) + align256(gr * hidden * 4) + align256(gr * hidden * 2) * 2 + 1024;
}

// The kept-logits path: row blocks of one chunk each.
static int lmhead_ce_kept_logits(int qt, const void* hidden, const void* packed, const int64_t* labels, int64_t rows, int64_t vocab,
                                 int64_t hidden_dim, int64_t chunk, int64_t ignore_index, int reduction_mean, float* loss_1d,
                                 void* grad_hidden, float* lse_out, int* n_valid_out, int64_t* predicted, float* correct, void* ws, hipStream_t s) {
    const int64_t br_max = std::min(rows, chunk);
    const int64_t ld = padded_vocab(vocab);
    char* w = (char*)ws;
    float* row_scale = (float*)w; w += align256(rows * 4);
    float* lse = lse_out ? lse_out : (float*)w; w += align256(rows * 4);
    bf16_t* logits = (bf16_t*)w;  // [br_max, ld]

    hipLaunchKernelGGL(ce_row_scale_kernel, dim3(1), dim3(1024), 0, s, labels, rows, vocab, ignore_index, reduction_mean, row_scale, n_valid_out);
    for (int64_t b0 = 0; b0 < rows; b0 += br_max) {
        const int br = (int)std::min(rows - b0, br_max);
        // (1) logits = hidden . W^T
        MmqParams p;
        if (int rcode = init_params(p, qt, kModeNT, br, (int)vocab, (int)hidden_dim, 1)) return rcode;
        p.a[0] = (const bf16_t*)hidden + b0 * hidden_dim, p.lda = hidden_dim;
        p.w[0] = (const uint8_t*)packed;
        p.c[0] = logits, p.ldc = ld;
        if (int rcode = launch_mmq(qt, kModeNT, kEpiStore, p, s)) return rcode;
        // (2) loss per row; the logits become the gradient with respect to them
        hipLaunchKernelGGL(ce_loss_and_grad_kernel, dim3((unsigned)br), dim3(256), 0, s, logits, ld, vocab, labels + b0, row_scale + b0, lse + b0, loss_1d + b0,
                           ignore_index, predicted ? predicted + b0 : nullptr, correct ? correct + b0 : nullptr);
        // (3) dH = dlogits . W over the whole vocabulary
        MmqParams g;
        if (int rcode = init_params(g, qt, kModeNN, br, (int)vocab, (int)hidden_dim, 1)) return rcode;
        g.a[0] = logits, g.lda = ld, g.a_zero_padded = 1;
        g.w[0] = (const uint8_t*)packed;
        g.c[0] = (bf16_t*)grad_hidden + b0 * hidden_dim, g.ldc = hidden_dim;
        if (int rcode = launch_mmq(qt, kModeNN, kEpiStore, g, s)) return rcode;
    }
    return check_launch("lmhead_ce");
}

int lmhead_ce(int qt, const void* hidden, const void* packed, const int64_t* labels, int64_t rows, int64_t vocab,
              int64_t hidden_dim, int64_t chunk, int64_t ignore_index, int reduction_mean, float* loss_1d,
              void* grad_hidden, float* lse_out, int* n_valid_out, int64_t* predicted, float* correct, void* ws, int64_t ws_bytes, hipStream_t s) {
    if (rows < 0 || vocab <= 0 || hidden_dim <= 0 || chunk <= 0) return set_error(GGQ_ERR_SHAPE, "lmhead_ce: bad shape");
    if (rows >= (1 << 30) || vocab >= (1 << 30)) return set_error(GGQ_ERR_SHAPE, "lmhead_ce: shape too large");
    if (!hidden || !packed || !labels || !loss_1d || !grad_hidden || !ws) return set_error(GGQ_ERR_NULL, "lmhead_ce: null pointer");
    if (ws_bytes < lmhead_ce_workspace_bytes(rows, vocab, hidden_dim, chunk)) return set_error(GGQ_ERR_WORKSPACE, "lmhead_ce: workspace too small");
    if (((uintptr_t)hidden | (uintptr_t)packed | (uintptr_t)grad_hidden | (uintptr_t)ws) & 15) return set_error(GGQ_ERR_ALIGN, "lmhead_ce: pointers must be 16-byte aligned");
    if (rows == 0) return GGQ_OK;
    if (keeps_logits(rows, chunk))
        return lmhead_ce_kept_logits(qt, hidden, packed, labels, rows, vocab, hidden_dim, chunk, ignore_index, reduction_mean, loss_1d, grad_hidden,
                                     lse_out, n_valid_out, predicted, correct, ws, s);
    // One sweep over the vocabulary per block of up to kGradRows rows; nothing wider than kVocabBlock columns is ever held.
    const int64_t gr_max = std::min(rows, kGradRows);
    char* w = (char*)ws;
    float* row_scale = (float*)w; w += align256(rows * 4);
    float* lse = lse_out ? lse_out : (float*)w; w += align256(rows * 4);
    float* target = (float*)w; w += align256(rows * 4);
    float* run_max = (float*)w; w += align256(rows * 4);
    float* run_sum = (float*)w; w += align256(rows * 4);
    float* alpha = (float*)w; w += align256(rows * 4);
    int64_t* run_arg = (predicted || correct) ? (int64_t*)w : nullptr; w += align256(rows * 8);  // running argmax column per row
    bf16_t* slab = (bf16_t*)w; w += align256(gr_max * kVocabBlock * 2);
    float* dh32 = (float*)w; w += align256(gr_max * hidden_dim * 4);
    uint8_t* label_rows = (uint8_t*)w; w += align256(gr_max * hidden_dim * 2);  // packed rows are smaller than bf16 rows
    bf16_t* w_label = (bf16_t*)w;

    hipLaunchKernelGGL(ce_row_scale_kernel, dim3(1), dim3(1024), 0, s, labels, rows, vocab, ignore_index, reduction_mean, row_scale, n_valid_out);
    const int64_t row_bytes = packed_row_bytes(qt, hidden_dim);
    if (row_bytes <= 0 || row_bytes > hidden_dim * 2 || (row_bytes & 1)) return set_error(GGQ_ERR_QTYPE, "lmhead_ce: unsupported packed row size");
    hipLaunchKernelGGL(fill_f32_kernel, dim3(grid1d(rows)), dim3(256), 0, s, run_max, rows, -INFINITY);
    hipLaunchKernelGGL(fill_f32_kernel, dim3(grid1d(rows)), dim3(256), 0, s, run_sum, rows, 0.f);
    hipLaunchKernelGGL(fill_f32_kernel, dim3(grid1d(rows)), dim3(256), 0, s, target, rows, 0.f);
    for (int64_t r0 = 0; r0 < rows; r0 += gr_max) {
        const int rc = (int)std::min(rows - r0, gr_max);
        const bf16_t* hid = (const bf16_t*)hidden + r0 * hidden_dim;
        hipLaunchKernelGGL(fill_f32_kernel, dim3(grid1d((int64_t)rc * hidden_dim)), dim3(256), 0, s, dh32, (int64_t)rc * hidden_dim, 0.f);
        for (int64_t v0 = 0; v0 < vocab; v0 += kVocabBlock) {
            const int nb = (int)((vocab - v0) < kVocabBlock ? (vocab - v0) : kVocabBlock);
            // (1) the block's logits
            MmqParams g;
            if (int rcode = init_params(g, qt, kModeNT, rc, nb, (int)hidden_dim, 1)) return rcode;
            g.a[0] = hid, g.lda = hidden_dim;
            g.w[0] = (const uint8_t*)packed + v0 * row_bytes;
            g.c[0] = slab, g.ldc = kVocabBlock;
            if (int rcode = launch_mmq(qt, kModeNT, kEpiStore, g, s)) return rcode;
            // (2) running statistics; the slab becomes exp(logit - running max)
            hipLaunchKernelGGL(ce_stream_block_kernel, dim3((unsigned)rc), dim3(256), 0, s, slab, kVocabBlock, nb, v0, labels + r0, run_max + r0, run_sum + r0,
                               target + r0, alpha + r0, run_arg ? run_arg + r0 : nullptr);
            // (3) acc = acc * alpha + p . W_block
            MmqParams b;
            if (int rcode = init_params(b, qt, kModeNN, rc, nb, (int)hidden_dim, 1)) return rcode;
            b.a[0] = slab, b.lda = kVocabBlock, b.a_zero_padded = 1;
            b.w[0] = (const uint8_t*)packed + v0 * row_bytes;
            b.c[0] = dh32, b.ldc = hidden_dim;
            b.row_scale = alpha + r0;
            if (int rcode = launch_mmq(qt, kModeNN, kEpiAccumF32, b, s)) return rcode;
        }
        hipLaunchKernelGGL(gather_label_rows_kernel, dim3((unsigned)rc), dim3(256), 0, s, (const uint8_t*)packed, row_bytes, labels + r0, vocab, label_rows);
        if (int rcode = dequantize(qt, label_rows, rc, hidden_dim, w_label, 0, s)) return rcode;
        hipLaunchKernelGGL(ce_stream_finish_kernel, dim3((unsigned)rc), dim3(256), 0, s, dh32, w_label, hidden_dim, labels + r0, vocab, run_max + r0, run_sum + r0,
                           target + r0, row_scale + r0, lse + r0, loss_1d + r0, (bf16_t*)grad_hidden + r0 * hidden_dim, ignore_index,
                           run_arg ? run_arg + r0 : nullptr, predicted ? predicted + r0 : nullptr, correct ? correct + r0 : nullptr);
    }
    return check_launch("lmhead_ce");
}

}  // namespace ggq
