// Chunked cross-entropy through a packed lm_head without ever holding [rows, vocab] logits.
//
// Pass 1, per row chunk: the packed-weight tile kernel runs over the whole vocabulary with an epilogue
// that reduces every 128-column slab of a logits tile to (max, sum exp) per row and records the target
// logit; a small kernel merges the slabs into log-sum-exp and the per-row loss.  Pass 2, per block of up to
// kGradRows rows, walks the vocabulary in blocks of kVocabBlock columns: the tile kernel recomputes that
// block's logits and its epilogue turns them into d(loss)/d(logits) (bf16, [rows of the block, kVocabBlock]
// only); the grad-input form of the tile kernel contracts the block with the same packed rows into an fp32
// accumulator.  Three vocabulary-sized matmuls instead of two is the price of not materialising the logits.
#include <algorithm>

#include "common.h"
#include "launch.h"
#include "mmq_host.h"

namespace ggq {

constexpr int kVocabBlock = 8192;
// The gradient pass takes up to this many rows at a time, whatever the caller's chunk (which bounds the statistics pass
// and stands for the reference's [chunk, vocab] logits): 4096 rows fill the chip with tiles of the [rows, hidden]
// grad-input output (a 1024-row chunk makes 64 tiles for 256 compute units) and cost a 64 MiB gradient slab.
constexpr int64_t kGradRows = 4096;

// row_scale[m] = 0 for ignored rows, else 1/n_valid (mean) or 1 (sum); n_valid = 0 gives all zeros.
__global__ __launch_bounds__(1024) void ce_row_scale_kernel(const int64_t* labels, int64_t rows, int64_t ignore_index,
                                                             int mean, float* row_scale, int* n_valid_out) {
    __shared__ int partial[1024];
    int c = 0;
    for (int64_t i = threadIdx.x; i < rows; i += 1024) c += labels[i] != ignore_index;
    partial[threadIdx.x] = c;
    __syncthreads();
    for (int off = 512; off >= 1; off >>= 1) {
        if ((int)threadIdx.x < off) partial[threadIdx.x] += partial[threadIdx.x + off];
        __syncthreads();
    }
    const int n = partial[0];
    const float scale = n == 0 ? 0.f : (mean ? 1.0f / (float)n : 1.0f);
    for (int64_t i = threadIdx.x; i < rows; i += 1024) row_scale[i] = labels[i] != ignore_index ? scale : 0.f;
    if (threadIdx.x == 0 && n_valid_out) *n_valid_out = n;
}

// One wave per row: merge the slab partials into lse, then loss = (lse - target logit) * row_scale.
__global__ __launch_bounds__(256) void ce_finalize_kernel(const float2* partials, int ld, int nparts, const float* target_logit,
                                                          const float* row_scale, int rows, float* lse_out, float* loss_out) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const float2* p = partials + (int64_t)r * ld;
    float mx = -INFINITY;
    for (int i = lane; i < nparts; i += 64) mx = fmaxf(mx, p[i].x);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    float sum = 0.f;
    for (int i = lane; i < nparts; i += 64) {
        const float2 v = p[i];
        if (v.y > 0.f) sum += v.y * __expf(v.x - mx);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (lane == 0) {
        const float lse = mx + __logf(sum);
        lse_out[r] = lse;
        const float rs = row_scale[r];
        loss_out[r] = rs != 0.f ? (lse - target_logit[r]) * rs : 0.f;
    }
}

__global__ void fill_f32_kernel(float* p, int64_t n, float v) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = v;
}

__global__ void f32_to_bf16_kernel(const float* src, bf16_t* dst, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) dst[i] = to_bf16(src[i]);
}

static unsigned grid1d(int64_t n) {
    int64_t g = (n + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 16384 ? 16384 : g));
}

static int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

int64_t lmhead_ce_workspace_bytes(int64_t rows, int64_t vocab, int64_t hidden, int64_t chunk) {
    const int64_t rc = chunk < rows ? chunk : rows;
    const int64_t gr = std::min(rows, std::max(chunk, kGradRows));
    const int64_t nparts = (vocab + kBN - 1) / kBN * 2;
    return align256(rows * 4) * 3 + align256(rc * nparts * 8) + align256(gr * kVocabBlock * 2) + align256(gr * hidden * 4) + 1024;
}

int lmhead_ce(int qt, const void* hidden, const void* packed, const int64_t* labels, int64_t rows, int64_t vocab,
              int64_t hidden_dim, int64_t chunk, int64_t ignore_index, int reduction_mean, float* loss_1d,
              void* grad_hidden, float* lse_out, int* n_valid_out, void* ws, int64_t ws_bytes, hipStream_t s) {
    if (rows < 0 || vocab <= 0 || hidden_dim <= 0 || chunk <= 0) return set_error(GGQ_ERR_SHAPE, "lmhead_ce: bad shape");
    if (rows >= (1 << 30) || vocab >= (1 << 30)) return set_error(GGQ_ERR_SHAPE, "lmhead_ce: shape too large");
    if (!hidden || !packed || !labels || !loss_1d || !grad_hidden || !ws) return set_error(GGQ_ERR_NULL, "lmhead_ce: null pointer");
    if (ws_bytes < lmhead_ce_workspace_bytes(rows, vocab, hidden_dim, chunk)) return set_error(GGQ_ERR_WORKSPACE, "lmhead_ce: workspace too small");
    if (((uintptr_t)hidden | (uintptr_t)packed | (uintptr_t)grad_hidden | (uintptr_t)ws) & 15) return set_error(GGQ_ERR_ALIGN, "lmhead_ce: pointers must be 16-byte aligned");
    if (rows == 0) return GGQ_OK;
    const int64_t rc_max = chunk < rows ? chunk : rows;
    const int64_t gr_max = std::min(rows, std::max(chunk, kGradRows));
    const int nparts = (int)((vocab + kBN - 1) / kBN) * 2;
    char* w = (char*)ws;
    float* row_scale = (float*)w; w += align256(rows * 4);
    float* lse = lse_out ? lse_out : (float*)w; w += align256(rows * 4);
    float* target = (float*)w; w += align256(rows * 4);
    float2* partials = (float2*)w; w += align256(rc_max * nparts * 8);
    bf16_t* dlogits = (bf16_t*)w; w += align256(gr_max * kVocabBlock * 2);
    float* dh32 = (float*)w;

    hipLaunchKernelGGL(ce_row_scale_kernel, dim3(1), dim3(1024), 0, s, labels, rows, ignore_index, reduction_mean, row_scale, n_valid_out);
    const int64_t row_bytes = packed_row_bytes(qt, hidden_dim);
    for (int64_t r0 = 0; r0 < rows; r0 += chunk) {
        const int rc = (int)((rows - r0) < chunk ? (rows - r0) : chunk);
        const bf16_t* hid = (const bf16_t*)hidden + r0 * hidden_dim;
        MmqParams p;
        if (int rcode = init_params(p, qt, kModeNT, rc, (int)vocab, (int)hidden_dim, 1)) return rcode;
        p.a[0] = hid, p.lda = hidden_dim;
        p.w[0] = (const uint8_t*)packed;
        p.labels = labels + r0, p.ce_partials = partials, p.ce_partials_ld = nparts, p.ce_target_logit = target + r0;
        p.ignore_index = ignore_index;
        if (int rcode = launch_mmq(qt, kModeNT, kEpiCeStats, p, s)) return rcode;
        hipLaunchKernelGGL(ce_finalize_kernel, dim3((rc + 3) / 4), dim3(256), 0, s, partials, nparts, nparts, target + r0, row_scale + r0, rc, lse + r0, loss_1d + r0);
    }
    // gradient pass: the log-sum-exp of every row is known; row blocks of up to gr_max rows
    for (int64_t r0 = 0; r0 < rows; r0 += gr_max) {
        const int rc = (int)std::min(rows - r0, gr_max);
        const bf16_t* hid = (const bf16_t*)hidden + r0 * hidden_dim;
        hipLaunchKernelGGL(fill_f32_kernel, dim3(grid1d((int64_t)rc * hidden_dim)), dim3(256), 0, s, dh32, (int64_t)rc * hidden_dim, 0.f);
        for (int64_t v0 = 0; v0 < vocab; v0 += kVocabBlock) {
            const int nb = (int)((vocab - v0) < kVocabBlock ? (vocab - v0) : kVocabBlock);
            MmqParams g;
            if (int rcode = init_params(g, qt, kModeNT, rc, nb, (int)hidden_dim, 1)) return rcode;
            g.a[0] = hid, g.lda = hidden_dim;
            g.w[0] = (const uint8_t*)packed + v0 * row_bytes;
            g.c[0] = dlogits, g.ldc = kVocabBlock;
            g.labels = labels + r0, g.lse = lse + r0, g.row_scale = row_scale + r0, g.ce_col_offset = (int)v0;
            if (int rcode = launch_mmq(qt, kModeNT, kEpiCeGrad, g, s)) return rcode;
            MmqParams b;
            if (int rcode = init_params(b, qt, kModeNN, rc, nb, (int)hidden_dim, 1)) return rcode;
            b.a[0] = dlogits, b.lda = kVocabBlock;
            b.w[0] = (const uint8_t*)packed + v0 * row_bytes;
            b.c[0] = dh32, b.ldc = hidden_dim;
            if (int rcode = launch_mmq(qt, kModeNN, kEpiAccumF32, b, s)) return rcode;
        }
        hipLaunchKernelGGL(f32_to_bf16_kernel, dim3(grid1d((int64_t)rc * hidden_dim)), dim3(256), 0, s, dh32, (bf16_t*)grad_hidden + r0 * hidden_dim, (int64_t)rc * hidden_dim);
    }
    return check_launch("lmhead_ce");
}

}  // namespace ggq
