// Chunked cross-entropy through a packed lm_head without ever holding [rows, vocab] logits.
//
// Per block of up to kBlockRows rows: (1) per chunk of rows, the packed-weight tile kernel runs over the whole vocabulary
// with an epilogue that stores the bf16 logits, reduces every 128-column slab of a logits tile to (max, sum exp) per row
// and records the target logit; a small kernel merges the slabs into log-sum-exp and the per-row loss; (2) one
// element-wise kernel turns the block's logits into d(loss)/d(logits) in place; (3) one grad-input launch of the tile
// kernel contracts them with the same packed rows over the whole vocabulary.  Two vocabulary-sized matmuls, as in the
// reference, whose [chunk, vocab] logits tensor this buffer corresponds to.
#include <algorithm>

#include "common.h"
#include "launch.h"
#include "mmq_host.h"

namespace ggq {

// The logits of up to this many rows are kept (bf16, rows padded with zeros to a multiple of 64 columns) between the
// statistics pass and the gradient pass: 4096 rows fill the chip with tiles of the [rows, hidden] grad-input output (a
// 1024-row chunk makes 64 tiles for 256 compute units), at 2 bytes per row and vocabulary entry (1.2 GB for a 152k
// vocabulary).  The caller's chunk bounds the rows of one statistics launch.
constexpr int64_t kBlockRows = 4096;

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

// logits -> d(loss)/d(logits) in place: (exp(logit - lse) - [column == label]) * row_scale, bf16; the padding columns
// [vocab, ld) of every row become zero.  One workgroup per row, eight columns per lane and trip (ld is a multiple of 64).
__global__ __launch_bounds__(256) void ce_grad_kernel(bf16_t* logits, int64_t ld, int64_t vocab, const float* lse, const float* row_scale,
                                                      const int64_t* labels) {
    const int64_t row = blockIdx.x;
    const float l = lse[row], rs = row_scale[row];
    const int64_t label = labels[row];
    uint4* p = (uint4*)(logits + row * ld);
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
                float d = __expf(logit - l);
                if (col == label) d -= 1.0f;
                g[h] = col < vocab ? d * rs : 0.0f;
            }
            o[e] = pack_bf16(g[0], g[1]);
        }
        p[c8] = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

static int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

static int64_t padded_vocab(int64_t vocab) { return (vocab + 63) / 64 * 64; }

int64_t lmhead_ce_workspace_bytes(int64_t rows, int64_t vocab, int64_t hidden, int64_t chunk) {
    (void)hidden;
    const int64_t rc = chunk < rows ? chunk : rows;
    const int64_t br = std::min(rows, kBlockRows);
    const int64_t nparts = (vocab + kBN - 1) / kBN * 2;
    return align256(rows * 4) * 3 + align256(rc * nparts * 8) + align256(br * padded_vocab(vocab) * 2) + 1024;
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
    const int64_t br_max = std::min(rows, kBlockRows);
    const int64_t ld = padded_vocab(vocab);
    const int nparts = (int)((vocab + kBN - 1) / kBN) * 2;
    char* w = (char*)ws;
    float* row_scale = (float*)w; w += align256(rows * 4);
    float* lse = lse_out ? lse_out : (float*)w; w += align256(rows * 4);
    float* target = (float*)w; w += align256(rows * 4);
    float2* partials = (float2*)w; w += align256(rc_max * nparts * 8);
    bf16_t* logits = (bf16_t*)w;  // [br_max, ld]

    hipLaunchKernelGGL(ce_row_scale_kernel, dim3(1), dim3(1024), 0, s, labels, rows, ignore_index, reduction_mean, row_scale, n_valid_out);
    for (int64_t b0 = 0; b0 < rows; b0 += br_max) {
        const int64_t br = std::min(rows - b0, br_max);
        // (1) statistics and logits, chunk by chunk
        for (int64_t r0 = b0; r0 < b0 + br; r0 += chunk) {
            const int rc = (int)std::min(b0 + br - r0, chunk);
            MmqParams p;
            if (int rcode = init_params(p, qt, kModeNT, rc, (int)vocab, (int)hidden_dim, 1)) return rcode;
            p.a[0] = (const bf16_t*)hidden + r0 * hidden_dim, p.lda = hidden_dim;
            p.w[0] = (const uint8_t*)packed;
            p.c[0] = logits + (r0 - b0) * ld, p.ldc = ld;
            p.labels = labels + r0, p.ce_partials = partials, p.ce_partials_ld = nparts, p.ce_target_logit = target + r0;
            p.ignore_index = ignore_index;
            if (int rcode = launch_mmq(qt, kModeNT, kEpiCeStats, p, s)) return rcode;
            hipLaunchKernelGGL(ce_finalize_kernel, dim3((rc + 3) / 4), dim3(256), 0, s, partials, nparts, nparts, target + r0, row_scale + r0, rc, lse + r0, loss_1d + r0);
        }
        // (2) the block's logits become the gradient with respect to them, in place
        hipLaunchKernelGGL(ce_grad_kernel, dim3((unsigned)br), dim3(256), 0, s, logits, ld, vocab, lse + b0, row_scale + b0, labels + b0);
        // (3) dH = dlogits . W over the whole vocabulary
        MmqParams g;
        if (int rcode = init_params(g, qt, kModeNN, (int)br, (int)vocab, (int)hidden_dim, 1)) return rcode;
        g.a[0] = logits, g.lda = ld, g.a_zero_padded = 1;
        g.w[0] = (const uint8_t*)packed;
        g.c[0] = (bf16_t*)grad_hidden + b0 * hidden_dim, g.ldc = hidden_dim;
        if (int rcode = launch_mmq(qt, kModeNN, kEpiStore, g, s)) return rcode;
    }
    return check_launch("lmhead_ce");
}

}  // namespace ggq
