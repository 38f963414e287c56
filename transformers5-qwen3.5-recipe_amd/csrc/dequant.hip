// Standalone GGUF block decoders: packed payload -> bf16 or fp32, bit-exact with ggml's
// dequantize_row_* (including the sign of zero).  HBM-bound: every workgroup copies a 16-byte aligned
// run of whole blocks into LDS with coalesced 128-bit loads, then each lane unpacks runs of eight
// consecutive elements from LDS and writes them with one (bf16) or two (fp32) 128-bit stores.
#include "blocks.h"
#include "iq2xxs_grid.h"
#include "launch.h"

namespace ggq {

static __device__ const uint64_t d_iq2xxs_grid[256] = GGQ_IQ2XXS_GRID_INIT;

constexpr int kElemsPerWg = 8192;

__device__ __forceinline__ uint32_t lds_u16(const uint8_t* p) { return *(const uint16_t*)p; }

template <int QT>
__device__ __forceinline__ void decode8(const uint8_t* raw, int g, float* y) {
    if constexpr (QT == kQ8_0) {
        const uint8_t* blk = raw + (g >> 2) * 34;
        const float d = half_bits_to_f32(lds_u16(blk));
        const uint8_t* q = blk + 2 + 8 * (g & 3);
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = d * (float)(int8_t)q[i];
    } else if constexpr (QT == kQ4_K) {
        const uint8_t* blk = raw + (g >> 5) * 144;
        const int e0 = 8 * (g & 31), j = e0 >> 5, l0 = e0 & 31;
        const float d = half_bits_to_f32(lds_u16(blk)), dmin = half_bits_to_f32(lds_u16(blk + 2));
        const uint8_t* s = blk + 4;
        uint32_t sc, m;
        if (j < 4) {
            sc = s[j] & 63u;
            m = s[j + 4] & 63u;
        } else {
            sc = (s[j + 4] & 0xFu) | ((uint32_t)(s[j - 4] >> 6) << 4);
            m = (uint32_t)(s[j + 4] >> 4) | ((uint32_t)(s[j] >> 6) << 4);
        }
        const float dl = d * (float)sc, ml = dmin * (float)m;
        const uint8_t* q = blk + 16 + 32 * (j >> 1) + l0;
        const int shift = 4 * (j & 1);
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = __fsub_rn(__fmul_rn(dl, (float)((q[i] >> shift) & 0xFu)), ml);
    } else if constexpr (QT == kQ5_K) {
        const uint8_t* blk = raw + (g >> 5) * 176;
        const int e0 = 8 * (g & 31), j = e0 >> 5, l0 = e0 & 31;
        const float d = half_bits_to_f32(lds_u16(blk)), dmin = half_bits_to_f32(lds_u16(blk + 2));
        const uint8_t* s = blk + 4;
        uint32_t sc, m;
        if (j < 4) {
            sc = s[j] & 63u;
            m = s[j + 4] & 63u;
        } else {
            sc = (s[j + 4] & 0xFu) | ((uint32_t)(s[j - 4] >> 6) << 4);
            m = (uint32_t)(s[j + 4] >> 4) | ((uint32_t)(s[j] >> 6) << 4);
        }
        const float dl = d * (float)sc, ml = dmin * (float)m;
        const uint8_t* qh = blk + 16 + l0;
        const uint8_t* q = blk + 48 + 32 * (j >> 1) + l0;
        const int shift = 4 * (j & 1);
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = __fsub_rn(__fmul_rn(dl, (float)(((q[i] >> shift) & 0xFu) + (((qh[i] >> j) & 1u) << 4))), ml);
    } else if constexpr (QT == kQ2_K) {
        const uint8_t* blk = raw + (g >> 5) * 84;
        const int e0 = 8 * (g & 31), n = e0 >> 7, j = (e0 & 127) >> 5, l0 = e0 & 31;
        const float d = half_bits_to_f32(lds_u16(blk + 80)), dmin = half_bits_to_f32(lds_u16(blk + 82));
        const uint32_t sb = blk[e0 >> 4];
        const float dl = d * (float)(sb & 0xFu), ml = dmin * (float)(sb >> 4);
        const uint8_t* q = blk + 16 + 32 * n + l0;
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = __fsub_rn(__fmul_rn(dl, (float)((q[i] >> (2 * j)) & 3u)), ml);
    } else if constexpr (QT == kQ3_K) {
        const uint8_t* blk = raw + (g >> 5) * 110;
        const int e0 = 8 * (g & 31), n = e0 >> 7, u = e0 >> 5, l0 = e0 & 31, k = e0 >> 4, kg = k >> 2, kb = k & 3;
        const float d = half_bits_to_f32(lds_u16(blk + 108));
        const int sc = (int)(((blk[96 + 4 * (kg & 1) + kb] >> (4 * (kg >> 1))) & 0xFu) | (((blk[104 + kb] >> (2 * kg)) & 3u) << 4)) - 32;
        const float dl = d * (float)sc;
        const uint8_t* q = blk + 32 + 32 * n + l0;
        const uint8_t* hm = blk + l0;
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = dl * (float)((int)((q[i] >> (2 * (u & 3))) & 3u) - (((hm[i] >> u) & 1u) ? 0 : 4));
    } else if constexpr (QT == kQ6_K) {
        const uint8_t* blk = raw + (g >> 5) * 210;
        const int e0 = 8 * (g & 31), h = e0 >> 7, part = (e0 & 127) >> 5, l0 = e0 & 31;
        const float d = half_bits_to_f32(lds_u16(blk + 208));
        const float dl = d * (float)(int8_t)blk[192 + (e0 >> 4)];
        const uint8_t* ql = blk + 64 * h + 32 * (part & 1) + l0;
        const uint8_t* qh = blk + 128 + 32 * h + l0;
        const int nshift = 4 * (part >> 1), hshift = 2 * part;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            int q = (int)(((ql[i] >> nshift) & 0xFu) | (((qh[i] >> hshift) & 3u) << 4)) - 32;
            y[i] = dl * (float)q;
        }
    } else {  // IQ2_XXS
        const uint8_t* blk = raw + (g >> 5) * 66;
        const int grp = (g & 31) >> 2, l = g & 3;
        const float d = half_bits_to_f32(lds_u16(blk));
        const uint8_t* a = blk + 2 + 8 * grp;
        const uint32_t aux = lds_u16(a + 4) | (lds_u16(a + 6) << 16);
        const float db = d * (0.5f + (float)(aux >> 28)) * 0.25f;
        const uint64_t gr = d_iq2xxs_grid[a[l]];
        const uint32_t s7 = (aux >> (7 * l)) & 127u;
        const uint32_t signs = s7 | ((__builtin_popcount(s7) & 1u) << 7);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float mag = (float)(uint32_t)((gr >> (8 * i)) & 0xFFu);
            y[i] = db * mag * (((signs >> i) & 1u) ? -1.0f : 1.0f);
        }
    }
}

template <int QT, bool OUT_F32>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ payload, int64_t total_elems,
                                                       void* __restrict__ out) {
    constexpr int kBE = Fmt<QT>::kBlockElems, kBB = Fmt<QT>::kBlockBytes;
    constexpr int kBlocksPerWg = kElemsPerWg / kBE;
    constexpr int kRawBytes = kBlocksPerWg * kBB;  // a multiple of 16 for every format
    __shared__ __attribute__((aligned(16))) uint8_t raw[kRawBytes];
    const int64_t e_begin = (int64_t)blockIdx.x * kElemsPerWg;
    const int64_t e_left = total_elems - e_begin;
    const int n_elems = e_left < kElemsPerWg ? (int)e_left : kElemsPerWg;
    const int n_bytes = n_elems / kBE * kBB;
    const uint8_t* src = payload + (int64_t)blockIdx.x * kRawBytes;
    for (int o = threadIdx.x * 16; o + 16 <= n_bytes; o += 256 * 16) *(uint4*)(raw + o) = *(const uint4*)(src + o);
    for (int o = (n_bytes & ~15) + threadIdx.x * 2; o < n_bytes; o += 512) *(uint16_t*)(raw + o) = *(const uint16_t*)(src + o);
    __syncthreads();
    for (int g = threadIdx.x; g * 8 < n_elems; g += 256) {
        float y[8];
        decode8<QT>(raw, g, y);
        const int64_t e = e_begin + (int64_t)g * 8;
        if constexpr (OUT_F32) {
            float4* dst = (float4*)((float*)out + e);
            dst[0] = make_float4(y[0], y[1], y[2], y[3]);
            dst[1] = make_float4(y[4], y[5], y[6], y[7]);
        } else {
            uint4 v;
            v.x = pack_bf16(y[0], y[1]), v.y = pack_bf16(y[2], y[3]);
            v.z = pack_bf16(y[4], y[5]), v.w = pack_bf16(y[6], y[7]);
            *(uint4*)((bf16_t*)out + e) = v;
        }
    }
}

template <int QT>
static int launch_dequant(const void* payload, int64_t total, void* out, int out_f32, hipStream_t stream) {
    if (total == 0) return 0;
    const int64_t wgs = (total + kElemsPerWg - 1) / kElemsPerWg;
    if (wgs > 0x7FFFFFFF) return set_error(GGQ_ERR_SHAPE, "dequantize: payload too large for one launch");
    if (out_f32)
        hipLaunchKernelGGL((dequant_kernel<QT, true>), dim3((unsigned)wgs), dim3(256), 0, stream, (const uint8_t*)payload, total, out);
    else
        hipLaunchKernelGGL((dequant_kernel<QT, false>), dim3((unsigned)wgs), dim3(256), 0, stream, (const uint8_t*)payload, total, out);
    return check_launch("dequantize");
}

int dequantize(int qt, const void* payload, int64_t rows, int64_t k, void* out, int out_f32, hipStream_t stream) {
    if (rows < 0 || k < 0) return set_error(GGQ_ERR_SHAPE, "dequantize: negative shape");
    if (!block_multiple(qt, k)) return set_error(GGQ_ERR_SHAPE, "dequantize: K is not a multiple of the block size");
    if (((uintptr_t)payload | (uintptr_t)out) & 15) return set_error(GGQ_ERR_ALIGN, "dequantize: pointers must be 16-byte aligned");
    const int64_t total = rows * k;
    switch (qt) {
        case kQ8_0: return launch_dequant<kQ8_0>(payload, total, out, out_f32, stream);
        case kQ2_K: return launch_dequant<kQ2_K>(payload, total, out, out_f32, stream);
        case kQ3_K: return launch_dequant<kQ3_K>(payload, total, out, out_f32, stream);
        case kQ4_K: return launch_dequant<kQ4_K>(payload, total, out, out_f32, stream);
        case kQ5_K: return launch_dequant<kQ5_K>(payload, total, out, out_f32, stream);
        case kQ6_K: return launch_dequant<kQ6_K>(payload, total, out, out_f32, stream);
        case kIQ2_XXS: return launch_dequant<kIQ2_XXS>(payload, total, out, out_f32, stream);
    }
    return set_error(GGQ_ERR_QTYPE, "dequantize: unsupported GGML type id");
}

}  // namespace ggq
