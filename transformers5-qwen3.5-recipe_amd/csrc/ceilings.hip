// Measurement aid: what the MFMA pipes of this device sustain with operands of given statistics.  The chip is power
// limited and its matrix clock depends on the data (all-zero operands run faster than noise-like ones), so a kernel's
// MFMA-bound ceiling on a workload is this figure measured with that workload's values, not the nominal peak.
#include "common.h"
#include "launch.h"
#include "mmq_host.h"

namespace ggq {

// Register-only loop of 32x32x16 bf16 MFMAs over eight independent accumulators; two waves per SIMD.  Every lane takes its
// operands once from the sample buffers (eight values each), so the multipliers see the samples' statistics.
__global__ __launch_bounds__(512) void mfma_ceiling_kernel(const bf16_t* a_samples, const bf16_t* b_samples, int64_t elems, int iters, float* sink) {
    const int64_t slot = ((int64_t)blockIdx.x * 512 + threadIdx.x) * 8 % (elems - 8);
    const bf16x8_t a = *(const bf16x8_t*)(a_samples + (slot & ~7ll));
    const bf16x8_t b = *(const bf16x8_t*)(b_samples + (slot & ~7ll));
    f32x16_t c[8];
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) c[j][e] = 0.0f;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int j = 0; j < 8; j++) c[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c[j], 0, 0, 0);
    }
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) s += c[j][j];
    if (s == 1.2345e-30f) sink[0] = s;  // keeps the loop alive without a store in practice
}

int measure_mfma_ceiling(const void* a_samples, const void* b_samples, int64_t elems, int iters, void* sink_buffer, float* tflops_out, hipStream_t s) {
    if (!a_samples || !b_samples || !tflops_out || !sink_buffer) return set_error(GGQ_ERR_NULL, "measure_mfma_ceiling: null pointer");
    if (elems < 4096 || iters < 1 || (((uintptr_t)a_samples | (uintptr_t)b_samples) & 15)) return set_error(GGQ_ERR_SHAPE, "measure_mfma_ceiling: needs at least 4096 aligned samples and iters >= 1");
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0)
        return set_error(GGQ_ERR_RUNTIME, "measure_mfma_ceiling: cannot query the device");
    float* sink = (float*)sink_buffer;  // the caller's: nothing is allocated here
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return set_error(GGQ_ERR_RUNTIME, "measure_mfma_ceiling: event creation failed");
    hipLaunchKernelGGL(mfma_ceiling_kernel, dim3(cus), dim3(512), 0, s, (const bf16_t*)a_samples, (const bf16_t*)b_samples, elems, 64, sink);  // warm-up
    (void)hipEventRecord(e0, s);
    hipLaunchKernelGGL(mfma_ceiling_kernel, dim3(cus), dim3(512), 0, s, (const bf16_t*)a_samples, (const bf16_t*)b_samples, elems, iters, sink);
    (void)hipEventRecord(e1, s);
    float ms = 0.0f;
    const bool ok = hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&ms, e0, e1) == hipSuccess && ms > 0.0f;
    (void)hipEventDestroy(e0), (void)hipEventDestroy(e1);
    if (!ok) return set_error(GGQ_ERR_RUNTIME, "measure_mfma_ceiling: timing failed");
    *tflops_out = (float)((double)cus * 8 /* waves */ * iters * 8 * 32768.0 / (ms * 1e-3) / 1e12);
    return check_launch("mfma_ceiling_kernel");
}

}  // namespace ggq
