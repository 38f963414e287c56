// Shared device helpers for the gfx950 quantized-weight matmul kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ggq {

// GGML type ids of the supported block formats.
enum : int { kQ8_0 = 8, kQ2_K = 10, kQ3_K = 11, kQ4_K = 12, kQ5_K = 13, kQ6_K = 14, kIQ2_XXS = 16 };

// Decoder helpers are host+device so the bit unpacking can also be exercised in a CPU build.
#define GGQ_HD __host__ __device__ __forceinline__

typedef uint16_t bf16_t;  // raw bf16 bits
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

// Two floats -> packed bf16 pair (lo in bits 0..15), round to nearest even (v_cvt_pk_bf16_f32).
GGQ_HD uint32_t pack_bf16(float lo, float hi) {
    f32x2_t v = {lo, hi};
    bf16x2_t r = __builtin_convertvector(v, bf16x2_t);
    return __builtin_bit_cast(uint32_t, r);
}
GGQ_HD bf16_t to_bf16(float x) { return (bf16_t)(pack_bf16(x, 0.0f) & 0xFFFFu); }
GGQ_HD float bf16_to_f32(bf16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }
GGQ_HD float bf16_lo(uint32_t p) { return __builtin_bit_cast(float, p << 16); }
GGQ_HD float bf16_hi(uint32_t p) { return __builtin_bit_cast(float, p & 0xFFFF0000u); }

GGQ_HD float half_bits_to_f32(uint32_t h16) {
    _Float16 h = __builtin_bit_cast(_Float16, (uint16_t)h16);
    return (float)h;
}

// Hides the value's known bits from the optimizer so that a following
// (float)((x >> 8*i) & 0xff) stays a single v_cvt_f32_ubyte<i> instead of bfe + cvt.
GGQ_HD uint32_t opaque(uint32_t x) {
#if defined(__HIP_DEVICE_COMPILE__)
    asm("" : "+v"(x));
#endif
    return x;
}
GGQ_HD float ubyte0(uint32_t x) { return (float)(x & 0xFFu); }
GGQ_HD float ubyte1(uint32_t x) { return (float)((x >> 8) & 0xFFu); }
GGQ_HD float ubyte2(uint32_t x) { return (float)((x >> 16) & 0xFFu); }
GGQ_HD float ubyte3(uint32_t x) { return (float)(x >> 24); }

// Small unsigned integers sitting in the 16-bit halves of a register are read as half-precision
// denormals (value = integer * 2^-24, exact), so one mixed-precision fma (v_fma_mix_f32) computes
// fma(scale, integer, offset) without a separate integer->float conversion: pass scale * 2^24
// (kMixScale), the product is the same real number and the single rounding is the same.
constexpr float kMixScale = 16777216.0f;
GGQ_HD float mix_lo(uint32_t r, float scale24, float offset) {
    return __builtin_fmaf((float)__builtin_bit_cast(_Float16, (uint16_t)(r & 0xFFFFu)), scale24, offset);
}
GGQ_HD float mix_hi(uint32_t r, float scale24, float offset) {
    return __builtin_fmaf((float)__builtin_bit_cast(_Float16, (uint16_t)(r >> 16)), scale24, offset);
}

// Unaligned (2-byte aligned) global loads: the target allows unaligned vector memory access, so
// these stay single global_load instructions.
GGQ_HD uint32_t ld_u32(const uint8_t* p) {
    uint32_t v;
    __builtin_memcpy(&v, p, 4);
    return v;
}
GGQ_HD uint4 ld_u128(const uint8_t* p) {
    uint4 v;
    __builtin_memcpy(&v, p, 16);
    return v;
}
GGQ_HD uint32_t ld_u16(const uint8_t* p) {
    uint16_t v;
    __builtin_memcpy(&v, p, 2);
    return v;
}

#if defined(__HIP_DEVICE_COMPILE__) || defined(__HIPCC__)
// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains every outstanding
// global load (s_waitcnt vmcnt(0)), which would serialise the prefetches behind each step.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Wait until at most n of this wave's global loads are outstanding (loads return in issue order).
__device__ __forceinline__ void wait_loads_at_most(int n) {
    switch (n) {
        case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
        case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
        case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
        case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
        case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
        case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
        case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
        case 7: asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); break;
        default: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
    }
}

// 16-byte slot that holds contraction chunk kc (0..7) of A-tile row r.  Sixteen consecutive rows at one
// kc cover all sixteen 16-byte bank groups exactly once.
__device__ __forceinline__ int a_slot(int r, int kc) { return kc ^ ((r >> 1) & 7); }

// One direct global -> LDS load: every lane moves the 16 bytes at sbase + voff to LDS address
// lds + 16 * lane (lds is wave-uniform).  The data never passes through registers; the instruction
// counts as one outstanding vector-memory load of the wave.
__device__ __forceinline__ void load16_to_lds(uint32_t lds, uint32_t voff, const void* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds), "v"(voff), "s"(sbase) : "memory");
}
#endif

}  // namespace ggq
