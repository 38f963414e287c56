// Host-side plumbing shared by the C-ABI entry points: error codes, last-error text, launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace ggq {

enum : int {
    GGQ_OK = 0,
    GGQ_ERR_QTYPE = -1,    // unsupported GGML type id
    GGQ_ERR_SHAPE = -2,    // negative / inconsistent / unsupported shape
    GGQ_ERR_ALIGN = -3,    // pointer or leading dimension not aligned as required
    GGQ_ERR_NULL = -4,     // required pointer is null
    GGQ_ERR_RUNTIME = -5,  // HIP runtime reported an error
    GGQ_ERR_WORKSPACE = -6 // workspace too small
};

int set_error(int code, const char* fmt, ...);
int check_launch(const char* what);

// A kernel that needs more than 64 KB of dynamic LDS has that limit raised once per device (the attribute belongs to the
// function as it is loaded on a device).  One static LdsLimit per kernel; any thread may call: the bit of a device is set
// only after the attribute has been set there, and setting it twice is harmless.
struct LdsLimit {
    std::atomic<uint64_t> devices_done{0};
};
inline int raise_lds_limit(LdsLimit& state, const void* kernel, int bytes, const char* what) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0) return set_error(GGQ_ERR_RUNTIME, "%s: no current device", what);
    const uint64_t bit = device < 64 ? 1ull << device : 0;  // (devices past 63 set the attribute on every launch)
    if (state.devices_done.load(std::memory_order_acquire) & bit) return GGQ_OK;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess)
        return set_error(GGQ_ERR_RUNTIME, "%s: could not raise the dynamic LDS limit to %d bytes", what, bytes);
    state.devices_done.fetch_or(bit, std::memory_order_release);
    return GGQ_OK;
}

inline bool block_multiple(int qt, int64_t k) {
    switch (qt) {
        case 8: return k % 32 == 0;
        case 10: case 11: case 12: case 13: case 14: case 16: return k % 256 == 0;
    }
    return true;  // unknown types are rejected by the callers' switch
}
inline int64_t packed_row_bytes(int qt, int64_t k) {
    switch (qt) {
        case 8: return k / 32 * 34;
        case 10: return k / 256 * 84;
        case 11: return k / 256 * 110;
        case 12: return k / 256 * 144;
        case 13: return k / 256 * 176;
        case 14: return k / 256 * 210;
        case 16: return k / 256 * 66;
    }
    return -1;
}

}  // namespace ggq
