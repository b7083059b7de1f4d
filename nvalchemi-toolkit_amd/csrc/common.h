// Shared host/device helpers for the gfx950 kernels of libnvalchemi_amd.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "nvalchemi_amd.h"

#define NVAMD_EXPORT extern "C" __attribute__((visibility("default")))

namespace nvamd {

constexpr int kWave = 64;  // CDNA wavefront width

// thread-local message behind nvamd_last_error()
char* error_buffer();
int32_t fail(int32_t code, const char* fmt, ...);

inline size_t align_up(size_t x, size_t a = 256) { return (x + a - 1) / a * a; }

inline int32_t check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return NVAMD_OK;
    return fail(NVAMD_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define NVAMD_LAUNCH_CHECK(what)                                     \
    do {                                                             \
        int32_t _rc = ::nvamd::check_hip(hipGetLastError(), (what)); \
        if (_rc != NVAMD_OK) return _rc;                             \
    } while (0)

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- device helpers -----------------------------------------------------------------------

__device__ __forceinline__ int lane_id() { return (int)__lane_id(); }

// wave-wide sum of a double via xor shuffles (all 64 lanes end with the total)
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// hardware fp64 add to global memory (no compare-and-swap loop)
__device__ __forceinline__ void atomic_add_f64(double* p, double v) { unsafeAtomicAdd(p, v); }

// order-preserving map float -> uint32 so that atomicMin/Max on the image orders the floats
__device__ __forceinline__ uint32_t float_order_key(float f) {
    uint32_t b = __float_as_uint(f);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float float_from_order_key(uint32_t k) {
    uint32_t b = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __uint_as_float(b);
}

}  // namespace nvamd
