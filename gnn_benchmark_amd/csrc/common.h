// Shared host-side helpers of libgnnagg.so (error reporting, HIP call checking,
// owned device buffers).  gfx950 only; no other backend is supported.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>
#include <string>

#include "gnn_agg.h"

namespace gnnagg {

std::string &last_error_slot();

inline int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error_slot() = buf;
    return code;
}

#define GNNAGG_HIP(expr)                                                                           \
    do {                                                                                           \
        hipError_t e__ = (expr);                                                                   \
        if (e__ != hipSuccess)                                                                     \
            return ::gnnagg::fail(GNNAGG_ERR_HIP, "%s failed: %s (%s:%d)", #expr,                  \
                                  hipGetErrorString(e__), __FILE__, __LINE__);                     \
    } while (0)

#define GNNAGG_REQUIRE(cond, ...)                                                                  \
    do {                                                                                           \
        if (!(cond)) return ::gnnagg::fail(GNNAGG_ERR_INVALID, __VA_ARGS__);                       \
    } while (0)

// Device allocation released on scope exit (setup-time paths only).
template <typename T>
struct DevBuf {
    T *p = nullptr;
    size_t n = 0;
    DevBuf() = default;
    DevBuf(const DevBuf &) = delete;
    DevBuf &operator=(const DevBuf &) = delete;
    ~DevBuf() { reset(); }
    hipError_t alloc(size_t count) {
        reset();
        n = count;
        if (count == 0) return hipSuccess;
        return hipMalloc(reinterpret_cast<void **>(&p), count * sizeof(T));
    }
    void reset() {
        if (p) (void)hipFree(p);
        p = nullptr;
        n = 0;
    }
    T *release() {
        T *r = p;
        p = nullptr;
        n = 0;
        return r;
    }
};

// the largest of the 64 lanes' values, in every lane (all lanes of the wave must call it)
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const unsigned long long o = __shfl_xor(v, off, 64);
        v = o > v ? o : v;
    }
    return v;
}

inline int ceil_log2_u64(uint64_t x) {  // smallest b with 2^b >= x (x >= 1)
    int b = 0;
    while ((uint64_t(1) << b) < x) ++b;
    return b;
}

inline unsigned grid_for(int64_t n, int block) { return (unsigned)((n + block - 1) / block); }

// fp32 -> bf16 as the tensor copy does it: round to nearest even, NaN -> 0x7FC0
__device__ __forceinline__ unsigned short bf16_bits(float x) {
    const uint32_t u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)0x7fc0;
    return (unsigned short)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

}  // namespace gnnagg
