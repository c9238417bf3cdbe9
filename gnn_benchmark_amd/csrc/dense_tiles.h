// Building blocks of the dense MFMA kernels: vector types, the chunk size of the LDS pipeline,
// and the loader that copies a contiguous run of rows from global memory into an LDS tile
// through registers.
#pragma once

#include "common.h"

namespace gnnagg {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// Four fp32 values as three times four bf16: hi = bf16(v), mid = bf16(v - hi), lo = bf16(v - hi - mid).  Both
// differences are exact in fp32, so hi + mid + lo is v to 2^-25 of its size (three 8-bit pieces of a 24-bit mantissa).
__device__ inline void split_bf16x3(float a, float b, float c, float d, shortx4 (&out)[3]) {
    union {
        bf16x2 h[2];
        shortx4 s;
    } u[3];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const floatx2 v = q == 0 ? floatx2{a, b} : floatx2{c, d};
        u[0].h[q] = __builtin_convertvector(v, bf16x2);
        const floatx2 r = v - __builtin_convertvector(u[0].h[q], floatx2);
        u[1].h[q] = __builtin_convertvector(r, bf16x2);
        u[2].h[q] = __builtin_convertvector(r - __builtin_convertvector(u[1].h[q], floatx2), bf16x2);
    }
    out[0] = u[0].s;
    out[1] = u[1].s;
    out[2] = u[2].s;
}

// four fp32 values -> four bf16 (round to nearest even, the hardware's packed conversion) in 8 bytes
__device__ inline shortx4 to_bf16x4(float a, float b, float c, float d) {
    union {
        bf16x2 h[2];
        shortx4 s;
    } u;
    u.h[0] = __builtin_convertvector(floatx2{a, b}, bf16x2);
    u.h[1] = __builtin_convertvector(floatx2{c, d}, bf16x2);
    return u.s;
}

constexpr int kChunk = 16;    // rows per LDS stage
constexpr int kLdsPad = 32;   // floats: shifts the second row of a k-pair onto the other half of the banks

// One operand's share of the loader: thread t moves float4 number t + 256*j of the chunk's
// kChunk * width values.  The rows may sit `stride` floats apart in global memory (a column
// block of a wider row-major array).
template <int NV, int LD>
struct ChunkLoader {
    int lds_off[NV];   // destination (floats) inside one LDS buffer, or -1 for a vector beyond the chunk
    int elem[NV];      // number of the vector's first value inside the chunk, 0 when unused
    int src_off[NV];   // where that value sits (floats from the start of the chunk's first row), 0 when unused
    floatx4 reg[NV];
    int width, stride;

    __device__ int offset_of(int e) const { return (e / width) * stride + e % width; }

    __device__ void init(int tid, int w, int ld) {
        width = w;
        stride = ld;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int e = 4 * (tid + 256 * j);
            const bool used = e < kChunk * w;
            lds_off[j] = used ? (e / w) * LD + (e % w) : -1;
            elem[j] = used ? e : 0;
            src_off[j] = used ? offset_of(e) : 0;
        }
    }
    // all kChunk rows exist
    __device__ void fetch(const float *chunk) {
#pragma unroll
        for (int j = 0; j < NV; ++j)
            reg[j] = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(chunk + src_off[j]));
    }
    // the same for an operand that every block reads again (stays in cache)
    __device__ void fetch_cached(const float *chunk) {
#pragma unroll
        for (int j = 0; j < NV; ++j) reg[j] = *reinterpret_cast<const floatx4 *>(chunk + src_off[j]);
    }
    // only the first `valid` values of the chunk exist; the rest reads as zeros.  `aligned` is false
    // when rows are not a whole number of float4 (then fetch() is never used either).
    __device__ void fetch_tail(const float *chunk, int valid, bool aligned) {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            const int e = elem[j];
            if (lds_off[j] >= 0) {
                if (aligned) {
                    if (e < valid) v = *reinterpret_cast<const floatx4 *>(chunk + src_off[j]);
                } else {
                    if (e + 0 < valid) v.x = chunk[offset_of(e + 0)];
                    if (e + 1 < valid) v.y = chunk[offset_of(e + 1)];
                    if (e + 2 < valid) v.z = chunk[offset_of(e + 2)];
                    if (e + 3 < valid) v.w = chunk[offset_of(e + 3)];
                }
            }
            reg[j] = v;
        }
    }
    // Steady-state store: unconditional, so that no load is tied to a branch; a vector beyond the
    // chunk goes to the thread's own 16 bytes of `dump`.
    __device__ void store_all(float *buf, float *dump) const {
#pragma unroll
        for (int j = 0; j < NV; ++j)
            *reinterpret_cast<floatx4 *>(lds_off[j] >= 0 ? buf + lds_off[j] : dump) = reg[j];
    }
    __device__ void store(float *buf, bool aligned) const {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            if (lds_off[j] < 0) continue;
            if (aligned) {
                *reinterpret_cast<floatx4 *>(buf + lds_off[j]) = reg[j];
            } else {  // a float4 of the stream may straddle two rows
                const int e = elem[j];
                const float v[4] = {reg[j].x, reg[j].y, reg[j].z, reg[j].w};
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (e + q < kChunk * width) buf[((e + q) / width) * LD + (e + q) % width] = v[q];
            }
        }
    }
};

// Dynamic LDS beyond 64 KB has to be allowed per kernel and per device before the first launch.
inline hipError_t allow_lds(const void *kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return hipSuccess;
    return hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

}  // namespace gnnagg
