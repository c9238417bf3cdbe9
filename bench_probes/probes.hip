// Memory-system probes of the benchmark (libbenchprobes.so, loaded by bench.py for `--only ceilings` and by nothing
// else): plain kernels with the access mixes of the aggregation path and nothing else, so that a benchmark can put
// the rate of a product kernel next to what the machine delivers for the same mix of row gathers, row reads and row
// writes in the same run.  Not part of libgnnagg.so and not part of its ABI.  Return codes: 0 ok, 1 bad argument,
// 2 HIP error, 3 unsupported row width.
//
//   bench_probe_memory(kind, src, index, dst, count, row_floats, per_row, stream)
//     kind 0  read `count` floats of src as a stream (dst: 4 writable bytes, never written for finite data)
//     kind 1  write `count` floats of dst as a stream
//     kind 2  copy `count` floats from src to dst
//     kind 3  `count` result rows, each the sum of `per_row` rows of src gathered through index[count * per_row]
//             (int32 row numbers of src); the results are dropped: reads only
//     kind 4  the same, every result row written to dst[count, row_floats]
//     kind 5  the same, every result row added onto the row dst holds: one row read and one written per result
//     row_floats (kinds 3-5): 64, 128 or 256; src and dst 16-byte aligned; count a multiple of 4 for kinds 0-2.
//   bench_probe_issue(mfma_rounds, valu_rounds, sink, stream)
//     one block of eight waves per compute unit: waves 0-3 (one per SIMD) issue `mfma_rounds` x 8 independent
//     v_mfma_f32_32x32x16_bf16, waves 4-7 run `valu_rounds` x 8 rounds of the vector-ALU sequence that cuts a pair of
//     fp32 values into bf16 pieces.  Timing (mfma, 0), (0, valu) and (mfma, valu) shows whether the two pipes of a
//     SIMD overlap when different waves feed them.  sink: 4 writable bytes, never written.
// Both allocate nothing and do not synchronise with the host.
#include <hip/hip_runtime.h>
#include <stdint.h>

#define PROBE_REQUIRE(cond) \
    do {                    \
        if (!(cond)) return 1; \
    } while (0)
#define PROBE_HIP(expr)                    \
    do {                                   \
        if ((expr) != hipSuccess) return 2; \
    } while (0)

namespace benchprobes {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// every lane streams 16-byte pieces, U of them in flight
template <int U>
__global__ __launch_bounds__(256) void probe_stream_read_kernel(const f32x4 *__restrict__ x, size_t n4,
                                                                float *__restrict__ sink) {
    size_t i = (size_t)blockIdx.x * 256 * U + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256 * U;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (; i + 256 * (U - 1) < n4; i += stride) {
        f32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(x + i + 256 * u);
#pragma unroll
        for (int u = 0; u < U; ++u) acc += v[u];
    }
    // never true for finite data: keeps the loads alive without a store in the measured stream
    if (acc.x + acc.y + acc.z + acc.w == 1.2345678e38f) sink[0] = acc.x;
}

__global__ __launch_bounds__(256) void probe_stream_write_kernel(f32x4 *__restrict__ y, size_t n4) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    const f32x4 v = {1.f, 2.f, 3.f, 4.f};
    for (; i < n4; i += stride) __builtin_nontemporal_store(v, y + i);
}

__global__ __launch_bounds__(256) void probe_stream_copy_kernel(const f32x4 *__restrict__ x, f32x4 *__restrict__ y,
                                                                size_t n4) {
    size_t i = (size_t)blockIdx.x * 1024 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 1024;
    for (; i + 768 < n4; i += stride) {
        f32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(x + i + 256 * u);
#pragma unroll
        for (int u = 0; u < 4; ++u) __builtin_nontemporal_store(v[u], y + i + 256 * u);
    }
}

// A group of LPR lanes sums `per_row` gathered rows of LPR * 16 bytes (8 gathers in flight) into one result row:
// mode 0 drops the result (reads only), 1 writes it, 2 adds it onto the row the destination holds (read + write).
template <int LPR>
__global__ __launch_bounds__(256) void probe_gather_kernel(const float *__restrict__ x, const int32_t *__restrict__ index,
                                                           float *__restrict__ dst, int64_t results, int per_row,
                                                           int mode, float *__restrict__ sink) {
    constexpr int U = 8;
    const int lig = (int)threadIdx.x & (LPR - 1);
    const int64_t group = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LPR;
    const int64_t ngroups = (int64_t)gridDim.x * 256 / LPR;
    constexpr int kRowFloats = LPR * 4;
    f32x4 keep = {0.f, 0.f, 0.f, 0.f};
    for (int64_t o = group; o < results; o += ngroups) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        float *row = dst + o * kRowFloats + lig * 4;
        if (mode == 2) acc = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(row));
        const int32_t *ip = index + o * per_row;
        for (int j = 0; j < per_row; j += U) {
            f32x4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int jj = j + u < per_row ? j + u : per_row - 1;  // (a repeated gather: a cache hit)
                v[u] = *reinterpret_cast<const f32x4 *>(x + (size_t)ip[jj] * kRowFloats + lig * 4);
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (j + u < per_row) acc += v[u];
        }
        if (mode == 0) keep += acc;
        else __builtin_nontemporal_store(acc, reinterpret_cast<f32x4 *>(row));
    }
    if (mode == 0 && keep.x + keep.y + keep.z + keep.w == 1.2345678e38f) sink[0] = keep.x;
}


// Issue probe: do the matrix pipe and the vector ALU of a SIMD work at the same time when different waves feed
// them?  One block of eight waves per compute unit; waves 0-3 (one per SIMD) issue independent bf16 MFMAs
// (v_mfma_f32_32x32x16_bf16, eight accumulators), waves 4-7 (one per SIMD) run the vector-ALU sequence that cuts fp32
// values into three bf16 pieces.  Either side can be switched off; the caller times the three combinations.
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 probe_bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));

__global__ __launch_bounds__(512) void probe_issue_kernel(float *__restrict__ sink, int mfma_rounds, int valu_rounds) {
    const int wave = threadIdx.x >> 6;
    float s = 0.f;
    if (wave < 4) {
        f32x16 acc[8];
#pragma unroll
        for (int a = 0; a < 8; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][r] = 0.f;
        probe_bf16x8 x, y;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            x[e] = (__bf16)(float)((threadIdx.x + e) & 7);
            y[e] = (__bf16)(float)(e + 1);
        }
        for (int i = 0; i < mfma_rounds; ++i) {
#pragma unroll
            for (int a = 0; a < 8; ++a) acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, acc[a], 0, 0, 0);
        }
#pragma unroll
        for (int a = 0; a < 8; ++a) s += acc[a][0] + acc[a][15];
    } else {
        f32x2 v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = f32x2{(float)(threadIdx.x + e) * 1.37f, (float)(e + 1) * 0.77f};
        for (int i = 0; i < valu_rounds; ++i) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {  // hi = bf16(v), mid = bf16(v - hi), what is left feeds the next round
                const probe_bf16x2 hi = __builtin_convertvector(v[e], probe_bf16x2);
                const f32x2 r = v[e] - __builtin_convertvector(hi, f32x2);
                const probe_bf16x2 mid = __builtin_convertvector(r, probe_bf16x2);
                const f32x2 r2 = r - __builtin_convertvector(mid, f32x2);
                v[e] = r2 * 65536.0f + v[e];
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) s += v[e].x + v[e].y;
    }
    if (s == 1.2345678e38f) sink[0] = s;  // never true: keeps the work alive
}

}  // namespace
}  // namespace benchprobes

using namespace benchprobes;

extern "C" int bench_probe_memory(int kind, const float *src, const int32_t *index, float *dst, int64_t count,
                                   int64_t row_floats, int64_t per_row, void *stream) {
    PROBE_REQUIRE(kind >= 0 && kind <= 5);
    PROBE_REQUIRE(count >= 0 && count < (int64_t(1) << 40));
    if (count == 0) return 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (kind <= 2) {  // streams over `count` floats
        PROBE_REQUIRE(count % 4 == 0);
        PROBE_REQUIRE((kind == 1 || src) && (kind == 0 || dst));
        PROBE_REQUIRE(((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0);
        const size_t n4 = (size_t)count / 4;
        const unsigned blocks = 32768;
        if (kind == 0) {
            PROBE_REQUIRE(dst);
            hipLaunchKernelGGL(probe_stream_read_kernel<8>, dim3(blocks), dim3(256), 0, st,
                               reinterpret_cast<const f32x4 *>(src), n4, dst);
        } else if (kind == 1) {
            hipLaunchKernelGGL(probe_stream_write_kernel, dim3(blocks), dim3(256), 0, st, reinterpret_cast<f32x4 *>(dst), n4);
        } else {
            hipLaunchKernelGGL(probe_stream_copy_kernel, dim3(blocks), dim3(256), 0, st,
                               reinterpret_cast<const f32x4 *>(src), reinterpret_cast<f32x4 *>(dst), n4);
        }
        PROBE_HIP(hipGetLastError());
        return 0;
    }
    // row gathers: `count` result rows, each the sum of `per_row` gathered rows
    PROBE_REQUIRE(src && index && dst);
    PROBE_REQUIRE(per_row >= 1 && per_row < (1 << 20));
    PROBE_REQUIRE(((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0);
    const int mode = kind - 3;
    const unsigned blocks = 65536;
    // in mode 0 the last 4 bytes of dst stand in for the sink (never written for finite data)
    float *sink = dst;
    if (row_floats == 64)
        hipLaunchKernelGGL(probe_gather_kernel<16>, dim3(blocks), dim3(256), 0, st, src, index, dst, count, (int)per_row, mode, sink);
    else if (row_floats == 128)
        hipLaunchKernelGGL(probe_gather_kernel<32>, dim3(blocks), dim3(256), 0, st, src, index, dst, count, (int)per_row, mode, sink);
    else if (row_floats == 256)
        hipLaunchKernelGGL(probe_gather_kernel<64>, dim3(blocks), dim3(256), 0, st, src, index, dst, count, (int)per_row, mode, sink);
    else
        return 3;
    PROBE_HIP(hipGetLastError());
    return 0;
}

extern "C" int bench_probe_issue(int mfma_rounds, int valu_rounds, float *sink, void *stream) {
    PROBE_REQUIRE(mfma_rounds >= 0 && valu_rounds >= 0 && mfma_rounds <= (1 << 20) && valu_rounds <= (1 << 20));
    PROBE_REQUIRE(sink);
    int dev = 0, cus = 0;
    PROBE_HIP(hipGetDevice(&dev));
    PROBE_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    hipLaunchKernelGGL(probe_issue_kernel, dim3(cus > 0 ? cus : 256), dim3(512), 0, static_cast<hipStream_t>(stream), sink,
                       mfma_rounds, valu_rounds);
    PROBE_HIP(hipGetLastError());
    return 0;
}
