// Codec of the boundary buffers: fp32 rows <-> int2 / int4 / int8 with one (zero_point, scale)
// pair per row.  Two layouts, both the reference's:
//
//  * row-packed per destination rank: 8/bits consecutive rows of one rank's segment share a
//    byte per feature column, row k of a group at bit (8/bits - k - 1) * bits
//    (model/ops/src/quantization_arm.cpp:78-300, :364-479; quantization_x86.cpp:17-162);
//  * feature-packed with a width per row ("mixed bits"): 8/bits consecutive features of a row
//    share a byte, same shift rule (quantization_x86.cpp:164-305).
//
// Arithmetic is the reference's: zero_point = min(row), scale = (max - min) / (2^bits - 1)
// (1 when that is 0), q = rint((x - zero_point) / scale) to nearest even with an IEEE
// division, x' = fma(q, scale, zero_point).
//
// All kernels stream: HBM-bound.  One lane group (16, 32 or 64 lanes, by row width) owns
// one group of rows that share bytes; the rows are held in registers between the min/max
// pass and the packing pass when they fit (F <= 1024), so the fp32 rows are read from
// memory once.
#include "common.h"

namespace gnnagg {
namespace {

typedef float f4 __attribute__((ext_vector_type(4)));

template <int VEC>
struct QVec;
template <>
struct QVec<4> {
    f4 v;
    __device__ __forceinline__ static QVec load(const float *p) {
        return QVec{__builtin_nontemporal_load(reinterpret_cast<const f4 *>(p))};
    }
    __device__ __forceinline__ float get(int i) const { return v[i]; }
    __device__ __forceinline__ static void store(float *p, const float (&x)[4]) {
        const f4 o = {x[0], x[1], x[2], x[3]};
        __builtin_nontemporal_store(o, reinterpret_cast<f4 *>(p));
    }
    __device__ __forceinline__ static void store_bytes(uint8_t *p, const uint32_t (&b)[4]) {
        *reinterpret_cast<uint32_t *>(p) = (b[0] & 0xFF) | ((b[1] & 0xFF) << 8) | ((b[2] & 0xFF) << 16) | (b[3] << 24);
    }
    __device__ __forceinline__ static void load_bytes(const uint8_t *p, uint32_t (&b)[4]) {
        const uint32_t w = *reinterpret_cast<const uint32_t *>(p);
        b[0] = w & 0xFF;
        b[1] = (w >> 8) & 0xFF;
        b[2] = (w >> 16) & 0xFF;
        b[3] = w >> 24;
    }
};
template <>
struct QVec<1> {
    float v;
    __device__ __forceinline__ static QVec load(const float *p) { return QVec{__builtin_nontemporal_load(p)}; }
    __device__ __forceinline__ float get(int) const { return v; }
    __device__ __forceinline__ static void store(float *p, const float (&x)[1]) { __builtin_nontemporal_store(x[0], p); }
    __device__ __forceinline__ static void store_bytes(uint8_t *p, const uint32_t (&b)[1]) { *p = (uint8_t)b[0]; }
    __device__ __forceinline__ static void load_bytes(const uint8_t *p, uint32_t (&b)[1]) { b[0] = *p; }
};

// min / max over the lanes of one group (G a power of two <= 64)
template <int G>
__device__ __forceinline__ void group_min_max(float &lo, float &hi) {
#pragma unroll
    for (int d = G / 2; d >= 1; d >>= 1) {
        lo = fminf(lo, __shfl_xor(lo, d, G));
        hi = fmaxf(hi, __shfl_xor(hi, d, G));
    }
}

// rint((x - zp) / scale) as the 32-bit pattern the reference shifts and ORs (cvt to int32, ties to even)
__device__ __forceinline__ uint32_t quantize_one(float x, float zp, float scale) {
    return (uint32_t)__float2int_rn(__fdiv_rn(__fsub_rn(x, zp), scale));
}

__device__ __forceinline__ void params_of(float lo, float hi, int bits, float &zp, float &scale) {
    zp = lo;
    scale = __fdiv_rn(__fsub_rn(hi, lo), (float)((1 << bits) - 1));
    if (scale == 0.0f) scale = 1.0f;
}

// Which segment a packed row belongs to: the last p with packed_range[p] <= g.
__device__ __forceinline__ int segment_of(const int32_t *__restrict__ packed_range, int segments, int g) {
    int lo = 0, hi = segments;  // invariant: packed_range[lo] <= g < packed_range[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (packed_range[mid] <= g) lo = mid;
        else hi = mid;
    }
    return lo;
}

struct RowGroup {
    int first;  // first fp32 row
    int count;  // rows of the group that exist (0 = nothing to do)
};

template <int EPB>
__device__ __forceinline__ RowGroup locate_group(const int32_t *__restrict__ row_range,
                                                 const int32_t *__restrict__ packed_range, int segments, int g,
                                                 int rows) {
    const int p = segment_of(packed_range, segments, g);
    const int first = row_range[p] + (g - packed_range[p]) * EPB;
    int end = row_range[p + 1];
    if (end > rows) end = rows;
    int count = end - first;
    if (count > EPB) count = EPB;
    if (count < 0 || first < 0) count = 0;
    return RowGroup{first, count};
}

// NV = float vectors a lane keeps per row between the two passes (0: rows are read twice).
template <int BITS, int VEC, int G, int NV>
__global__ __launch_bounds__(256) void quantize_segments_kernel(const float *__restrict__ x, uint8_t *__restrict__ packed,
                                                                float *__restrict__ params,
                                                                const int32_t *__restrict__ row_range,
                                                                const int32_t *__restrict__ packed_range, int segments,
                                                                int rows, int packed_rows, int feat) {
    constexpr int EPB = 8 / BITS;
    constexpr int KEEP = NV > 0 ? NV : 1;
    const int g = (int)(((int64_t)blockIdx.x * 256 + threadIdx.x) / G);
    if (g >= packed_rows) return;  // whole lane groups leave together
    const int l = (int)threadIdx.x & (G - 1);
    const RowGroup rg = locate_group<EPB>(row_range, packed_range, segments, g, rows);
    const int nvec = (feat + VEC - 1) / VEC;  // VEC == 4 implies feat % 4 == 0

    QVec<VEC> held[EPB][KEEP];
    float zp[EPB], scale[EPB];
#pragma unroll
    for (int k = 0; k < EPB; ++k) {
        zp[k] = 0.0f;
        scale[k] = 1.0f;
        if (k < rg.count) {
            const float *row = x + (size_t)(rg.first + k) * (size_t)feat;
            float lo = INFINITY, hi = -INFINITY;
            if (NV > 0) {
#pragma unroll
                for (int j = 0; j < KEEP; ++j) {
                    const int v = l + G * j;
                    if (v < nvec) {
                        held[k][j] = QVec<VEC>::load(row + (size_t)v * VEC);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) {
                            lo = fminf(lo, held[k][j].get(e));
                            hi = fmaxf(hi, held[k][j].get(e));
                        }
                    }
                }
            } else {
                for (int v = l; v < nvec; v += G) {
                    const QVec<VEC> t = QVec<VEC>::load(row + (size_t)v * VEC);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        lo = fminf(lo, t.get(e));
                        hi = fmaxf(hi, t.get(e));
                    }
                }
            }
            group_min_max<G>(lo, hi);
            params_of(lo, hi, BITS, zp[k], scale[k]);
            if (l == 0) {
                params[(size_t)(rg.first + k) * 2 + 0] = zp[k];
                params[(size_t)(rg.first + k) * 2 + 1] = scale[k];
            }
        }
    }

    uint8_t *dst = packed + (size_t)g * (size_t)feat;
    auto pack = [&](int v, int j) {
        uint32_t byte[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) byte[e] = 0;
#pragma unroll
        for (int k = 0; k < EPB; ++k) {
            if (k < rg.count) {
                QVec<VEC> t;
                if (NV > 0) t = held[k][j];
                else t = QVec<VEC>::load(x + (size_t)(rg.first + k) * (size_t)feat + (size_t)v * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e) byte[e] |= quantize_one(t.get(e), zp[k], scale[k]) << ((EPB - k - 1) * BITS);
            }
        }
        QVec<VEC>::store_bytes(dst + (size_t)v * VEC, byte);
    };
    if (NV > 0) {
#pragma unroll
        for (int j = 0; j < KEEP; ++j) {
            const int v = l + G * j;
            if (v < nvec) pack(v, j);
        }
    } else {
        for (int v = l; v < nvec; v += G) pack(v, 0);
    }
}

template <int BITS, int VEC, int G>
__global__ __launch_bounds__(256) void dequantize_segments_kernel(const uint8_t *__restrict__ packed,
                                                                  const float *__restrict__ params,
                                                                  float *__restrict__ out,
                                                                  const int32_t *__restrict__ row_range,
                                                                  const int32_t *__restrict__ packed_range,
                                                                  int segments, int rows, int packed_rows, int feat) {
    constexpr int EPB = 8 / BITS;
    constexpr uint32_t kMask = (1u << BITS) - 1u;
    const int g = (int)(((int64_t)blockIdx.x * 256 + threadIdx.x) / G);
    if (g >= packed_rows) return;
    const int l = (int)threadIdx.x & (G - 1);
    const RowGroup rg = locate_group<EPB>(row_range, packed_range, segments, g, rows);
    const int nvec = (feat + VEC - 1) / VEC;
    float zp[EPB], scale[EPB];
#pragma unroll
    for (int k = 0; k < EPB; ++k) {
        zp[k] = 0.0f;
        scale[k] = 0.0f;
        if (k < rg.count) {
            zp[k] = params[(size_t)(rg.first + k) * 2 + 0];
            scale[k] = params[(size_t)(rg.first + k) * 2 + 1];
        }
    }
    const uint8_t *src = packed + (size_t)g * (size_t)feat;
    for (int v = l; v < nvec; v += G) {
        uint32_t byte[VEC];
        QVec<VEC>::load_bytes(src + (size_t)v * VEC, byte);
#pragma unroll
        for (int k = 0; k < EPB; ++k) {
            if (k < rg.count) {
                float o[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    o[e] = __fmaf_rn((float)((byte[e] >> ((EPB - k - 1) * BITS)) & kMask), scale[k], zp[k]);
                QVec<VEC>::store(out + (size_t)(rg.first + k) * (size_t)feat + (size_t)v * VEC, o);
            }
        }
    }
}

// ---- mixed bits: one wavefront per row, width read from params[row][0]

__global__ __launch_bounds__(256) void quantize_mixed_kernel(const float *__restrict__ x, uint8_t *__restrict__ data,
                                                             const int64_t *__restrict__ feat_range,
                                                             float *__restrict__ params, int rows, int feat,
                                                             int *__restrict__ bad_width) {
    const int row = (int)(((int64_t)blockIdx.x * 256 + threadIdx.x) >> 6);
    if (row >= rows) return;
    const int l = (int)threadIdx.x & 63;
    const int bits = (int)params[(size_t)row * 3];
    if (bits != 2 && bits != 4 && bits != 8) {  // the reference prints an error and leaves the row alone
        if (l == 0) atomicOr(bad_width, 1);
        return;
    }
    const float *src = x + (size_t)row * (size_t)feat;
    float lo = INFINITY, hi = -INFINITY;
    for (int j = l; j < feat; j += 64) {
        const float t = src[j];
        lo = fminf(lo, t);
        hi = fmaxf(hi, t);
    }
    group_min_max<64>(lo, hi);
    float zp, scale;
    params_of(lo, hi, bits, zp, scale);
    if (l == 0) {
        params[(size_t)row * 3 + 1] = zp;
        params[(size_t)row * 3 + 2] = scale;
    }
    const int epb = 8 / bits;
    const int nbytes = (feat + epb - 1) / epb;
    uint8_t *dst = data + feat_range[row];
    for (int b = l; b < nbytes; b += 64) {
        uint32_t byte = 0;
        for (int k = 0; k < epb; ++k) {
            const int j = b * epb + k;
            if (j < feat) byte |= quantize_one(src[j], zp, scale) << ((epb - k - 1) * bits);
        }
        dst[b] = (uint8_t)byte;
    }
}

__global__ __launch_bounds__(256) void dequantize_mixed_kernel(const uint8_t *__restrict__ data,
                                                               const int64_t *__restrict__ feat_range,
                                                               const float *__restrict__ params,
                                                               float *__restrict__ out, int rows, int feat,
                                                               int *__restrict__ bad_width) {
    const int row = (int)(((int64_t)blockIdx.x * 256 + threadIdx.x) >> 6);
    if (row >= rows) return;
    const int l = (int)threadIdx.x & 63;
    const int bits = (int)params[(size_t)row * 3];
    if (bits != 2 && bits != 4 && bits != 8) {
        if (l == 0) atomicOr(bad_width, 1);
        return;
    }
    const float zp = params[(size_t)row * 3 + 1], scale = params[(size_t)row * 3 + 2];
    const int epb = 8 / bits;
    const uint32_t mask = (1u << bits) - 1u;
    const int64_t begin = feat_range[row];
    const int nbytes = (int)(feat_range[row + 1] - begin);
    float *dst = out + (size_t)row * (size_t)feat;
    for (int j = l; j < feat; j += 64) {
        const int b = j / epb, k = j - b * epb;
        if (b < nbytes) dst[j] = __fmaf_rn((float)(((uint32_t)data[begin + b] >> ((epb - k - 1) * bits)) & mask), scale, zp);
    }
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
bool aligned4(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 3) == 0; }

struct SegArgs {
    const int32_t *row_range, *packed_range;
    int segments, rows, packed_rows, feat;
    hipStream_t st;
};

template <int BITS, int VEC, int G>
void launch_quantize(const float *x, uint8_t *packed, float *params, const SegArgs &a) {
    const int nvec = (a.feat + VEC - 1) / VEC;
    const unsigned blocks = grid_for((int64_t)a.packed_rows * G, 256);
    if (nvec <= G)
        hipLaunchKernelGGL((quantize_segments_kernel<BITS, VEC, G, 1>), dim3(blocks), dim3(256), 0, a.st, x, packed, params,
                           a.row_range, a.packed_range, a.segments, a.rows, a.packed_rows, a.feat);
    else if (nvec <= 4 * G)
        hipLaunchKernelGGL((quantize_segments_kernel<BITS, VEC, G, 4>), dim3(blocks), dim3(256), 0, a.st, x, packed, params,
                           a.row_range, a.packed_range, a.segments, a.rows, a.packed_rows, a.feat);
    else
        hipLaunchKernelGGL((quantize_segments_kernel<BITS, VEC, G, 0>), dim3(blocks), dim3(256), 0, a.st, x, packed, params,
                           a.row_range, a.packed_range, a.segments, a.rows, a.packed_rows, a.feat);
}

template <int BITS, int VEC>
void launch_quantize_g(const float *x, uint8_t *packed, float *params, const SegArgs &a) {
    const int nvec = (a.feat + VEC - 1) / VEC;
    if (nvec <= 16) launch_quantize<BITS, VEC, 16>(x, packed, params, a);
    else if (nvec <= 32) launch_quantize<BITS, VEC, 32>(x, packed, params, a);
    else launch_quantize<BITS, VEC, 64>(x, packed, params, a);
}

template <int BITS, int VEC>
void launch_dequantize_g(const uint8_t *packed, const float *params, float *out, const SegArgs &a) {
    const int nvec = (a.feat + VEC - 1) / VEC;
#define GNNAGG_DEQ(G)                                                                                              \
    hipLaunchKernelGGL((dequantize_segments_kernel<BITS, VEC, G>), dim3(grid_for((int64_t)a.packed_rows * G, 256)), \
                       dim3(256), 0, a.st, packed, params, out, a.row_range, a.packed_range, a.segments, a.rows,   \
                       a.packed_rows, a.feat)
    if (nvec <= 16) GNNAGG_DEQ(16);
    else if (nvec <= 32) GNNAGG_DEQ(32);
    else GNNAGG_DEQ(64);
#undef GNNAGG_DEQ
}

int check_segments(const void *a, const void *b, const void *c, const int32_t *row_range, const int32_t *packed_range,
                   int64_t segments, int64_t rows, int64_t packed_rows, int64_t feat, int bits) {
    GNNAGG_REQUIRE(bits == 2 || bits == 4 || bits == 8, "bits must be 2, 4 or 8 (got %d)", bits);
    GNNAGG_REQUIRE(segments >= 1 && rows >= 0 && packed_rows >= 0 && feat >= 0, "bad size");
    GNNAGG_REQUIRE(rows < (int64_t(1) << 31) - 8 && feat <= (1 << 20) && segments < (1 << 24), "size out of range");
    GNNAGG_REQUIRE(packed_rows * (8 / bits) >= rows && packed_rows <= rows + segments,
                   "packed_rows=%lld does not fit rows=%lld in %lld segments", (long long)packed_rows, (long long)rows,
                   (long long)segments);
    if (rows == 0 || feat == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(a && b && c && row_range && packed_range, "null pointer");
    return GNNAGG_OK;
}

}  // namespace
}  // namespace gnnagg

using namespace gnnagg;

extern "C" int gnnagg_quantize_segments_f32(const float *x, uint8_t *packed, float *params, const int32_t *row_range,
                                            const int32_t *packed_range, int64_t segments, int64_t rows,
                                            int64_t packed_rows, int64_t feat, int bits, void *stream) {
    const int rc = check_segments(x, packed, params, row_range, packed_range, segments, rows, packed_rows, feat, bits);
    if (rc != GNNAGG_OK || rows == 0 || feat == 0) return rc;
    const SegArgs a{row_range, packed_range, (int)segments, (int)rows, (int)packed_rows, (int)feat,
                    static_cast<hipStream_t>(stream)};
    const bool v4 = feat % 4 == 0 && aligned16(x) && aligned4(packed);
#define GNNAGG_Q(B)                                                      \
    if (bits == B) {                                                     \
        if (v4) launch_quantize_g<B, 4>(x, packed, params, a);           \
        else launch_quantize_g<B, 1>(x, packed, params, a);              \
    }
    GNNAGG_Q(2) GNNAGG_Q(4) GNNAGG_Q(8)
#undef GNNAGG_Q
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

extern "C" int gnnagg_dequantize_segments_f32(const uint8_t *packed, const float *params, float *out,
                                              const int32_t *row_range, const int32_t *packed_range,
                                              int64_t segments, int64_t rows, int64_t packed_rows, int64_t feat,
                                              int bits, void *stream) {
    const int rc = check_segments(packed, params, out, row_range, packed_range, segments, rows, packed_rows, feat, bits);
    if (rc != GNNAGG_OK || rows == 0 || feat == 0) return rc;
    const SegArgs a{row_range, packed_range, (int)segments, (int)rows, (int)packed_rows, (int)feat,
                    static_cast<hipStream_t>(stream)};
    const bool v4 = feat % 4 == 0 && aligned16(out) && aligned4(packed);
#define GNNAGG_D(B)                                                      \
    if (bits == B) {                                                     \
        if (v4) launch_dequantize_g<B, 4>(packed, params, out, a);       \
        else launch_dequantize_g<B, 1>(packed, params, out, a);          \
    }
    GNNAGG_D(2) GNNAGG_D(4) GNNAGG_D(8)
#undef GNNAGG_D
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

extern "C" int gnnagg_quantize_mixed_f32(const float *x, uint8_t *data, const int64_t *feat_range, float *params,
                                         int64_t rows, int64_t feat, int32_t *bad_width, void *stream) {
    GNNAGG_REQUIRE(rows >= 0 && feat >= 0 && rows < (int64_t(1) << 31) && feat <= (1 << 20), "bad size");
    if (rows == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(params && feat_range && bad_width, "null params / feat_range / bad_width");
    if (feat == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(x && data, "null x / data");
    hipLaunchKernelGGL(quantize_mixed_kernel, dim3(grid_for(rows * 64, 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), x, data, feat_range, params, (int)rows, (int)feat, bad_width);
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

extern "C" int gnnagg_dequantize_mixed_f32(const uint8_t *data, const int64_t *feat_range, const float *params,
                                           float *out, int64_t rows, int64_t feat, int32_t *bad_width, void *stream) {
    GNNAGG_REQUIRE(rows >= 0 && feat >= 0 && rows < (int64_t(1) << 31) && feat <= (1 << 20), "bad size");
    if (rows == 0 || feat == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(data && feat_range && params && out && bad_width, "null pointer");
    hipLaunchKernelGGL(dequantize_mixed_kernel, dim3(grid_for(rows * 64, 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), data, feat_range, params, out, (int)rows, (int)feat, bad_width);
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}
