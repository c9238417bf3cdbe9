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
// All kernels stream: HBM-bound (quantise reads 4F + writes F*bits/8 + 8 bytes per row,
// dequantise the reverse).  One lane group (16, 32 or 64 lanes, by row width) owns four fp32
// rows at a time -- one, two or four groups of rows that share bytes; the rows are held in
// registers between the min/max pass and the packing pass when they fit (F <= 1024), so the
// fp32 rows are read from memory once.  The per-rank prefix arrays are staged in LDS.
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

// The same value without an IEEE division per element.  t = d * rcp(scale) lies within 2.4e-7 * |t|
// of the correctly rounded quotient fl(d / scale) (v_rcp_f32 is good to 1 ulp, the product adds
// half an ulp, fl() itself another half).  For |t| < 512 that is less than 1.3e-4, so unless t comes
// closer than 2e-4 to a half-integer, t and fl(d / scale) round to the same integer; the rare close
// calls, and anything large or not finite (every comparison with a NaN is false), take the exact
// division.  (Codes are at most 255, so a larger |t| only arises from non-finite or overflowing input.)
__device__ __forceinline__ uint32_t quantize_one_fast(float x, float zp, float scale, float inv_scale) {
    const float d = __fsub_rn(x, zp);
    const float t = __fmul_rn(d, inv_scale);
    float k = rintf(t);
    const bool safe = fabsf(__fsub_rn(t, k)) < 0.4998f && fabsf(t) < 512.0f;
    if (!safe) k = rintf(__fdiv_rn(d, scale));
    return (uint32_t)(int)k;
}

__device__ __forceinline__ void params_of(float lo, float hi, int bits, float &zp, float &scale) {
    zp = lo;
    scale = __fdiv_rn(__fsub_rn(hi, lo), (float)((1 << bits) - 1));
    if (scale == 0.0f) scale = 1.0f;
}

// Which segment a packed row belongs to: the last p with packed_range[p] <= g.
__device__ __forceinline__ int segment_of(const int32_t *packed_range, int segments, int g) {
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
__device__ __forceinline__ RowGroup locate_group(const int32_t *row_range, const int32_t *packed_range, int segments,
                                                 int g, int rows, int packed_rows) {
    if (g >= packed_rows) return RowGroup{0, 0};
    const int p = segment_of(packed_range, segments, g);
    const int first = row_range[p] + (g - packed_range[p]) * EPB;
    int end = row_range[p + 1];
    if (end > rows) end = rows;
    int count = end - first;
    if (count > EPB) count = EPB;
    if (count < 0 || first < 0) count = 0;
    return RowGroup{first, count};
}

constexpr int kCodecIters = 8;         // slices a lane group walks per launch
constexpr int kRowsPerLaneGroup = 4;   // fp32 rows one lane group handles, whatever the width
constexpr int kMaxLdsSegments = 4095;  // both prefix arrays of up to this many segments are staged in LDS

// The per-rank prefix arrays are searched by every lane group; a block copies them into LDS
// once (when they fit) so that the search costs no chain of global-memory round trips.
__device__ __forceinline__ void stage_ranges(const int32_t *__restrict__ row_range,
                                             const int32_t *__restrict__ packed_range, int segments, int32_t *lds,
                                             const int32_t *&rr, const int32_t *&pr) {
    if (segments <= kMaxLdsSegments) {
        for (int i = (int)threadIdx.x; i <= segments; i += 256) {
            lds[i] = row_range[i];
            lds[segments + 1 + i] = packed_range[i];
        }
        __syncthreads();
        rr = lds;
        pr = lds + segments + 1;
    } else {
        rr = row_range;
        pr = packed_range;
    }
}

// One lane group of G lanes handles GPL = kRowsPerLaneGroup / EPB consecutive packed rows at a
// time, i.e. the same number of fp32 rows whatever the width, and walks kCodecIters such slices of
// its block's share: the rows of the next slice are loaded before the current slice is reduced,
// packed and stored, so loads stay in flight throughout.
// NV = float vectors a lane keeps per row between the two passes (0: rows are read twice, no
// prefetch).
template <int BITS, int VEC, int G, int NV>
__global__ __launch_bounds__(256) void quantize_segments_kernel(const float *__restrict__ x, uint8_t *__restrict__ packed,
                                                                float *__restrict__ params,
                                                                const int32_t *__restrict__ row_range,
                                                                const int32_t *__restrict__ packed_range, int segments,
                                                                int rows, int packed_rows, int feat,
                                                                const int64_t *__restrict__ index, int64_t src_rows) {
    constexpr int EPB = 8 / BITS;
    constexpr int GPL = kRowsPerLaneGroup / EPB;
    constexpr int KEEP = NV > 0 ? NV : 1;
    constexpr int kLaneGroups = 256 / G;
    constexpr bool kPrefetch = NV == 1;  // two slices of rows in registers
    extern __shared__ int32_t range_lds[];
    const int32_t *rr, *pr;
    stage_ranges(row_range, packed_range, segments, range_lds, rr, pr);

    const int l = (int)threadIdx.x & (G - 1);
    const int nvec = (feat + VEC - 1) / VEC;  // VEC == 4 implies feat % 4 == 0
    // where fp32 row r of the buffer lies: in x itself, or (index given: the gather of raw boundary rows folded in)
    // at row index[r] of x -- an index outside x is never dereferenced, row 0 is read in its place and the row's
    // parameters are stored as NaN, so that whoever dequantises the row gets NaN (what the plain row gather stores
    // for such an index)
    auto row_is_bad = [&](int r) -> bool { return index && (uint64_t)index[r] >= (uint64_t)src_rows; };
    auto row_at = [&](int r) -> const float * {
        size_t at = (size_t)r;
        if (index) {
            const int64_t i = index[r];
            at = (uint64_t)i < (uint64_t)src_rows ? (size_t)i : 0;
        }
        return x + at * (size_t)feat;
    };

    struct Slice {
        int g0;
        RowGroup rg[GPL];
        QVec<VEC> held[GPL][EPB][KEEP];
    };
    auto slice_start = [&](int it) {
        return (int)((((int64_t)blockIdx.x * kCodecIters + it) * kLaneGroups + (int)threadIdx.x / G) * GPL);
    };
    // locate the slice's rows and (NV > 0) issue their loads
    auto fetch = [&](int it, Slice &sl) {
        sl.g0 = slice_start(it);
#pragma unroll
        for (int u = 0; u < GPL; ++u) sl.rg[u] = locate_group<EPB>(rr, pr, segments, sl.g0 + u, rows, packed_rows);
        if (NV > 0) {
#pragma unroll
            for (int u = 0; u < GPL; ++u)
#pragma unroll
                for (int k = 0; k < EPB; ++k) {
                    // a row the group does not have reads row 0 instead (never used): loads without branches
                    const float *row = row_at(k < sl.rg[u].count ? sl.rg[u].first + k : 0);
#pragma unroll
                    for (int j = 0; j < KEEP; ++j) {
                        const int v = l + G * j;
                        if (v < nvec) sl.held[u][k][j] = QVec<VEC>::load(row + (size_t)v * VEC);
                    }
                }
        }
    };
    auto process = [&](const Slice &sl) {
        float zp[GPL][EPB], scale[GPL][EPB], inv[GPL][EPB];
#pragma unroll
        for (int u = 0; u < GPL; ++u)
#pragma unroll
            for (int k = 0; k < EPB; ++k) {
                zp[u][k] = 0.0f;
                scale[u][k] = 1.0f;
                inv[u][k] = 1.0f;
                if (k < sl.rg[u].count) {
                    float lo = INFINITY, hi = -INFINITY;
                    if (NV > 0) {
#pragma unroll
                        for (int j = 0; j < KEEP; ++j) {
                            if (l + G * j < nvec) {
#pragma unroll
                                for (int e = 0; e < VEC; ++e) {
                                    lo = fminf(lo, sl.held[u][k][j].get(e));
                                    hi = fmaxf(hi, sl.held[u][k][j].get(e));
                                }
                            }
                        }
                    } else {
                        const float *row = row_at(sl.rg[u].first + k);
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
                    params_of(lo, hi, BITS, zp[u][k], scale[u][k]);
                    inv[u][k] = __builtin_amdgcn_rcpf(scale[u][k]);
                    if (l == 0) {
                        float2 zs = make_float2(zp[u][k], scale[u][k]);
                        if (row_is_bad(sl.rg[u].first + k)) zs = make_float2(NAN, NAN);
                        *reinterpret_cast<float2 *>(params + (size_t)(sl.rg[u].first + k) * 2) = zs;
                    }
                }
            }
#pragma unroll
        for (int u = 0; u < GPL; ++u) {
            if (sl.g0 + u >= packed_rows) continue;
            uint8_t *dst = packed + (size_t)(sl.g0 + u) * (size_t)feat;
            auto pack = [&](int v, int j) {
                uint32_t byte[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) byte[e] = 0;
#pragma unroll
                for (int k = 0; k < EPB; ++k) {
                    if (k < sl.rg[u].count) {
                        QVec<VEC> t;
                        if (NV > 0) t = sl.held[u][k][j];
                        else t = QVec<VEC>::load(row_at(sl.rg[u].first + k) + (size_t)v * VEC);
#pragma unroll
                        for (int e = 0; e < VEC; ++e)
                            byte[e] |= quantize_one_fast(t.get(e), zp[u][k], scale[u][k], inv[u][k])
                                       << ((EPB - k - 1) * BITS);
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
    };

    // Whole lane groups leave together, and no barrier follows the staging above.
    if (kPrefetch) {
        Slice cur, nxt;
        if (slice_start(0) >= packed_rows) return;
        fetch(0, cur);
        for (int it = 0; it < kCodecIters; ++it) {
            const bool more = it + 1 < kCodecIters && slice_start(it + 1) < packed_rows;
            if (more) fetch(it + 1, nxt);
            process(cur);
            if (!more) break;
            cur = nxt;
        }
    } else {
        for (int it = 0; it < kCodecIters; ++it) {
            if (slice_start(it) >= packed_rows) break;
            Slice cur;
            fetch(it, cur);
            process(cur);
        }
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
    constexpr int GPL = kRowsPerLaneGroup / EPB;
    constexpr uint32_t kMask = (1u << BITS) - 1u;
    extern __shared__ int32_t range_lds[];
    const int32_t *rr, *pr;
    stage_ranges(row_range, packed_range, segments, range_lds, rr, pr);

    // a lane group walks kCodecIters slices of the block's share, so that the staging above is paid once
    constexpr int kLaneGroups = 256 / G;
    for (int it = 0; it < kCodecIters; ++it) {
    const int g0 = (int)((((int64_t)blockIdx.x * kCodecIters + it) * kLaneGroups + (int)threadIdx.x / G) * GPL);
    if (g0 >= packed_rows) break;  // whole lane groups leave together; no barrier follows
    const int l = (int)threadIdx.x & (G - 1);
    const int nvec = (feat + VEC - 1) / VEC;
    RowGroup rg[GPL];
    float zp[GPL][EPB], scale[GPL][EPB];
#pragma unroll
    for (int u = 0; u < GPL; ++u) {
        rg[u] = locate_group<EPB>(rr, pr, segments, g0 + u, rows, packed_rows);
#pragma unroll
        for (int k = 0; k < EPB; ++k) {
            zp[u][k] = 0.0f;
            scale[u][k] = 0.0f;
            if (k < rg[u].count) {
                const float2 zs = *reinterpret_cast<const float2 *>(params + (size_t)(rg[u].first + k) * 2);
                zp[u][k] = zs.x;
                scale[u][k] = zs.y;
            }
        }
    }
    for (int v = l; v < nvec; v += G) {
        uint32_t byte[GPL][VEC];
#pragma unroll
        for (int u = 0; u < GPL; ++u)  // (a group past the end reads packed row 0 instead: loads without branches)
            QVec<VEC>::load_bytes(packed + (size_t)(rg[u].count > 0 ? g0 + u : 0) * (size_t)feat + (size_t)v * VEC, byte[u]);
#pragma unroll
        for (int u = 0; u < GPL; ++u)
#pragma unroll
            for (int k = 0; k < EPB; ++k) {
                if (k < rg[u].count) {
                    float o[VEC];
#pragma unroll
                    for (int e = 0; e < VEC; ++e)
                        o[e] = __fmaf_rn((float)((byte[u][e] >> ((EPB - k - 1) * BITS)) & kMask), scale[u][k], zp[u][k]);
                    QVec<VEC>::store(out + (size_t)(rg[u].first + k) * (size_t)feat + (size_t)v * VEC, o);
                }
            }
    }
    }
}

// ---- a product whose result rows leave quantised: packed = quantize(A @ X), segment by segment
//
// The pre-aggregation in front of a quantised exchange (model/layers/aggregator.py:44-49 followed by
// communicator/communicator.py:281-311) as one pass: a lane group owns one packed row at a time, computes the 8/bits
// fp32 rows that share its bytes one after the other -- each row the same single FMA chain over its stored elements,
// in their order, that the product kernels run -- and quantises every finished row out of its registers with the
// functions of the codec above, so parameters and bytes equal those of product-then-quantise while the fp32 rows are
// never written or read back.  Rows are walked in their natural order (the bytes of a packed row belong to
// consecutive rows); LPR lanes x NCH loads x 4 floats cover a row.
template <int BITS, int LPR, int NCH>
__global__ __launch_bounds__(256) void spmm_quantize_segments_kernel(
    const int64_t *__restrict__ rowptr, const int64_t *__restrict__ col, const float *__restrict__ val,
    const float *__restrict__ x, int ldx, uint8_t *__restrict__ packed, float *__restrict__ params,
    const int32_t *__restrict__ row_range, const int32_t *__restrict__ packed_range, int segments, int rows,
    int packed_rows, int feat) {
    constexpr int EPB = 8 / BITS;
    constexpr int GPB = 256 / LPR;
    constexpr int U = NCH == 1 ? 8 : 4;  // gathers in flight per lane group
    extern __shared__ int32_t range_lds[];
    const int32_t *rr, *pr;
    stage_ranges(row_range, packed_range, segments, range_lds, rr, pr);

    const int lig = (int)threadIdx.x & (LPR - 1);
    const int group = (int)threadIdx.x / LPR;
    int foff[NCH];
    bool fok[NCH];
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const int f = (k * LPR + lig) * 4;
        fok[k] = f < feat;
        foff[k] = fok[k] ? f : 0;  // lanes past the row keep a valid address; their values are never used
    }

    // Whole lane groups leave together, and no barrier follows the staging above.
    for (int it = 0; it < kCodecIters; ++it) {
        const int g = (int)(((int64_t)blockIdx.x * kCodecIters + it) * GPB + group);
        if (g >= packed_rows) break;
        const RowGroup rg = locate_group<EPB>(rr, pr, segments, g, rows, packed_rows);
        if (rg.count == 0) continue;
        // the extents of the group's rows: lane k holds rowptr[first + k], k <= count.  The rows are consecutive, so
        // their stored elements are one stretch [begin, end) of the index arrays, walked below as one stream with up
        // to U gathers in flight whatever row they belong to; a row is closed when the stream passes its end.
        const int64_t ext = lig <= rg.count ? rowptr[rg.first + lig] : 0;
        const int64_t begin = __shfl(ext, 0, LPR), end = __shfl(ext, rg.count, LPR);
        uint32_t word[NCH];
        f4 acc[NCH];
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            word[k] = 0;
            acc[k] = f4{0.0f, 0.0f, 0.0f, 0.0f};
        }
        int r = 0;
        int64_t row_end = __shfl(ext, 1, LPR);
        // the finished row r: parameters, then its codes into the bytes it shares
        auto close_row = [&]() {
            float lo = INFINITY, hi = -INFINITY;
#pragma unroll
            for (int k = 0; k < NCH; ++k) {
                if (fok[k]) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        lo = fminf(lo, acc[k][e]);
                        hi = fmaxf(hi, acc[k][e]);
                    }
                }
            }
            group_min_max<LPR>(lo, hi);
            float zp, scale;
            params_of(lo, hi, BITS, zp, scale);
            const float inv = __builtin_amdgcn_rcpf(scale);
            if (lig == 0) *reinterpret_cast<float2 *>(params + (size_t)(rg.first + r) * 2) = make_float2(zp, scale);
#pragma unroll
            for (int k = 0; k < NCH; ++k) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    word[k] |= ((quantize_one_fast(acc[k][e], zp, scale, inv) << ((EPB - r - 1) * BITS)) & 0xFFu) << (8 * e);
                acc[k] = f4{0.0f, 0.0f, 0.0f, 0.0f};
            }
            ++r;
            row_end = __shfl(ext, r + 1 <= rg.count ? r + 1 : rg.count, LPR);
        };
        for (int64_t e0 = begin; e0 < end; e0 += LPR) {
            const int n = (int)(end - e0 < LPR ? end - e0 : LPR);
            // one coalesced fetch of up to LPR (column, value) pairs, handed round below
            const int64_t c_mine = lig < n ? col[e0 + lig] : 0;
            const float v_mine = lig < n ? val[e0 + lig] : 0.0f;
            for (int j0 = 0; j0 < n; j0 += U) {
                f4 xv[U][NCH];
                float vv[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    // a surplus gather reads row 0 (a valid address); its result never enters a chain
                    const int64_t cc = j0 + u < n ? __shfl(c_mine, j0 + u, LPR) : 0;
                    vv[u] = __shfl(v_mine, j0 + u < n ? j0 + u : 0, LPR);
                    const float *xr = x + (size_t)cc * (size_t)ldx;
#pragma unroll
                    for (int k = 0; k < NCH; ++k) xv[u][k] = *reinterpret_cast<const f4 *>(xr + foff[k]);
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (j0 + u < n) {
                        if constexpr (EPB > 1) {
                            while (e0 + j0 + u >= row_end) close_row();  // (rows without elements close at once)
                        }
#pragma unroll
                        for (int k = 0; k < NCH; ++k) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[k][e] = __builtin_fmaf(vv[u], xv[u][k][e], acc[k][e]);
                        }
                    }
                }
            }
        }
        while (r < rg.count) close_row();
#pragma unroll
        for (int k = 0; k < NCH; ++k)
            if (fok[k]) *reinterpret_cast<uint32_t *>(packed + (size_t)g * (size_t)feat + foff[k]) = word[k];
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
    const int64_t *index = nullptr;  // quantise: fp32 row r is row index[r] of the source (a gather folded in)
    int64_t src_rows = 0;
};

// packed rows handled by one lane group
constexpr int groups_per_lane_group(int bits) { return kRowsPerLaneGroup / (8 / bits); }

size_t range_lds_bytes(int segments) {
    return segments <= kMaxLdsSegments ? 2 * (size_t)(segments + 1) * sizeof(int32_t) : 0;
}

template <int BITS, int VEC, int G>
void launch_quantize(const float *x, uint8_t *packed, float *params, const SegArgs &a) {
    const int nvec = (a.feat + VEC - 1) / VEC;
    constexpr int gpl = groups_per_lane_group(BITS);
    const unsigned blocks = grid_for(((int64_t)a.packed_rows + gpl - 1) / gpl * G, 256 * kCodecIters);
    const size_t lds = range_lds_bytes(a.segments);
    if (nvec <= G)
        hipLaunchKernelGGL((quantize_segments_kernel<BITS, VEC, G, 1>), dim3(blocks), dim3(256), lds, a.st, x, packed,
                           params, a.row_range, a.packed_range, a.segments, a.rows, a.packed_rows, a.feat, a.index,
                           a.src_rows);
    else if (nvec <= 4 * G)
        hipLaunchKernelGGL((quantize_segments_kernel<BITS, VEC, G, 4>), dim3(blocks), dim3(256), lds, a.st, x, packed,
                           params, a.row_range, a.packed_range, a.segments, a.rows, a.packed_rows, a.feat, a.index,
                           a.src_rows);
    else
        hipLaunchKernelGGL((quantize_segments_kernel<BITS, VEC, G, 0>), dim3(blocks), dim3(256), lds, a.st, x, packed,
                           params, a.row_range, a.packed_range, a.segments, a.rows, a.packed_rows, a.feat, a.index,
                           a.src_rows);
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
    constexpr int gpl = groups_per_lane_group(BITS);
    const int64_t lane_groups = ((int64_t)a.packed_rows + gpl - 1) / gpl;
    const size_t lds = range_lds_bytes(a.segments);
#define GNNAGG_DEQ(G)                                                                                            \
    hipLaunchKernelGGL((dequantize_segments_kernel<BITS, VEC, G>),                                               \
                       dim3(grid_for(lane_groups * G, 256 * kCodecIters)), dim3(256), lds, a.st, packed, params, \
                       out, a.row_range, a.packed_range, a.segments, a.rows, a.packed_rows, a.feat)
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


// ---- bf16 rows on the wire (communicator.py:111-137: send_buf_fp16.copy_(send_buf), the exchange,
// recv_buf.copy_(recv_buf_fp16)): round to nearest even, NaN -> 0x7FC0, as the tensor copy does.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned short u16x4_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void f32_to_bf16_kernel(const float *__restrict__ x, unsigned short *__restrict__ y,
                                                          int64_t count, int vec) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t n4 = vec ? count / 4 : 0;
    for (int64_t i = tid; i < n4; i += stride) {
        const f32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(x) + i);
        u16x4_t r;
        r.x = bf16_bits(v.x);
        r.y = bf16_bits(v.y);
        r.z = bf16_bits(v.z);
        r.w = bf16_bits(v.w);
        __builtin_nontemporal_store(r, reinterpret_cast<u16x4_t *>(y) + i);
    }
    for (int64_t i = n4 * 4 + tid; i < count; i += stride) y[i] = bf16_bits(x[i]);
}

__global__ __launch_bounds__(256) void bf16_to_f32_kernel(const unsigned short *__restrict__ x, float *__restrict__ y,
                                                          int64_t count, int vec) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t n4 = vec ? count / 4 : 0;
    for (int64_t i = tid; i < n4; i += stride) {
        const u16x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u16x4_t *>(x) + i);
        f32x4_t r;
        r.x = __uint_as_float((uint32_t)v.x << 16);
        r.y = __uint_as_float((uint32_t)v.y << 16);
        r.z = __uint_as_float((uint32_t)v.z << 16);
        r.w = __uint_as_float((uint32_t)v.w << 16);
        __builtin_nontemporal_store(r, reinterpret_cast<f32x4_t *>(y) + i);
    }
    for (int64_t i = n4 * 4 + tid; i < count; i += stride) y[i] = __uint_as_float((uint32_t)x[i] << 16);
}

unsigned stream_blocks(int64_t items) {
    const int64_t blocks = (items + 255) / 256;
    return (unsigned)(blocks < 256 * 64 ? (blocks > 0 ? blocks : 1) : 256 * 64);
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

extern "C" int gnnagg_gather_quantize_segments_f32(const float *src, int64_t src_rows, const int64_t *index,
                                                   uint8_t *packed, float *params, const int32_t *row_range,
                                                   const int32_t *packed_range, int64_t segments, int64_t rows,
                                                   int64_t packed_rows, int64_t feat, int bits, void *stream) {
    const int rc = check_segments(src, packed, params, row_range, packed_range, segments, rows, packed_rows, feat, bits);
    if (rc != GNNAGG_OK || rows == 0 || feat == 0) return rc;
    GNNAGG_REQUIRE(index, "null index");
    GNNAGG_REQUIRE(src_rows > 0, "rows are asked of a source without rows");
    SegArgs a{row_range, packed_range, (int)segments, (int)rows, (int)packed_rows, (int)feat,
              static_cast<hipStream_t>(stream)};
    a.index = index;
    a.src_rows = src_rows;
    const bool v4 = feat % 4 == 0 && aligned16(src) && aligned4(packed);
#define GNNAGG_Q(B)                                                      \
    if (bits == B) {                                                     \
        if (v4) launch_quantize_g<B, 4>(src, packed, params, a);         \
        else launch_quantize_g<B, 1>(src, packed, params, a);            \
    }
    GNNAGG_Q(2) GNNAGG_Q(4) GNNAGG_Q(8)
#undef GNNAGG_Q
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

extern "C" int gnnagg_spmm_csr_quantize_segments_f32(const int64_t *rowptr, const int64_t *col, const float *value,
                                                     const float *mat, int64_t mat_stride, uint8_t *packed,
                                                     float *params, const int32_t *row_range,
                                                     const int32_t *packed_range, int64_t segments, int64_t rows,
                                                     int64_t packed_rows, int64_t feat, int bits, void *stream) {
    const int rc = check_segments(mat, packed, params, row_range, packed_range, segments, rows, packed_rows, feat, bits);
    if (rc != GNNAGG_OK || rows == 0 || feat == 0) return rc;
    GNNAGG_REQUIRE(rowptr && col && value, "null rowptr/col/value");
    GNNAGG_REQUIRE(mat_stride >= feat && mat_stride < (int64_t(1) << 31), "row stride %lld must be at least the width %lld "
                   "and below 2^31", (long long)mat_stride, (long long)feat);
    if (feat % 4 != 0 || feat > 512 || mat_stride % 4 != 0 || !aligned16(mat) || !aligned4(packed))
        return fail(GNNAGG_ERR_UNSUPPORTED, "the product with quantised result rows takes widths that are multiples of 4 "
                    "up to 512 (got %lld), rows of the dense operand on 16-byte boundaries and a 4-byte aligned result",
                    (long long)feat);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t lds = range_lds_bytes((int)segments);
    const int nvec = (int)(feat / 4);
#define GNNAGG_PQ(B, LPR, NCH)                                                                                       \
    hipLaunchKernelGGL((spmm_quantize_segments_kernel<B, LPR, NCH>),                                                 \
                       dim3(grid_for(packed_rows, (256 / LPR) * kCodecIters)), dim3(256), lds, st, rowptr, col, value, \
                       mat, (int)mat_stride, packed, params, row_range, packed_range, (int)segments, (int)rows,      \
                       (int)packed_rows, (int)feat)
#define GNNAGG_PQ_BITS(B)                             \
    if (bits == B) {                                  \
        if (nvec <= 16) GNNAGG_PQ(B, 16, 1);          \
        else if (nvec <= 32) GNNAGG_PQ(B, 32, 1);     \
        else if (nvec <= 64) GNNAGG_PQ(B, 64, 1);     \
        else GNNAGG_PQ(B, 64, 2);                     \
    }
    GNNAGG_PQ_BITS(2) GNNAGG_PQ_BITS(4) GNNAGG_PQ_BITS(8)
#undef GNNAGG_PQ_BITS
#undef GNNAGG_PQ
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

extern "C" int gnnagg_f32_to_bf16(const float *x, uint16_t *y, int64_t count, void *stream) {
    GNNAGG_REQUIRE(count >= 0, "negative size");
    if (count == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(x && y, "null x / y");
    const int vec = (reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 8 == 0) ? 1 : 0;
    hipLaunchKernelGGL(f32_to_bf16_kernel, dim3(stream_blocks(vec ? count / 4 + 3 : count)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), x, y, count, vec);
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

extern "C" int gnnagg_bf16_to_f32(const uint16_t *x, float *y, int64_t count, void *stream) {
    GNNAGG_REQUIRE(count >= 0, "negative size");
    if (count == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(x && y, "null x / y");
    const int vec = (reinterpret_cast<uintptr_t>(x) % 8 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0) ? 1 : 0;
    hipLaunchKernelGGL(bf16_to_f32_kernel, dim3(stream_blocks(vec ? count / 4 + 3 : count)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), x, y, count, vec);
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}
