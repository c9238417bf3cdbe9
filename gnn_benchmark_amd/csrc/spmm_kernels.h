// Device kernels of the CSR SpMM (out (+)= A @ X, fp32) for gfx950.
//
// Work decomposition.  A "task" is one sparse row.  A wavefront (64 lanes) is cut into
// groups of LPR lanes; one group owns one task at a time.  Inside a group the lanes lie ALONG THE FEATURE DIMENSION: lane l
// holds features [(k*LPR + l)*VEC, +VEC) for k < NCH, so every gather of a dense row
// X[col,:] is one contiguous, fully coalesced run of LPR*VEC*4 bytes per k.
//
// Column indices / values of a task are fetched LPR at a time by the group's lanes
// (one coalesced, non-temporal load each), then handed round lane by lane:
// v_readlane for a whole-wave group (the index lands in a scalar register and the
// row address is scalar+lane), ds_bpermute for sub-wavefront groups.  UNROLL gathers
// are issued back to back before their FMAs so that each group keeps UNROLL*NCH
// vector loads in flight -- the kernel is bound by HBM latency/bandwidth, not issue.
//
// Arithmetic.  EVERY row, whatever its length, is one fp32 FMA chain in CSR order
// starting from the value in `out` (or 0), i.e. the recurrence of the reference's
// kernel_1xN (self_benchmark/a64fx/model/ops/src/spmm.cpp:37-53): results are
// bit-identical to the reference's CPU operator.  Long rows are therefore not split over
// their stored elements; the plan schedules them first, one lane group each, and the
// short rows fill in behind them.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.h"

namespace gnnagg {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int VEC>
struct FVec;

template <>
struct FVec<1> {
    float d;
    __device__ __forceinline__ static FVec zero() { return FVec{0.0f}; }
    __device__ __forceinline__ static FVec load(const float *p) { return FVec{*p}; }
    __device__ __forceinline__ void store(float *p) const { *p = d; }
    __device__ __forceinline__ static FVec load_stream(const float *p) { return FVec{__builtin_nontemporal_load(p)}; }
    __device__ __forceinline__ void store_stream(float *p) const { __builtin_nontemporal_store(d, p); }
    __device__ __forceinline__ void fma(float a, const FVec &x) { d = __builtin_fmaf(a, x.d, d); }
    __device__ __forceinline__ void add(const FVec &x) { d += x.d; }
    __device__ __forceinline__ float at(int) const { return d; }
};

template <>
struct FVec<2> {
    f32x2 d;
    __device__ __forceinline__ static FVec zero() { return FVec{f32x2{0.0f, 0.0f}}; }
    __device__ __forceinline__ static FVec load(const float *p) {
        return FVec{*reinterpret_cast<const f32x2 *>(p)};
    }
    __device__ __forceinline__ void store(float *p) const { *reinterpret_cast<f32x2 *>(p) = d; }
    __device__ __forceinline__ static FVec load_stream(const float *p) {
        return FVec{__builtin_nontemporal_load(reinterpret_cast<const f32x2 *>(p))};
    }
    __device__ __forceinline__ void store_stream(float *p) const {
        __builtin_nontemporal_store(d, reinterpret_cast<f32x2 *>(p));
    }
    __device__ __forceinline__ void fma(float a, const FVec &x) {
        d.x = __builtin_fmaf(a, x.d.x, d.x);
        d.y = __builtin_fmaf(a, x.d.y, d.y);
    }
    __device__ __forceinline__ void add(const FVec &x) {
        d.x += x.d.x;
        d.y += x.d.y;
    }
    __device__ __forceinline__ float at(int i) const { return d[i]; }
};

template <>
struct FVec<4> {
    f32x4 d;
    __device__ __forceinline__ static FVec zero() { return FVec{f32x4{0.0f, 0.0f, 0.0f, 0.0f}}; }
    __device__ __forceinline__ static FVec load(const float *p) {
        return FVec{*reinterpret_cast<const f32x4 *>(p)};
    }
    __device__ __forceinline__ void store(float *p) const { *reinterpret_cast<f32x4 *>(p) = d; }
    __device__ __forceinline__ static FVec load_stream(const float *p) {
        return FVec{__builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p))};
    }
    __device__ __forceinline__ void store_stream(float *p) const {
        __builtin_nontemporal_store(d, reinterpret_cast<f32x4 *>(p));
    }
    __device__ __forceinline__ void fma(float a, const FVec &x) {
        d.x = __builtin_fmaf(a, x.d.x, d.x);
        d.y = __builtin_fmaf(a, x.d.y, d.y);
        d.z = __builtin_fmaf(a, x.d.z, d.z);
        d.w = __builtin_fmaf(a, x.d.w, d.w);
    }
    __device__ __forceinline__ void add(const FVec &x) {
        d.x += x.d.x;
        d.y += x.d.y;
        d.z += x.d.z;
        d.w += x.d.w;
    }
    __device__ __forceinline__ float at(int i) const { return d[i]; }
};

// Lane-to-lane hand-over of a 32-bit word inside a group of LPR lanes.  For LPR == 64
// the source lane index must be wave-uniform.
template <int LPR>
__device__ __forceinline__ int group_bcast(int v, int src) {
    if constexpr (LPR == 64) {
        return __builtin_amdgcn_readlane(v, src);
    } else {
        const int self = (int)__lane_id();
        const int idx = (self & ~(LPR - 1)) | (src & (LPR - 1));
        return __builtin_amdgcn_ds_bpermute(idx << 2, v);
    }
}

template <int LPR>
__device__ __forceinline__ int64_t group_bcast_idx(int64_t v, int src) {
    const int lo = group_bcast<LPR>((int)(uint32_t)(v & 0xffffffffll), src);
    const int hi = group_bcast<LPR>((int)(v >> 32), src);
    return ((int64_t)hi << 32) | (uint32_t)lo;
}
template <int LPR>
__device__ __forceinline__ int64_t group_bcast_idx(int32_t v, int src) {
    return (int64_t)group_bcast<LPR>(v, src);
}

// Which lanes of the group hold `p` (bit i: the group's lane i); wave-uniform for a whole-wave group.
template <int LPR>
__device__ __forceinline__ uint64_t group_ballot(bool p) {
    const uint64_t b = __builtin_amdgcn_ballot_w64(p);
    if constexpr (LPR == 64) {
        return b;
    } else {
        const int first = (int)__lane_id() & ~(LPR - 1);
        return (b >> first) & ((uint64_t(1) << LPR) - 1);
    }
}

__device__ __forceinline__ int64_t uniform_i64(int64_t v) {
    const int lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)(v & 0xffffffffll));
    const int hi = __builtin_amdgcn_readfirstlane((int)(v >> 32));
    return ((int64_t)hi << 32) | (uint32_t)lo;
}

enum TaskMode : int {
    kRowsNatural = 0,  // task t is row t, described by rowptr        (plan-less entry point)
    kRowsPlanned = 1   // task t is described by task[t] of a plan    (degree-ordered)
};

// One row of a plan's schedule: 16 bytes, fetched with a single load.
struct __attribute__((aligned(16))) RowTask {
    int64_t start;  // first stored element
    int32_t len;    // stored elements
    int32_t row;    // output row
};

struct SpmmArgs {
    const int64_t *rowptr;    // [rows+1]                       (kRowsNatural)
    const RowTask *task;      // [ntasks]                       (kRowsPlanned)
    const void *col;          // IdxT [nnz]
    const float *val;         // [nnz]
    const float *x;           // dense operand [K, F] (packed source: non-zero values at the front of each row)
    // two dense sources (kSrcDense2): columns [0, x_rows) are rows of x, columns x_rows + k are rows k of x2
    const float *x2;
    int x_rows, ldx2;         // ldx2: row stride of x2 in floats; 0 stands for F
    // a dense fp32 source followed by a second source in its exchange format (kSrcDenseThenBf16: x2 points at bf16
    // rows, ldx2 counts 16-bit values; kSrcDenseThenQuant: qdata / qparams / qcode): the first split[row] stored
    // elements of a row read x, the rest read row (column - x_rows) of the second source
    const int32_t *split;     // [rows]
    const uint32_t *hdr;      // packed source only: [K, hdr_words] row headers
    int hdr_words;
    // quantised source only (row-packed codec of the boundary buffers): byte rows [packed_rows, F] in
    // which 8/qbits rows share a byte per column, (zero_point, scale) per row, and per row the code
    // packed_row * 8 + (position inside its byte group)
    const uint8_t *qdata;
    const float *qparams;     // [K, 2]
    const int32_t *qcode;     // [K]
    int qbits;
    float *dst;               // out [rows, F]
    int64_t ntasks;
    int feat;                 // F
    int ldx, ldd;             // row strides of x and dst in floats; 0 stands for F (rows back to back)
    int f_base;               // first feature handled by this launch
    int accumulate;           // start every row from dst (1) or from 0 (0)
    int dst_bf16;             // 1: dst points at bf16 rows (ldd counts 16-bit values), rounded on the way out;
                              // overwriting launches with 16-byte vector lanes only
    int tasks_per_block;      // tasks handled by one block of the middle region
    int64_t head_tasks;       // the first head_tasks tasks (the longest rows) get one lane group each
    int head_blocks;          // = ceil(head_tasks / groups per block)
    // The tasks from tail_first on (the shortest rows: a plan orders its rows by length) are handed out
    // tail_tasks_per_block to a block, more rows per lane group than in the middle region: what a group pays once
    // per block (row descriptors, the first column chunk: two dependent round trips) is spread over more rows.
    int64_t tail_first;       // first task of the tail region (== ntasks: none)
    int mid_blocks;           // blocks of the middle region
    int tail_tasks_per_block;
    // kRowsNatural only (no plan to order the rows by length): with long_len > 0 the first scan_blocks blocks walk
    // rowptr, scan_rows rows per lane group, and run the rows of more than long_len elements they meet -- the longest
    // chains start with the launch, spread over the whole device; the blocks behind them leave those rows out.
    int long_len;
    int scan_blocks;
    int scan_rows;
};

enum SourceKind : int {
    kSrcDense = 0,   // x[col, :] is a dense fp32 row
    kSrcPacked = 1,  // x[col, :] holds the row's non-zero values at its front, hdr[col, :] says which
    kSrcQuant = 2,   // row col is held quantised: qdata / qparams / qcode (boundary-buffer codec layout)
    kSrcBf16 = 3,    // x[col, :] is a bf16 row (x points at 16-bit values, ldx counts them): widened in the gather
    kSrcDense2 = 4,  // dense fp32 rows of two arrays: x[col, :] for col < x_rows, x2[col - x_rows, :] above
    // the first split[row] elements of a row gather dense fp32 rows of x, the others rows of a second source:
    kSrcDenseThenBf16 = 5,   // ... bf16 rows (x2)
    kSrcDenseThenQuant = 6   // ... quantised rows (qdata / qparams / qcode)
};

typedef float f32x4_unaligned __attribute__((ext_vector_type(4), aligned(4)));

// One lane's four features (f .. f+3, f a multiple of 4) of a packed row: `h` is the row's
// header -- for every 32 features a (bitmap, non-zeros in front) pair of words -- fetched with
// one 8-byte load; `position` then says where in the row the lane's first non-zero value sits.
struct PackedLane {
    uint32_t word, before;
    __device__ __forceinline__ void request(const uint32_t *__restrict__ h, int f) {
        const uint2 pair = *reinterpret_cast<const uint2 *>(h + 2 * (f >> 5));
        word = pair.x;
        before = pair.y;
    }
    __device__ __forceinline__ uint32_t nibble(int f) const { return (word >> (f & 31)) & 15u; }
    __device__ __forceinline__ int position(int f) const {
        return (int)before + __popc(word & ((1u << (f & 31)) - 1u));
    }
};

__device__ __forceinline__ FVec<4> expand_packed(uint32_t nib, const f32x4_unaligned v) {
    // value e sits at rank popc(nib & ((1 << e) - 1)) among the up to four loaded ones
    FVec<4> r;
    const float a0 = v.x, a1 = v.y, a2 = v.z, a3 = v.w;
    r.d.x = (nib & 1u) ? a0 : 0.0f;
    const float s1 = (nib & 1u) ? a1 : a0;
    r.d.y = (nib & 2u) ? s1 : 0.0f;
    const int r2 = __popc(nib & 3u);
    const float s2 = r2 == 0 ? a0 : (r2 == 1 ? a1 : a2);
    r.d.z = (nib & 4u) ? s2 : 0.0f;
    const int r3 = __popc(nib & 7u);
    const float s3 = r3 == 0 ? a0 : (r3 == 1 ? a1 : (r3 == 2 ? a2 : a3));
    r.d.w = (nib & 8u) ? s3 : 0.0f;
    return r;
}

// UU gathers issued back to back, then their FMAs in CSR order: elements j .. j+UU-1 of
// the chunk held in (c_l, v_l) across the group's lanes.  For a packed source the zero
// values are not fetched; fma(v, 0, acc) == acc, so the chain is the same (up to the sign
// of a zero result).
// `valid` < UU (the tail of a row's last chunk): all UU gathers are still issued at once -- one memory round trip
// instead of a cascade of ever shorter dependent ones; the lanes past the row's end hold column 0 with value 0, so the
// surplus gathers read row 0 of x (a valid, hot address) -- and only the first `valid` results enter the chain (selected,
// not multiplied by zero: row 0 of x may hold anything).
// SECOND: the elements belong to the second source of a two-format launch (x2 / ldx2, or the quantised buffers):
// their column counts from x_rows.  CLAMP: the surplus gathers of a TAIL round must not use what the lanes behind the
// stretch hold (elements of the other source, whose columns mean something else): they read row 0.
template <int UU, int VEC, int LPR, int NCH, int SRC, typename IdxT, bool TAIL = false, bool SECOND = false, bool CLAMP = false>
__device__ __forceinline__ void gather_fma(FVec<VEC> (&acc)[NCH], IdxT c_l, float v_l, int j, const SpmmArgs &a,
                                           const int (&foff)[NCH], int valid = UU) {
    const float *__restrict__ x = SECOND ? a.x2 : a.x;
    const int F = a.feat;
    const int ldx = SECOND ? (a.ldx2 ? a.ldx2 : F) : (a.ldx ? a.ldx : F);
    const float *xr[UU];
    float vv[UU];
    int64_t cc[UU];
#pragma unroll
    for (int u = 0; u < UU; ++u) {
        cc[u] = group_bcast_idx<LPR>(c_l, j + u);
        if constexpr (SECOND) cc[u] -= (int64_t)a.x_rows;
        if constexpr (TAIL && CLAMP) {
            if (u >= valid) cc[u] = 0;
        }
        vv[u] = __int_as_float(group_bcast<LPR>(__float_as_int(v_l), j + u));
        if constexpr (SRC == kSrcDense2) {
            const bool second = cc[u] >= (int64_t)a.x_rows;
            const float *__restrict__ from = second ? a.x2 : x;
            const int64_t r = second ? cc[u] - (int64_t)a.x_rows : cc[u];
            const int ld = second ? (a.ldx2 ? a.ldx2 : F) : ldx;
            xr[u] = from + (size_t)r * (size_t)ld;
        } else {
            xr[u] = x + (size_t)cc[u] * (size_t)ldx;
        }
    }
    FVec<VEC> xv[UU][NCH];
    if constexpr (SRC == kSrcPacked) {
        static_assert(SRC == kSrcDense || (VEC == 4 && NCH == 1), "packed rows: 16-byte lanes, one load per lane");
        const int f = foff[0];
        PackedLane pl[UU];
#pragma unroll
        for (int u = 0; u < UU; ++u) pl[u].request(a.hdr + (size_t)cc[u] * (size_t)a.hdr_words, f);
        f32x4_unaligned raw[UU];
        uint32_t nib[UU];
#pragma unroll
        for (int u = 0; u < UU; ++u) {
            nib[u] = pl[u].nibble(f);
            // a lane with nothing to fetch reads the front of the row: a valid, hot address
            const float *src = xr[u] + (nib[u] ? pl[u].position(f) : 0);
            raw[u] = *reinterpret_cast<const f32x4_unaligned *>(src);
        }
#pragma unroll
        for (int u = 0; u < UU; ++u) xv[u][0] = expand_packed(nib[u], raw[u]);
    } else if constexpr (SRC == kSrcQuant) {
        static_assert(SRC != kSrcQuant || VEC == 4, "quantised rows: four bytes per lane and load");
        // x' = fma(q, scale, zero_point): the dequantisation of the codec, done on the gathered bytes
        const int per_byte = 8 / a.qbits;
        const uint32_t mask = (1u << a.qbits) - 1u;
        uint32_t raw[UU][NCH];
        float zp[UU], sc[UU];
        int shift[UU];
        int code[UU];
        if constexpr (sizeof(IdxT) == 8) {
            // 64-bit index elements carry the row code next to the column (code << 32 | column): translated once per
            // matrix, so that the bytes can be asked for as soon as the index chunk has arrived
#pragma unroll
            for (int u = 0; u < UU; ++u) {
                code[u] = (int)(cc[u] >> 32);
                cc[u] &= 0xffffffffll;
            }
        } else {
#pragma unroll
            for (int u = 0; u < UU; ++u) code[u] = a.qcode[cc[u]];
        }
#pragma unroll
        for (int u = 0; u < UU; ++u) {
            const float2 p = *reinterpret_cast<const float2 *>(a.qparams + 2 * (size_t)cc[u]);
            zp[u] = p.x;
            sc[u] = p.y;
        }
#pragma unroll
        for (int u = 0; u < UU; ++u) {
            const uint8_t *qrow = a.qdata + (size_t)(code[u] >> 3) * (size_t)F;
            shift[u] = (per_byte - (code[u] & 7) - 1) * a.qbits;
#pragma unroll
            for (int k = 0; k < NCH; ++k) raw[u][k] = *reinterpret_cast<const uint32_t *>(qrow + foff[k]);
        }
#pragma unroll
        for (int u = 0; u < UU; ++u) {
#pragma unroll
            for (int k = 0; k < NCH; ++k) {
                const uint32_t w = raw[u][k] >> shift[u];
                xv[u][k].d.x = __builtin_fmaf((float)(w & mask), sc[u], zp[u]);
                xv[u][k].d.y = __builtin_fmaf((float)((w >> 8) & mask), sc[u], zp[u]);
                xv[u][k].d.z = __builtin_fmaf((float)((w >> 16) & mask), sc[u], zp[u]);
                xv[u][k].d.w = __builtin_fmaf((float)((w >> 24) & mask), sc[u], zp[u]);
            }
        }
    } else if constexpr (SRC == kSrcBf16) {
        static_assert(SRC != kSrcBf16 || VEC == 4, "bf16 rows: four values (8 bytes) per lane and load");
        // a bf16 value is the upper half of the fp32 value it stands for: widening is exact
        const unsigned short *xb = reinterpret_cast<const unsigned short *>(x);
        uint2 raw[UU][NCH];
#pragma unroll
        for (int u = 0; u < UU; ++u) {
#pragma unroll
            for (int k = 0; k < NCH; ++k)
                raw[u][k] = *reinterpret_cast<const uint2 *>(xb + (size_t)cc[u] * (size_t)ldx + foff[k]);
        }
#pragma unroll
        for (int u = 0; u < UU; ++u) {
#pragma unroll
            for (int k = 0; k < NCH; ++k) {
                xv[u][k].d.x = __uint_as_float(raw[u][k].x << 16);
                xv[u][k].d.y = __uint_as_float(raw[u][k].x & 0xffff0000u);
                xv[u][k].d.z = __uint_as_float(raw[u][k].y << 16);
                xv[u][k].d.w = __uint_as_float(raw[u][k].y & 0xffff0000u);
            }
        }
    } else {
#pragma unroll
        for (int u = 0; u < UU; ++u) {
#pragma unroll
            for (int k = 0; k < NCH; ++k) xv[u][k] = FVec<VEC>::load(xr[u] + foff[k]);
        }
    }
#pragma unroll
    for (int u = 0; u < UU; ++u) {
        if constexpr (TAIL) {
            if (u < valid) {
#pragma unroll
                for (int k = 0; k < NCH; ++k) acc[k].fma(vv[u], xv[u][k]);
            }
        } else {
#pragma unroll
            for (int k = 0; k < NCH; ++k) acc[k].fma(vv[u], xv[u][k]);
        }
    }
}

// Gathers kept in flight per lane group, sized so that a wave stays near 64-90 VGPRs:
// measured on MI355X, deeper unrolls (fewer waves per SIMD) bring nothing -- the
// kernel already saturates the memory system.
template <int VEC, int NCH>
struct UnrollFor {
    static constexpr int regs = VEC * NCH;  // VGPRs per gathered row per lane
    static constexpr int raw = 32 / regs;
    static constexpr int value = raw >= 8 ? 8 : (raw >= 4 ? 4 : (raw >= 2 ? 2 : 1));
};

constexpr int kMaxRowsPerGroup = 16;  // a group's task descriptors live one per lane

// Elements [j0, j1) of the chunk held in (c_l, v_l): full blocks of U gathers, then ONE more round for what is left
// (the smallest power of two of gathers that covers it, the surplus ones masked): ceil((j1 - j0) / U) dependent
// round trips.
template <int VEC, int LPR, int NCH, int SRC, typename IdxT, bool SECOND = false, bool CLAMP = false>
__device__ __forceinline__ void gather_rounds(FVec<VEC> (&acc)[NCH], IdxT c_l, float v_l, int j0, int j1,
                                              const SpmmArgs &a, const int (&foff)[NCH]) {
    constexpr int U = UnrollFor<VEC, NCH>::value;
    int j = j0;
    for (; j + U <= j1; j += U) gather_fma<U, VEC, LPR, NCH, SRC, IdxT, false, SECOND, CLAMP>(acc, c_l, v_l, j, a, foff);
    const int rem = j1 - j;
    if (rem > 0) {
        if constexpr (U > 4) {
            if (rem > 4) gather_fma<8, VEC, LPR, NCH, SRC, IdxT, true, SECOND, CLAMP>(acc, c_l, v_l, j, a, foff, rem);
        }
        if constexpr (U > 2) {
            if (rem > 2 && rem <= 4) gather_fma<4, VEC, LPR, NCH, SRC, IdxT, true, SECOND, CLAMP>(acc, c_l, v_l, j, a, foff, rem);
        }
        if constexpr (U > 1) {
            if (rem == 2) gather_fma<2, VEC, LPR, NCH, SRC, IdxT, false, SECOND, CLAMP>(acc, c_l, v_l, j, a, foff);
        }
        if (rem == 1) gather_fma<1, VEC, LPR, NCH, SRC, IdxT, false, SECOND, CLAMP>(acc, c_l, v_l, j, a, foff);
    }
}

template <int VEC, int LPR, int NCH, typename IdxT, int MODE, int SRC = kSrcDense>
__global__ __launch_bounds__(256) void spmm_tasks_kernel(const SpmmArgs a) {
    constexpr int GPB = 256 / LPR;  // groups per 256-thread block
    typedef FVec<VEC> V;

    const int lane = (int)threadIdx.x & 63;
    const int lig = lane & (LPR - 1);  // lane in group
    int group = (int)threadIdx.x / LPR;
    if constexpr (LPR == 64) group = __builtin_amdgcn_readfirstlane(group);

    const IdxT *__restrict__ col = static_cast<const IdxT *>(a.col);
    const float *__restrict__ val = a.val;
    const int F = a.feat;

    // Lanes past the end of the feature row keep a valid address (the first feature of
    // this launch) so that gathers need no predication; only their loads of / stores to
    // `dst` are masked.  The host guarantees f_base < F and F % VEC == 0.
    int foff[NCH];
    bool fok[NCH];
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const int f = a.f_base + (k * LPR + lig) * VEC;
        fok[k] = f < F;
        foff[k] = fok[k] ? f : a.f_base;
    }

    // Rows without a plan: a scanner block's groups walk their stretch of rowptr for the long rows, LPR rows at a
    // time; the other blocks take the remaining rows in their natural order.
    bool scanner = false;
    int64_t scan_next = 0, scan_end = 0;
    int bid = (int)blockIdx.x;
    if constexpr (MODE == kRowsNatural) {
        scanner = bid < a.scan_blocks;
        if (scanner) {
            scan_next = ((int64_t)bid * GPB + group) * (int64_t)a.scan_rows;
            scan_end = scan_next + a.scan_rows;
            if (scan_end > a.ntasks) scan_end = a.ntasks;
            if (scan_next >= scan_end) return;
        }
        bid -= a.scan_blocks;
    }

    // Head region: one task per lane group, so that no group queues several of the
    // longest rows behind each other.  Blocks are dispatched in index order, hence the
    // longest rows start first and the short ones fill in behind them.
    int64_t t0 = 0, t1 = 0;
    if (!scanner) {
        if (bid < a.head_blocks) {
            t0 = (int64_t)bid * GPB;
            t1 = t0 + GPB;
            if (t1 > a.head_tasks) t1 = a.head_tasks;
        } else if (bid < a.head_blocks + a.mid_blocks) {
            t0 = a.head_tasks + (int64_t)(bid - a.head_blocks) * a.tasks_per_block;
            t1 = t0 + a.tasks_per_block;
            if (t1 > a.tail_first) t1 = a.tail_first;
        } else {
            t0 = a.tail_first + (int64_t)(bid - a.head_blocks - a.mid_blocks) * a.tail_tasks_per_block;
            t1 = t0 + a.tail_tasks_per_block;
            if (t1 > a.ntasks) t1 = a.ntasks;
        }
    }
    // this group's tasks: t0 + group + i * GPB, i < ntask  (ntask <= kMaxRowsPerGroup <= LPR)
    const int64_t tfirst = t0 + group;
    if (!scanner && tfirst >= t1) return;
    int ntask = scanner ? 0 : (int)((t1 - tfirst + GPB - 1) / GPB);
    if constexpr (LPR == 64) ntask = __builtin_amdgcn_readfirstlane(ntask);

    // One coalesced fetch brings every descriptor of the group: lane i holds task i.
    int d_row = 0, d_len = 0;
    int64_t d_start = 0;
    int d_split = 0;  // two-format launches: the row's leading elements that read the dense source
    // kRowsNatural: the group's lanes whose row is still to be done (a planned launch walks lanes 0 .. ntask-1)
    uint64_t todo = 0;
    if (!scanner && lig < ntask) {
        const int64_t t = tfirst + (int64_t)lig * GPB;
        if constexpr (MODE == kRowsPlanned) {
            const RowTask d = a.task[t];
            d_row = d.row;
            d_len = d.len;
            d_start = d.start;
            if constexpr (SRC == kSrcDenseThenBf16 || SRC == kSrcDenseThenQuant) d_split = a.split[d.row];
        } else {
            d_row = (int)t;
            d_start = a.rowptr[t];
            d_len = (int)(a.rowptr[t + 1] - d_start);
        }
    }
    if constexpr (MODE == kRowsNatural) {
        if (!scanner) {
            // rows without elements keep their value when accumulating: not visited; long rows belong to the scanners
            const bool mine = lig < ntask && (d_len > 0 || !a.accumulate) && !(a.long_len > 0 && d_len > a.long_len);
            todo = group_ballot<LPR>(mine);
            if (todo == 0) return;
        }
    }

    const bool from_dst = a.accumulate != 0;
    const int ldd = a.ldd ? a.ldd : F;

    for (;;) {  // one pass, except in a scanner block: one pass per stretch of LPR rows that holds long rows
        if constexpr (MODE == kRowsNatural) {
            if (scanner) {
                todo = 0;
                while (todo == 0 && scan_next < scan_end) {
                    const int64_t r = scan_next + lig;
                    d_len = 0;
                    if (r < scan_end) {
                        d_row = (int)r;
                        d_start = a.rowptr[r];
                        d_len = (int)(a.rowptr[r + 1] - d_start);
                    }
                    todo = group_ballot<LPR>(d_len > a.long_len);
                    scan_next += LPR;
                }
                if (todo == 0) return;
            }
        }

        // State of the row being accumulated and of the chunk of <= LPR (col, val) pairs held
        // across the group's lanes.  The NEXT chunk -- of the same row, or the first chunk of
        // the group's next row -- is always requested before the current chunk's gathers, so
        // that the index stream never sits on the critical path.
        int i = 0;
        if constexpr (MODE == kRowsNatural) {
            i = __builtin_ctzll(todo);
            todo &= todo - 1;
        }
        int row = group_bcast<LPR>(d_row, i);
        int64_t base = group_bcast_idx<LPR>(d_start, i);
        int64_t end = base + group_bcast<LPR>(d_len, i);
        int64_t first_end = base;  // (two-format launches) where the row's elements of the second source begin
        if constexpr (SRC == kSrcDenseThenBf16 || SRC == kSrcDenseThenQuant) first_end = base + group_bcast<LPR>(d_split, i);
        IdxT c_l = 0;
        float v_l = 0.0f;
        if (base + lig < end) {
            c_l = __builtin_nontemporal_load(col + base + lig);
            v_l = __builtin_nontemporal_load(val + base + lig);
        }
        float *dst = a.dst + (size_t)row * (size_t)ldd;
        V acc[NCH];
#pragma unroll
        for (int k = 0; k < NCH; ++k) {
            acc[k] = V::zero();
            if (from_dst && fok[k]) acc[k] = V::load_stream(dst + foff[k]);
        }

        while (true) {
            const int64_t left = end - base;
            const int cnt = left < LPR ? (int)left : LPR;

            // where the next chunk comes from
            int ni = i;
            int nrow = row;
            int64_t nbase = base + LPR, nend = end, nfirst_end = first_end;
            bool row_done = nbase >= end;
            bool more = true;
            if (row_done) {
                if constexpr (MODE == kRowsNatural) {
                    more = todo != 0;
                    if (more) {
                        ni = __builtin_ctzll(todo);
                        todo &= todo - 1;
                    }
                } else {
                    ni = i + 1;
                    more = ni < ntask;
                }
                if (more) {
                    nrow = group_bcast<LPR>(d_row, ni);
                    nbase = group_bcast_idx<LPR>(d_start, ni);
                    nend = nbase + group_bcast<LPR>(d_len, ni);
                    if constexpr (SRC == kSrcDenseThenBf16 || SRC == kSrcDenseThenQuant)
                        nfirst_end = nbase + group_bcast<LPR>(d_split, ni);
                }
            }
            IdxT nc = 0;
            float nv = 0.0f;
            if (more && nbase + lig < nend) {
                nc = __builtin_nontemporal_load(col + nbase + lig);
                nv = __builtin_nontemporal_load(val + nbase + lig);
            }

            if constexpr (SRC == kSrcDenseThenBf16 || SRC == kSrcDenseThenQuant) {
                // the chunk's elements in front of the row's split read the dense source, the others the second one
                const int64_t ahead = first_end - base;
                const int cnt_a = ahead <= 0 ? 0 : (ahead < cnt ? (int)ahead : cnt);
                gather_rounds<VEC, LPR, NCH, kSrcDense, IdxT, false, true>(acc, c_l, v_l, 0, cnt_a, a, foff);
                gather_rounds<VEC, LPR, NCH, SRC == kSrcDenseThenBf16 ? kSrcBf16 : kSrcQuant, IdxT, true, true>(
                    acc, c_l, v_l, cnt_a, cnt, a, foff);
            } else {
                gather_rounds<VEC, LPR, NCH, SRC, IdxT>(acc, c_l, v_l, 0, cnt, a, foff);
            }

            if (row_done) {
                if constexpr (VEC == 4) {
                    if (a.dst_bf16) {  // the result rows are bf16 (overwriting only): rounded once, here
                        unsigned short *d16 = reinterpret_cast<unsigned short *>(a.dst) + (size_t)row * (size_t)ldd;
#pragma unroll
                        for (int k = 0; k < NCH; ++k) {
                            if (fok[k]) {
                                typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
                                u32x2 r;
                                r.x = (uint32_t)bf16_bits(acc[k].d.x) | ((uint32_t)bf16_bits(acc[k].d.y) << 16);
                                r.y = (uint32_t)bf16_bits(acc[k].d.z) | ((uint32_t)bf16_bits(acc[k].d.w) << 16);
                                __builtin_nontemporal_store(r, reinterpret_cast<u32x2 *>(d16 + foff[k]));
                            }
                        }
                    } else {
#pragma unroll
                        for (int k = 0; k < NCH; ++k) {
                            if (fok[k]) acc[k].store_stream(dst + foff[k]);
                        }
                    }
                } else {
#pragma unroll
                    for (int k = 0; k < NCH; ++k) {
                        if (fok[k]) acc[k].store_stream(dst + foff[k]);
                    }
                }
                if (!more) break;
                dst = a.dst + (size_t)nrow * (size_t)ldd;
#pragma unroll
                for (int k = 0; k < NCH; ++k) {
                    acc[k] = V::zero();
                    if (from_dst && fok[k]) acc[k] = V::load_stream(dst + foff[k]);
                }
            }
            i = ni;
            row = nrow;
            base = nbase;
            end = nend;
            first_end = nfirst_end;
            c_l = nc;
            v_l = nv;
        }
        if constexpr (MODE == kRowsNatural) {
            if (!scanner) return;
        } else {
            return;
        }
    }
}


// ---------------------------------------------------------------------------------------
// Very long rows.  One block per (row, feature tile of 16 .. 64 floats): four FETCH waves and,
// behind them, one CHAIN wave.  The row's chain must stay
// sequential (bit-identical results), so what is parallelised is the fetch: the fetch waves
// gather a chunk of dense rows at once (up to 8 vector loads per thread and chunk) and land it
// in LDS, while in the chain wave the lane that owns a feature runs the FMA chain over the
// chunk landed before, in CSR order, and does nothing else.  A chunk lies TRANSPOSED in LDS --
// tile[feature][element of the chunk] -- so that the owner of a feature reads four consecutive
// elements with one 16-byte LDS read, and the four matrix values that go with them with
// another (the same address in every lane): 1.5 instructions per stored element, of which only
// the FMA is on the chain.  Measured in one wave on this part: 1.9 ns per element for the bare
// chain, 3.7 ns with these reads (sixteen and sixteen requested ahead of their 64 FMAs), 3.9 ns
// with the matrix value handed round by v_readlane instead, 5.8 ns with a 4-byte LDS read per
// element on top of that.  A row advances by one chunk per memory round trip, so the chunk is
// made as long as a tile buffer allows -- 96 rows of 64 floats, 384 rows of 16 -- and the host
// cuts the rows into narrow feature tiles (every feature's chain is its own), which also
// spreads one row's fetch over several compute units.  kLongDepth chunks are in
// flight in registers; the (col, val) pairs come in super-chunks of kLongDepth chunks, two
// super-chunks ahead.
// ---------------------------------------------------------------------------------------
constexpr int kLongTileFloats = 6144;  // most floats of one chunk (tile width x rows of the chunk)
constexpr int kLongMaxChunk = 384;     // most dense rows gathered per chunk
constexpr int kLongRowPad = 4;         // floats between the feature rows of a tile buffer: lanes f, f + 1, ... read
                                       // 16 bytes each at a stride of chunk + 4 floats, 16 lanes covering all banks
constexpr int kLongFeatTile = 64;      // most features per block: one chain wave (wider tiles mean shorter chunks, which
                                       // two chunks in flight no longer cover: 34 ns per element at 128 floats, 70 at 256)
constexpr int kLongFetchThreads = 256; // the fetch waves of a block; behind them the chain wave
// floats of one tile buffer: width x (chunk + pad) <= kLongTileFloats + kLongFeatTile * kLongRowPad, and four
// floats behind them where the fetch slots past a chunk's rows land
constexpr int kLongDump = kLongTileFloats + kLongFeatTile * kLongRowPad;
constexpr int kLongBufFloats = kLongDump + 4;
constexpr int kLongLoads = 8;          // most vector loads per thread and chunk
constexpr int kLongDepth = 2;          // chunks in flight
constexpr int kLongMinFeatTile = 16;   // fewest: one 64-byte piece of every gathered row
constexpr int kLongPairs = kLongDepth * kLongMaxChunk / 256;  // (col, val) pairs per thread and super-chunk
// dynamic LDS: two tile buffers, then three (col, val) super-chunk buffers
constexpr size_t kLongSmemBytes =
    2 * kLongBufFloats * sizeof(float) + 3 * kLongDepth * kLongMaxChunk * (sizeof(int) + sizeof(float));

struct LongArgs {
    const RowTask *task;  // rows handled: task[0 .. gridDim.x / tiles)
    const int32_t *col;
    const float *val;
    const float *x;
    float *dst;
    int feat;        // F
    int ldx, ldd;    // row strides of x and dst in floats; 0 stands for F
    int tile;        // features per block (a multiple of VEC, <= kLongFeatTile)
    int tiles;       // tiles per row: the grid is rows x tiles blocks, block b = row b / tiles, tile b % tiles
    int chunk;       // dense rows per chunk, a multiple of 4: chunk * tile <= kLongTileFloats, chunk * (tile / VEC) <= 2048
    int accumulate;
};

// The chain over `cnt` stored elements for the feature a thread owns: tb = the feature's row of the tile buffer
// (element j of the chunk at tb[j]), vb = the matrix values of the chunk; both 16-byte aligned.  Sixteen 16-byte
// reads of each are requested back to back ahead of their 64 FMAs.
__device__ __forceinline__ float chain_over_chunk(const float *tb, const float *vb, int cnt, float acc) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    // the matrix values sit at the same address for every lane; kept in a vector register all the same, so that
    // the sixteen reads of a round are one base and sixteen immediates instead of sixteen scalar adds and moves
    int same = 0;
    asm volatile("" : "+v"(same));
    vb += same;
    int j = 0;
    for (; j + 64 <= cnt; j += 64) {
        f4 xs[16], vs[16];
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            xs[q] = *reinterpret_cast<const f4 *>(tb + j + 4 * q);
            vs[q] = *reinterpret_cast<const f4 *>(vb + j + 4 * q);
        }
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            acc = __builtin_fmaf(vs[q].x, xs[q].x, acc);
            acc = __builtin_fmaf(vs[q].y, xs[q].y, acc);
            acc = __builtin_fmaf(vs[q].z, xs[q].z, acc);
            acc = __builtin_fmaf(vs[q].w, xs[q].w, acc);
        }
    }
    for (; j + 4 <= cnt; j += 4) {
        const f4 x = *reinterpret_cast<const f4 *>(tb + j);
        const f4 v = *reinterpret_cast<const f4 *>(vb + j);
        acc = __builtin_fmaf(v.x, x.x, acc);
        acc = __builtin_fmaf(v.y, x.y, acc);
        acc = __builtin_fmaf(v.z, x.z, acc);
        acc = __builtin_fmaf(v.w, x.w, acc);
    }
    for (; j < cnt; ++j) acc = __builtin_fmaf(vb[j], tb[j], acc);
    return acc;
}

// NL: vector loads per thread and chunk, the smallest of 1, 2, 4, 8 with NL * 256 >= chunk * (tile / VEC).
// FW: the width of EVERY tile of the launch when that is one of 16 .. 256 and divides F, else 0.
template <int VEC, int NL, int FW = 0>
__global__ __launch_bounds__(kLongFetchThreads + kLongFeatTile) void spmm_long_rows_kernel(const LongArgs a) {
    typedef FVec<VEC> V;
    constexpr int D = kLongDepth;
    constexpr int kSuper = D * kLongMaxChunk;  // index pairs per super-chunk buffer
    extern __shared__ __attribute__((aligned(16))) unsigned char long_smem[];
    float(*tile)[kLongBufFloats] = reinterpret_cast<float(*)[kLongBufFloats]>(long_smem);
    int(*s_col)[kSuper] = reinterpret_cast<int(*)[kSuper]>(long_smem + 2 * kLongBufFloats * sizeof(float));
    float(*s_val)[kSuper] = reinterpret_cast<float(*)[kSuper]>(long_smem + 2 * kLongBufFloats * sizeof(float) +
                                                               3 * kSuper * sizeof(int));

    const int t = (int)threadIdx.x;
    // blocks are handed out in the order of their index: the tiles of one row next to each other, rows in the order
    // of the schedule (longest first), so that the longest row's blocks all start at once
    const int row_of_block = (int)(blockIdx.x / (unsigned)a.tiles);
    const int tile_of_block = (int)(blockIdx.x % (unsigned)a.tiles);
    const RowTask d = a.task[row_of_block];
    const int F = a.feat;
    const int ldx = a.ldx ? a.ldx : F;
    const int f0 = tile_of_block * a.tile;
    const int fw = FW ? FW : (F - f0 < a.tile ? F - f0 : a.tile);    // width of this tile (multiple of VEC)
    const int vpr = fw / VEC;                                        // vectors per gathered row
    const int C = a.chunk;
    const int SC = D * C;                                            // stored elements per super-chunk
    const int nchunks = (d.len + C - 1) / C;
    const float *__restrict__ x = a.x + f0;
    const int32_t *__restrict__ col = a.col + d.start;
    const float *__restrict__ val = a.val + d.start;

    // fixed (dense row in chunk, vector in row) slots of this thread: slot e is row e / vpr, vector e % vpr; its
    // VEC floats land in the feature rows sv .. sv + VEC - 1 of a tile buffer at element sj
    const int stride = C + kLongRowPad;  // floats between the feature rows of a tile buffer (C is a multiple of 4)
    int sj[NL], sv[NL];
    int land_at[NL], land_step[NL];  // where the slot's first float lands, and how far apart its floats do
#pragma unroll
    for (int s = 0; s < NL; ++s) {
        const int e = t + s * 256;
        sj[s] = e / vpr;
        sv[s] = (e - sj[s] * vpr) * VEC;
        // a slot past the chunk's rows fetches a repeat of the last row: it lands behind the tile, where nobody
        // reads (no branch around the stores: with one, the compiler waits for every load in flight instead)
        land_at[s] = sj[s] < C ? sv[s] * stride + sj[s] : kLongDump;
        land_step[s] = sj[s] < C ? stride : 0;
    }

    auto chunk_len = [&](int k) { const int left = d.len - k * C; return left < C ? left : C; };
    // chunk k sits in super-chunk k / D (buffer (k / D) % 3) at offset (k % D) * C.  Every slot loads and
    // lands, whatever the chunk holds (a slot past the chunk's last row repeats that row and lands where
    // nobody reads): loads under a branch would make every later wait a wait for ALL loads in flight.
    auto request = [&](int k, V(&g)[NL]) {
        const int last = chunk_len(k) - 1;
        const int *cb = &s_col[(k / D) % 3][(k % D) * C];
#pragma unroll
        for (int s = 0; s < NL; ++s) {
            const int j = sj[s] < last ? sj[s] : last;
            g[s] = V::load(x + (size_t)cb[j] * (size_t)ldx + sv[s]);
        }
    };
    auto land = [&](int k, const V(&g)[NL]) {
        float *tb = tile[k & 1];
#pragma unroll
        for (int s = 0; s < NL; ++s) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) tb[land_at[s] + i * land_step[s]] = g[s].at(i);
        }
    };

    float *dst = a.dst + (size_t)d.row * (size_t)(a.ldd ? a.ldd : F) + f0;

    // Threads 256 and up are the chain wave, one lane per feature of the tile; it fetches nothing.  Both kinds of
    // wave pass the same barriers: two in the prologue, one per chunk.
    if (t >= 256) {
        const int f = t - 256;
        const bool own = f < fw;
        __syncthreads();
        __syncthreads();
        float acc = 0.0f;
        if (own && a.accumulate) acc = __builtin_nontemporal_load(dst + f);
        const float *mine = &tile[0][(own ? f : 0) * stride];
        for (int k = 0; k < nchunks; ++k) {
            // the chain over chunk k, in CSR order, out of LDS, while the fetch waves land chunk k + 1; lanes past
            // the tile's width sit it out (an LDS read costs by the lanes that take part)
            if (own)
                acc = chain_over_chunk(mine + (k & 1) * kLongBufFloats, &s_val[(k / D) % 3][(k % D) * C], chunk_len(k),
                                       acc);
            __syncthreads();
        }
        if (own) __builtin_nontemporal_store(acc, dst + f);
        return;
    }

    // prologue: index pairs of super-chunks 0 and 1, dense rows of chunks 0 .. D-1, chunk 0 landed
#pragma unroll
    for (int p = 0; p < kLongPairs; ++p) {
        const int e = t + p * 256;
        if (e < SC && e < d.len) {
            s_col[0][e] = __builtin_nontemporal_load(col + e);
            s_val[0][e] = __builtin_nontemporal_load(val + e);
        }
        if (e < SC && SC + e < d.len) {
            s_col[1][e] = __builtin_nontemporal_load(col + SC + e);
            s_val[1][e] = __builtin_nontemporal_load(val + SC + e);
        }
    }
    __syncthreads();
    V g[D][NL];
#pragma unroll
    for (int u = 0; u < D; ++u) request(u < nchunks ? u : nchunks - 1, g[u]);
    land(0, g[0]);
    __syncthreads();

    for (int kb = 0; kb < nchunks; kb += D) {
        // index pairs of the super-chunk after the next one: requested now, stored at the end
        const int super = kb / D;
        const int64_t base2 = (int64_t)(super + 2) * SC;
        int ci[kLongPairs];
        float vi[kLongPairs];
#pragma unroll
        for (int p = 0; p < kLongPairs; ++p) {
            // past the super-chunk or the row: the row's last pair once more, stored where nobody reads
            int64_t e2 = base2 + t + p * 256;
            if (e2 > d.len - 1) e2 = d.len - 1;
            ci[p] = __builtin_nontemporal_load(col + e2);
            vi[p] = __builtin_nontemporal_load(val + e2);
        }
#pragma unroll
        for (int u = 0; u < D; ++u) {
            const int k = kb + u;
            if (k >= nchunks) break;  // the same for every thread of the block
            // (1) chunk k left its registers for LDS in the step before: request chunk k + D into them
            //     (past the row's end: the last chunk once more, never landed where it is read)
            request(k + D < nchunks ? k + D : nchunks - 1, g[u]);
            // (2) land chunk k + 1 (requested D - 1 steps ago) in the tile buffer the chain wave is not reading
            land(k + 1, g[(u + 1) % D]);
            if (u == D - 1) {
#pragma unroll
                for (int p = 0; p < kLongPairs; ++p) {
                    s_col[(super + 2) % 3][t + p * 256] = ci[p];
                    s_val[(super + 2) % 3][t + p * 256] = vi[p];
                }
            }
            __syncthreads();
        }
    }
}

}  // namespace gnnagg
