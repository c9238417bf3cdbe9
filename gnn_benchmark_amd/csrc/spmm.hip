// Host side of the SpMM entry points: launch-shape selection, the direct (plan-less)
// path, and the cached degree-binned plan.  gfx950 only.
#include <hipcub/hipcub.hpp>

#include <algorithm>
#include <new>
#include <vector>

#include "common.h"
#include "spmm_kernels.h"

namespace gnnagg {

std::string &last_error_slot() {
    static thread_local std::string s;
    return s;
}

namespace {

// ------------------------------------------------------------------ launch shapes
// A launch shape is (VEC floats per lane-load, LPR lanes per task, NCH loads per lane):
// it covers VEC*LPR*NCH consecutive features.  The host picks the smallest shape that
// covers the feature row; wider rows are tiled over several launches.
struct Shape {
    int vec, lpr, nch;
    int width() const { return vec * lpr * nch; }
};

constexpr int kShapes[][2] = {{16, 1}, {32, 1}, {64, 1}, {64, 2}, {64, 3}, {64, 4}, {64, 5}, {64, 6}, {64, 8}};
constexpr int kNumShapes = sizeof(kShapes) / sizeof(kShapes[0]);

int pick_vec(int64_t feat, const void *x, const void *dst) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dst);
    if (feat % 4 == 0 && bits % 16 == 0) return 4;
    if (feat % 2 == 0 && bits % 8 == 0) return 2;
    return 1;
}

Shape pick_shape(int vec, int64_t feat_left) {
    for (int i = 0; i < kNumShapes; ++i) {
        Shape s{vec, kShapes[i][0], kShapes[i][1]};
        if (s.width() >= feat_left) return s;
    }
    return Shape{vec, kShapes[kNumShapes - 1][0], kShapes[kNumShapes - 1][1]};
}

template <int VEC, int LPR, int NCH, typename IdxT, int MODE>
hipError_t launch_tasks(const SpmmArgs &a, int rows_per_group, hipStream_t stream) {
    constexpr int GPB = 256 / LPR;
    SpmmArgs args = a;
    args.tasks_per_block = GPB * rows_per_group;
    const int64_t nblocks = (a.ntasks + args.tasks_per_block - 1) / args.tasks_per_block;
    if (nblocks == 0) return hipSuccess;
    if (nblocks > 0x7fffffffll) return hipErrorInvalidValue;
    hipLaunchKernelGGL((spmm_tasks_kernel<VEC, LPR, NCH, IdxT, MODE>), dim3((unsigned)nblocks), dim3(256), 0, stream,
                       args);
    return hipGetLastError();
}

template <int VEC, typename IdxT, int MODE>
hipError_t dispatch_shape(const Shape &s, const SpmmArgs &a, int rpg, hipStream_t st) {
#define GNNAGG_CASE(L, N) \
    if (s.lpr == L && s.nch == N) return launch_tasks<VEC, L, N, IdxT, MODE>(a, rpg, st)
    GNNAGG_CASE(16, 1);
    GNNAGG_CASE(32, 1);
    GNNAGG_CASE(64, 1);
    GNNAGG_CASE(64, 2);
    GNNAGG_CASE(64, 3);
    GNNAGG_CASE(64, 4);
    GNNAGG_CASE(64, 5);
    GNNAGG_CASE(64, 6);
    GNNAGG_CASE(64, 8);
#undef GNNAGG_CASE
    return hipErrorInvalidValue;
}

template <typename IdxT, int MODE>
hipError_t dispatch_tasks(const Shape &s, const SpmmArgs &a, int rpg, hipStream_t st) {
    if (s.vec == 4) return dispatch_shape<4, IdxT, MODE>(s, a, rpg, st);
    if (s.vec == 2) return dispatch_shape<2, IdxT, MODE>(s, a, rpg, st);
    return dispatch_shape<1, IdxT, MODE>(s, a, rpg, st);
}

template <int VEC>
hipError_t dispatch_reduce_vec(const Shape &s, const ReduceArgs &a, hipStream_t st) {
#define GNNAGG_CASE(L, N)                                                                               \
    if (s.lpr == L && s.nch == N) {                                                                     \
        constexpr int GPB = 256 / L;                                                                    \
        hipLaunchKernelGGL((heavy_reduce_kernel<VEC, L, N>), dim3((unsigned)((a.nheavy + GPB - 1) / GPB)), \
                           dim3(256), 0, st, a);                                                        \
        return hipGetLastError();                                                                       \
    }
    GNNAGG_CASE(16, 1)
    GNNAGG_CASE(32, 1)
    GNNAGG_CASE(64, 1)
    GNNAGG_CASE(64, 2)
    GNNAGG_CASE(64, 3)
    GNNAGG_CASE(64, 4)
    GNNAGG_CASE(64, 5)
    GNNAGG_CASE(64, 6)
    GNNAGG_CASE(64, 8)
#undef GNNAGG_CASE
    return hipErrorInvalidValue;
}

hipError_t dispatch_reduce(const Shape &s, const ReduceArgs &a, hipStream_t st) {
    if (a.nheavy == 0) return hipSuccess;
    if (s.vec == 4) return dispatch_reduce_vec<4>(s, a, st);
    if (s.vec == 2) return dispatch_reduce_vec<2>(s, a, st);
    return dispatch_reduce_vec<1>(s, a, st);
}

// ------------------------------------------------------------------ plan kernels
constexpr int kMaxClasses = 40;

struct ClassifyOut {
    unsigned long long class_count[kMaxClasses];
    unsigned long long max_deg;
    unsigned int bad_rowptr;  // rowptr decreasing somewhere
    unsigned int bad_col;     // a column index outside [0, cols)
};

// Degree class of a row: 0 = cut into segments (deg > heavy_thresh); then one class per
// power-of-two degree bucket in DESCENDING degree order; the last class holds empty rows.
__device__ __forceinline__ int degree_class(int64_t deg, int heavy_thresh, int heavy_log) {
    if (deg > heavy_thresh) return 0;
    if (deg == 0) return heavy_log + 2;
    const int clog = deg <= 1 ? 0 : 64 - __builtin_clzll((unsigned long long)(deg - 1));  // ceil(log2(deg))
    return 1 + (heavy_log - clog);
}

__global__ __launch_bounds__(256) void classify_rows_kernel(const int64_t *__restrict__ rowptr, int rows,
                                                            int heavy_thresh, int heavy_log,
                                                            uint32_t *__restrict__ key, int32_t *__restrict__ rowid,
                                                            ClassifyOut *__restrict__ out) {
    __shared__ unsigned int hist[kMaxClasses];
    __shared__ unsigned long long smax;
    if (threadIdx.x < kMaxClasses) hist[threadIdx.x] = 0;
    if (threadIdx.x == 0) smax = 0;
    __syncthreads();
    const int r = (int)blockIdx.x * 256 + (int)threadIdx.x;
    if (r < rows) {
        const int64_t d = rowptr[r + 1] - rowptr[r];
        if (d < 0) {
            atomicOr(&out->bad_rowptr, 1u);
            key[r] = (uint32_t)(heavy_log + 2);
        } else {
            const int c = degree_class(d, heavy_thresh, heavy_log);
            key[r] = (uint32_t)c;
            atomicAdd(&hist[c], 1u);
            atomicMax(&smax, (unsigned long long)d);
        }
        rowid[r] = r;
    }
    __syncthreads();
    if (threadIdx.x < kMaxClasses && hist[threadIdx.x])
        atomicAdd(&out->class_count[threadIdx.x], (unsigned long long)hist[threadIdx.x]);
    if (threadIdx.x == 0 && smax) atomicMax(&out->max_deg, smax);
}

__global__ __launch_bounds__(256) void narrow_cols_kernel(const int64_t *__restrict__ col, int64_t nnz, int64_t cols,
                                                          int32_t *__restrict__ col32, ClassifyOut *__restrict__ out) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    bool bad = false;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < nnz; e += stride) {
        const int64_t c = col[e];
        bad |= (c < 0) | (c >= cols);
        col32[e] = (int32_t)c;
    }
    if (bad) atomicOr(&out->bad_col, 1u);
}

// nseg[h] for the rows cut into segments (the first nheavy entries of perm).
__global__ __launch_bounds__(256) void heavy_count_kernel(const int64_t *__restrict__ rowptr,
                                                          const int32_t *__restrict__ perm, int nheavy, int seg_len,
                                                          int64_t *__restrict__ nseg) {
    const int h = (int)blockIdx.x * 256 + (int)threadIdx.x;
    if (h >= nheavy) return;
    const int r = perm[h];
    const int64_t d = rowptr[r + 1] - rowptr[r];
    nseg[h] = (d + seg_len - 1) / seg_len;
}

// One thread per segment: find its row by binary search in segbase, write (start, len).
__global__ __launch_bounds__(256) void heavy_expand_kernel(const int64_t *__restrict__ rowptr,
                                                           const int32_t *__restrict__ perm,
                                                           const int64_t *__restrict__ segbase, int nheavy,
                                                           int64_t nseg_total, int seg_len,
                                                           int64_t *__restrict__ seg_start,
                                                           int32_t *__restrict__ seg_n) {
    const int64_t s = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (s >= nseg_total) return;
    int lo = 0, hi = nheavy;  // last h with segbase[h] <= s
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (segbase[mid] <= s) lo = mid; else hi = mid;
    }
    const int r = perm[lo];
    const int64_t k = s - segbase[lo];
    const int64_t b = rowptr[r] + k * seg_len;
    const int64_t e = rowptr[r + 1];
    seg_start[s] = b;
    seg_n[s] = (int32_t)((e - b) < seg_len ? (e - b) : seg_len);
}

int env_int(const char *name, int dflt, int lo, int hi) {
    const char *v = getenv(name);
    if (!v || !*v) return dflt;
    const long x = strtol(v, nullptr, 10);
    if (x < lo || x > hi) return dflt;
    return (int)x;
}

}  // namespace
}  // namespace gnnagg

using namespace gnnagg;

struct gnnagg_plan {
    int64_t rows = 0, cols = 0, nnz = 0;
    int seg_len = 0;          // nnz per segment of a cut row
    int heavy_thresh = 0;     // rows longer than this are cut
    int64_t nheavy = 0;       // rows cut into segments
    int64_t nseg = 0;         // segments
    int64_t nempty = 0;       // rows with no stored element
    int64_t max_deg = 0;
    int device = 0;
    int64_t *rowptr = nullptr;     // [rows+1] own copy
    int32_t *col32 = nullptr;      // [nnz]
    int32_t *perm = nullptr;       // [rows] rows by class: cut rows, then descending degree, then empty
    int64_t *segbase = nullptr;    // [nheavy+1]
    int64_t *seg_start = nullptr;  // [nseg]
    int32_t *seg_n = nullptr;      // [nseg]
    float *partial = nullptr;      // [nseg, partial_feat] scratch of segment sums
    int64_t partial_feat = 0;
    int rows_per_group = 4;
    bool profile = false;
    bool profile_valid = false;
    hipEvent_t ev[4] = {nullptr, nullptr, nullptr, nullptr};  // call begin, rows-kernel begin/end, call end
};

extern "C" int gnnagg_abi_version(void) { return GNNAGG_ABI_VERSION; }

extern "C" const char *gnnagg_last_error(void) { return last_error_slot().c_str(); }

static int check_feat(int64_t feat) {
    if (feat <= 0 || feat > (1 << 20))
        return fail(GNNAGG_ERR_UNSUPPORTED, "feature width %lld outside [1, 2^20]", (long long)feat);
    return GNNAGG_OK;
}

extern "C" int gnnagg_spmm_csr_f32(const int64_t *rowptr, const int64_t *col, const float *value, const float *mat,
                                   float *out, int64_t sparse_rows, int64_t feat, void *stream) {
    GNNAGG_REQUIRE(sparse_rows >= 0 && feat >= 0, "negative size (rows=%lld feat=%lld)", (long long)sparse_rows,
                   (long long)feat);
    if (sparse_rows == 0 || feat == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(rowptr && out, "null rowptr/out");
    GNNAGG_REQUIRE(col && value && mat, "null col/value/mat");
    if (int rc = check_feat(feat)) return rc;
    if (sparse_rows >= (int64_t(1) << 31))
        return fail(GNNAGG_ERR_UNSUPPORTED, "more than 2^31-1 sparse rows (%lld)", (long long)sparse_rows);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int vec = pick_vec(feat, mat, out);
    for (int64_t f_base = 0; f_base < feat;) {
        const Shape s = pick_shape(vec, feat - f_base);
        SpmmArgs a{};
        a.rowptr = rowptr;
        a.col = col;
        a.val = value;
        a.x = mat;
        a.dst = out;
        a.ntasks = sparse_rows;
        a.feat = (int)feat;
        a.f_base = (int)f_base;
        a.accumulate = 1;
        GNNAGG_HIP((dispatch_tasks<int64_t, kRowsNatural>(s, a, 4, st)));
        f_base += s.width();
    }
    return GNNAGG_OK;
}

static void plan_free(gnnagg_plan *p) {
    if (!p) return;
    (void)hipFree(p->rowptr);
    (void)hipFree(p->col32);
    (void)hipFree(p->perm);
    (void)hipFree(p->segbase);
    (void)hipFree(p->seg_start);
    (void)hipFree(p->seg_n);
    (void)hipFree(p->partial);
    for (hipEvent_t e : p->ev)
        if (e) (void)hipEventDestroy(e);
    delete p;
}

extern "C" int gnnagg_plan_create(const int64_t *rowptr, const int64_t *col, int64_t rows, int64_t cols, int64_t nnz,
                                  void *stream, gnnagg_plan **plan_out) {
    GNNAGG_REQUIRE(plan_out, "null plan_out");
    *plan_out = nullptr;
    GNNAGG_REQUIRE(rows >= 0 && cols >= 0 && nnz >= 0, "negative size");
    GNNAGG_REQUIRE(rowptr, "null rowptr");
    GNNAGG_REQUIRE(nnz == 0 || col, "null col with nnz > 0");
    if (rows >= (int64_t(1) << 31) - 1 || cols >= (int64_t(1) << 31) - 1 || nnz >= (int64_t(1) << 40))
        return fail(GNNAGG_ERR_UNSUPPORTED, "plan limits: rows, cols < 2^31-1, nnz < 2^40 (got %lld, %lld, %lld)",
                    (long long)rows, (long long)cols, (long long)nnz);
    hipStream_t st = static_cast<hipStream_t>(stream);

    gnnagg_plan *p = new (std::nothrow) gnnagg_plan();
    if (!p) return fail(GNNAGG_ERR_HIP, "out of host memory");
    struct Guard {
        gnnagg_plan *p;
        ~Guard() { plan_free(p); }
    } guard{p};

    p->rows = rows;
    p->cols = cols;
    p->nnz = nnz;
    p->seg_len = env_int("GNNAGG_SEG_LEN", 256, 32, 1 << 20);
    p->heavy_thresh = env_int("GNNAGG_HEAVY_THRESH", 2 * p->seg_len, p->seg_len, 1 << 24);
    p->rows_per_group = env_int("GNNAGG_ROWS_PER_GROUP", 4, 1, 1024);
    GNNAGG_HIP(hipGetDevice(&p->device));
    const int heavy_log = ceil_log2_u64((uint64_t)p->heavy_thresh);
    const int nclasses = heavy_log + 3;
    GNNAGG_REQUIRE(nclasses <= kMaxClasses, "heavy threshold too large");

    // rowptr end points (host check; also forces the inputs to be ready)
    int64_t ends[2] = {0, 0};
    GNNAGG_HIP(hipMemcpyAsync(&ends[0], rowptr, sizeof(int64_t), hipMemcpyDeviceToHost, st));
    GNNAGG_HIP(hipMemcpyAsync(&ends[1], rowptr + rows, sizeof(int64_t), hipMemcpyDeviceToHost, st));
    GNNAGG_HIP(hipStreamSynchronize(st));
    GNNAGG_REQUIRE(ends[0] == 0 && ends[1] == nnz, "rowptr[0]=%lld, rowptr[rows]=%lld do not match nnz=%lld",
                   (long long)ends[0], (long long)ends[1], (long long)nnz);

    GNNAGG_HIP(hipMalloc((void **)&p->rowptr, sizeof(int64_t) * (size_t)(rows + 1)));
    GNNAGG_HIP(hipMemcpyAsync(p->rowptr, rowptr, sizeof(int64_t) * (size_t)(rows + 1), hipMemcpyDeviceToDevice, st));
    GNNAGG_HIP(hipMalloc((void **)&p->col32, sizeof(int32_t) * (size_t)std::max<int64_t>(nnz, 1)));
    GNNAGG_HIP(hipMalloc((void **)&p->perm, sizeof(int32_t) * (size_t)std::max<int64_t>(rows, 1)));

    DevBuf<ClassifyOut> d_out;
    GNNAGG_HIP(d_out.alloc(1));
    GNNAGG_HIP(hipMemsetAsync(d_out.p, 0, sizeof(ClassifyOut), st));

    ClassifyOut h_out{};
    if (rows > 0) {
        DevBuf<uint32_t> key_in, key_out;
        DevBuf<int32_t> row_in;
        GNNAGG_HIP(key_in.alloc((size_t)rows));
        GNNAGG_HIP(key_out.alloc((size_t)rows));
        GNNAGG_HIP(row_in.alloc((size_t)rows));
        hipLaunchKernelGGL(classify_rows_kernel, dim3(grid_for(rows, 256)), dim3(256), 0, st, p->rowptr, (int)rows,
                           p->heavy_thresh, heavy_log, key_in.p, row_in.p, d_out.p);
        GNNAGG_HIP(hipGetLastError());
        if (nnz > 0) {
            const unsigned g = (unsigned)std::min<int64_t>((nnz + 255) / 256, 1 << 20);
            hipLaunchKernelGGL(narrow_cols_kernel, dim3(g), dim3(256), 0, st, col, nnz, cols, p->col32, d_out.p);
            GNNAGG_HIP(hipGetLastError());
        }
        // stable sort of the rows by class: ascending row id inside a class
        size_t tmp_bytes = 0;
        const int end_bit = std::max(1, ceil_log2_u64((uint64_t)nclasses));
        GNNAGG_HIP(hipcub::DeviceRadixSort::SortPairs(nullptr, tmp_bytes, key_in.p, key_out.p, row_in.p, p->perm,
                                                      (int)rows, 0, end_bit, st));
        DevBuf<char> tmp;
        GNNAGG_HIP(tmp.alloc(std::max<size_t>(tmp_bytes, 1)));
        GNNAGG_HIP(hipcub::DeviceRadixSort::SortPairs(tmp.p, tmp_bytes, key_in.p, key_out.p, row_in.p, p->perm,
                                                      (int)rows, 0, end_bit, st));
        GNNAGG_HIP(hipMemcpyAsync(&h_out, d_out.p, sizeof(ClassifyOut), hipMemcpyDeviceToHost, st));
        GNNAGG_HIP(hipStreamSynchronize(st));
    }
    GNNAGG_REQUIRE(!h_out.bad_rowptr, "rowptr is not non-decreasing");
    GNNAGG_REQUIRE(!h_out.bad_col, "a column index lies outside [0, %lld)", (long long)cols);
    p->nheavy = (int64_t)h_out.class_count[0];
    p->nempty = (int64_t)h_out.class_count[nclasses - 1];
    p->max_deg = (int64_t)h_out.max_deg;

    if (p->nheavy > 0) {
        DevBuf<int64_t> nseg;
        GNNAGG_HIP(nseg.alloc((size_t)p->nheavy + 1));
        GNNAGG_HIP(hipMemsetAsync(nseg.p, 0, sizeof(int64_t) * ((size_t)p->nheavy + 1), st));
        hipLaunchKernelGGL(heavy_count_kernel, dim3(grid_for(p->nheavy, 256)), dim3(256), 0, st, p->rowptr, p->perm,
                           (int)p->nheavy, p->seg_len, nseg.p);
        GNNAGG_HIP(hipGetLastError());
        GNNAGG_HIP(hipMalloc((void **)&p->segbase, sizeof(int64_t) * ((size_t)p->nheavy + 1)));
        size_t tmp_bytes = 0;
        GNNAGG_HIP(hipcub::DeviceScan::ExclusiveSum(nullptr, tmp_bytes, nseg.p, p->segbase, (int)p->nheavy + 1, st));
        DevBuf<char> tmp;
        GNNAGG_HIP(tmp.alloc(std::max<size_t>(tmp_bytes, 1)));
        GNNAGG_HIP(hipcub::DeviceScan::ExclusiveSum(tmp.p, tmp_bytes, nseg.p, p->segbase, (int)p->nheavy + 1, st));
        GNNAGG_HIP(hipMemcpyAsync(&p->nseg, p->segbase + p->nheavy, sizeof(int64_t), hipMemcpyDeviceToHost, st));
        GNNAGG_HIP(hipStreamSynchronize(st));
        GNNAGG_HIP(hipMalloc((void **)&p->seg_start, sizeof(int64_t) * (size_t)p->nseg));
        GNNAGG_HIP(hipMalloc((void **)&p->seg_n, sizeof(int32_t) * (size_t)p->nseg));
        hipLaunchKernelGGL(heavy_expand_kernel, dim3(grid_for(p->nseg, 256)), dim3(256), 0, st, p->rowptr, p->perm,
                           p->segbase, (int)p->nheavy, p->nseg, p->seg_len, p->seg_start, p->seg_n);
        GNNAGG_HIP(hipGetLastError());
        GNNAGG_HIP(hipStreamSynchronize(st));
    }
    guard.p = nullptr;
    *plan_out = p;
    return GNNAGG_OK;
}

extern "C" int gnnagg_plan_destroy(gnnagg_plan *plan) {
    if (!plan) return GNNAGG_OK;
    GNNAGG_HIP(hipDeviceSynchronize());
    plan_free(plan);
    return GNNAGG_OK;
}

extern "C" int gnnagg_plan_info(const gnnagg_plan *plan, int64_t *info) {
    GNNAGG_REQUIRE(plan && info, "null plan/info");
    info[0] = plan->rows;
    info[1] = plan->cols;
    info[2] = plan->nnz;
    info[3] = plan->nheavy;
    info[4] = plan->nseg;
    info[5] = plan->seg_len;
    info[6] = plan->nempty;
    info[7] = plan->max_deg;
    return GNNAGG_OK;
}

extern "C" int gnnagg_plan_spmm_f32(gnnagg_plan *plan, const float *value, const float *mat, float *out, int64_t feat,
                                    int accumulate, void *stream) {
    GNNAGG_REQUIRE(plan, "null plan");
    GNNAGG_REQUIRE(feat >= 0, "negative feature width");
    if (plan->rows == 0 || feat == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(out, "null out");
    GNNAGG_REQUIRE(plan->nnz == 0 || (value && mat), "null value/mat");
    if (int rc = check_feat(feat)) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);

    if (plan->nseg > 0 && plan->partial_feat < feat) {
        GNNAGG_HIP(hipDeviceSynchronize());
        (void)hipFree(plan->partial);
        plan->partial = nullptr;
        plan->partial_feat = 0;
        GNNAGG_HIP(hipMalloc((void **)&plan->partial, sizeof(float) * (size_t)plan->nseg * (size_t)feat));
        plan->partial_feat = feat;
    }

    // the scratch of segment sums comes from hipMalloc (256-byte aligned) and has row
    // stride `feat`, so it never lowers the vector width chosen for mat/out
    const int vec = pick_vec(feat, mat, out);
    const int64_t nrow_tasks = plan->rows - plan->nheavy - (accumulate ? plan->nempty : 0);
    const bool prof = plan->profile;
    if (prof) {
        plan->profile_valid = false;
        GNNAGG_HIP(hipEventRecord(plan->ev[0], st));
    }
    for (int64_t f_base = 0; f_base < feat;) {
        const Shape s = pick_shape(vec, feat - f_base);
        if (plan->nseg > 0) {
            SpmmArgs a{};
            a.seg_start = plan->seg_start;
            a.seg_len = plan->seg_n;
            a.col = plan->col32;
            a.val = value;
            a.x = mat;
            a.dst = plan->partial;
            a.ntasks = plan->nseg;
            a.feat = (int)feat;
            a.f_base = (int)f_base;
            GNNAGG_HIP((dispatch_tasks<int32_t, kSegments>(s, a, 1, st)));
            ReduceArgs r{};
            r.heavy_row = plan->perm;
            r.heavy_segbase = plan->segbase;
            r.partial = plan->partial;
            r.out = out;
            r.nheavy = (int)plan->nheavy;
            r.feat = (int)feat;
            r.f_base = (int)f_base;
            r.accumulate = accumulate;
            GNNAGG_HIP(dispatch_reduce(s, r, st));
        }
        if (nrow_tasks > 0) {
            SpmmArgs a{};
            a.rowptr = plan->rowptr;
            a.perm = plan->perm + plan->nheavy;
            a.col = plan->col32;
            a.val = value;
            a.x = mat;
            a.dst = out;
            a.ntasks = nrow_tasks;
            a.feat = (int)feat;
            a.f_base = (int)f_base;
            a.accumulate = accumulate;
            const bool first_tile = prof && f_base == 0;
            if (first_tile) GNNAGG_HIP(hipEventRecord(plan->ev[1], st));
            GNNAGG_HIP((dispatch_tasks<int32_t, kRowsPermuted>(s, a, plan->rows_per_group, st)));
            if (first_tile) {
                GNNAGG_HIP(hipEventRecord(plan->ev[2], st));
                plan->profile_valid = true;
            }
        }
        f_base += s.width();
    }
    if (prof) GNNAGG_HIP(hipEventRecord(plan->ev[3], st));
    return GNNAGG_OK;
}

extern "C" int gnnagg_plan_profile(gnnagg_plan *plan, int enable) {
    GNNAGG_REQUIRE(plan, "null plan");
    if (enable) {
        for (hipEvent_t &e : plan->ev)
            if (!e) GNNAGG_HIP(hipEventCreate(&e));
    }
    plan->profile = enable != 0;
    plan->profile_valid = false;
    return GNNAGG_OK;
}

extern "C" int gnnagg_plan_profile_read(gnnagg_plan *plan, double *ms) {
    GNNAGG_REQUIRE(plan && ms, "null plan/ms");
    ms[0] = ms[1] = -1.0;
    if (!plan->profile || !plan->ev[3]) return GNNAGG_OK;
    GNNAGG_HIP(hipEventSynchronize(plan->ev[3]));
    float t = 0.0f;
    if (plan->profile_valid) {
        GNNAGG_HIP(hipEventElapsedTime(&t, plan->ev[1], plan->ev[2]));
        ms[0] = t;
    }
    GNNAGG_HIP(hipEventElapsedTime(&t, plan->ev[0], plan->ev[3]));
    ms[1] = t;
    return GNNAGG_OK;
}
