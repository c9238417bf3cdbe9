// Host side of the SpMM entry points: launch-shape selection, the direct (plan-less)
// path, and the cached degree-binned plan.  gfx950 only.
#include <algorithm>
#include <atomic>
#include <mutex>
#include <new>
#include <type_traits>
#include <vector>

#include "common.h"
#include "sort.h"
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

// (rows of up to 64 floats would fit 16 lanes, but measured on MI355X 32 lanes per row are 7-8 % faster at every
// such width -- 16, 20, 40, 48, 64 floats -- so the narrowest shape picked is 32 x 1)
constexpr int kShapes[][2] = {{32, 1}, {64, 1}, {64, 2}, {64, 3}, {64, 4}, {64, 5}, {64, 6}, {64, 8}};
constexpr int kNumShapes = sizeof(kShapes) / sizeof(kShapes[0]);
// every (lanes, loads) pair the row kernel is instantiated for; a plan's options may name one of them
constexpr int kAllShapes[][2] = {{16, 1}, {16, 2}, {32, 1}, {16, 3}, {32, 2}, {64, 1}, {64, 2},
                                 {64, 3}, {64, 4}, {64, 5}, {64, 6}, {64, 8}};

// widest vector access that every row of x and dst allows: base addresses and row strides
// (in floats; rows back to back when the stride is the width) must be multiples of it
int pick_vec(int64_t feat, const void *x, const void *dst, int64_t ldx, int64_t ldd) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dst) |
                           (uintptr_t)(ldx * 4) | (uintptr_t)(ldd * 4);
    if (feat % 4 == 0 && bits % 16 == 0) return 4;
    if (feat % 2 == 0 && bits % 8 == 0) return 2;
    return 1;
}
int pick_vec(int64_t feat, const void *x, const void *dst) { return pick_vec(feat, x, dst, feat, feat); }

bool shape_exists(int lanes, int loads) {
    for (const auto &sh : kAllShapes)
        if (sh[0] == lanes && sh[1] == loads) return true;
    return false;
}

Shape pick_shape(int vec, int64_t feat_left, int lanes = 0, int loads = 0) {
    if (lanes > 0 && loads > 0) return Shape{vec, lanes, loads};  // the plan's options name the shape
    for (int i = 0; i < kNumShapes; ++i) {
        Shape s{vec, kShapes[i][0], kShapes[i][1]};
        if (s.width() >= feat_left) return s;
    }
    return Shape{vec, kShapes[kNumShapes - 1][0], kShapes[kNumShapes - 1][1]};
}

// How the rows of one launch are handed to blocks: `rpg` rows per lane group in the middle region, `tail_rpg` in the
// tail region (the last `tail_tasks` tasks; 0: none).  Fills the region fields of `args`; returns the block count.
struct Regions {
    int rpg, tail_rpg;
    int64_t tail_tasks;
};

int64_t lay_out_blocks(SpmmArgs &args, int gpb, Regions r) {
    r.rpg = std::min(std::max(r.rpg, 1), kMaxRowsPerGroup);
    r.tail_rpg = std::min(std::max(r.tail_rpg, 1), kMaxRowsPerGroup);
    if (args.head_tasks > args.ntasks) args.head_tasks = args.ntasks;
    int64_t tail = std::min(std::max<int64_t>(r.tail_tasks, 0), args.ntasks - args.head_tasks);
    if (r.tail_rpg == r.rpg) tail = 0;  // one region does
    args.tail_first = args.ntasks - tail;
    args.tasks_per_block = gpb * r.rpg;
    args.tail_tasks_per_block = gpb * r.tail_rpg;
    const int64_t head_blocks = (args.head_tasks + gpb - 1) / gpb;
    const int64_t mid_blocks = (args.tail_first - args.head_tasks + args.tasks_per_block - 1) / args.tasks_per_block;
    const int64_t tail_blocks = (tail + args.tail_tasks_per_block - 1) / args.tail_tasks_per_block;
    // rows in their natural order: the blocks that look for the long rows come first (args.scan_rows rows a group)
    int64_t scan_blocks = 0;
    if (args.long_len > 0 && args.scan_rows > 0)
        scan_blocks = (args.ntasks + (int64_t)args.scan_rows * gpb - 1) / ((int64_t)args.scan_rows * gpb);
    else
        args.long_len = 0;
    if (head_blocks + mid_blocks + tail_blocks + scan_blocks > 0x7fffffffll) return -1;
    args.head_blocks = (int)head_blocks;
    args.mid_blocks = (int)mid_blocks;
    args.scan_blocks = (int)scan_blocks;
    return head_blocks + mid_blocks + tail_blocks + scan_blocks;
}

template <int VEC, int LPR, int NCH, typename IdxT, int MODE, int SRC = kSrcDense>
hipError_t launch_tasks(const SpmmArgs &a, Regions r, hipStream_t stream) {
    constexpr int GPB = 256 / LPR;
    SpmmArgs args = a;
    const int64_t nblocks = lay_out_blocks(args, GPB, r);
    if (nblocks == 0) return hipSuccess;
    if (nblocks < 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL((spmm_tasks_kernel<VEC, LPR, NCH, IdxT, MODE, SRC>), dim3((unsigned)nblocks), dim3(256), 0,
                       stream, args);
    return hipGetLastError();
}

// Packed source rows (16-byte lanes, one load per lane): widths 32 / 64 -> 16 lanes, 128 -> 32, 256 -> 64.
hipError_t launch_packed(const SpmmArgs &a, Regions r, hipStream_t stream) {
    if (a.feat > 128) return launch_tasks<4, 64, 1, int32_t, kRowsPlanned, kSrcPacked>(a, r, stream);
    if (a.feat > 64) return launch_tasks<4, 32, 1, int32_t, kRowsPlanned, kSrcPacked>(a, r, stream);
    return launch_tasks<4, 16, 1, int32_t, kRowsPlanned, kSrcPacked>(a, r, stream);
}

template <int VEC, typename IdxT, int MODE, int SRC = kSrcDense>
hipError_t dispatch_shape(const Shape &s, const SpmmArgs &a, Regions rpg, hipStream_t st) {
#define GNNAGG_CASE(L, N) \
    if (s.lpr == L && s.nch == N) return launch_tasks<VEC, L, N, IdxT, MODE, SRC>(a, rpg, st)
    GNNAGG_CASE(16, 1);
    GNNAGG_CASE(16, 2);
    GNNAGG_CASE(32, 1);
    GNNAGG_CASE(16, 3);
    GNNAGG_CASE(32, 2);
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

// The block-per-row kernel needs more than the default 64 KB of LDS per block; the limit
// is a per-device attribute of each instantiation (set when a plan with such rows is made).
template <int VEC, int NL>
hipError_t allow_long_rows_lds() {
    return hipFuncSetAttribute(reinterpret_cast<const void *>(spmm_long_rows_kernel<VEC, NL>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLongSmemBytes);
}

template <int VEC>
hipError_t allow_long_rows_lds_for_vec() {
    hipError_t e = allow_long_rows_lds<VEC, 1>();
    if (e == hipSuccess) e = allow_long_rows_lds<VEC, 2>();
    if (e == hipSuccess) e = allow_long_rows_lds<VEC, 4>();
    if (e == hipSuccess) e = allow_long_rows_lds<VEC, 8>();
    return e;
}

template <int FW>
hipError_t allow_long_rows_lds_fixed_width() {
    return hipFuncSetAttribute(reinterpret_cast<const void *>(spmm_long_rows_kernel<4, 8, FW>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLongSmemBytes);
}

// the block-per-row kernel uses more than 64 KB of dynamic LDS: every instance has to be told
hipError_t enable_long_rows_lds() {
    hipError_t e = allow_long_rows_lds_for_vec<4>();
    if (e == hipSuccess) e = allow_long_rows_lds_for_vec<2>();
    if (e == hipSuccess) e = allow_long_rows_lds_for_vec<1>();
    if (e == hipSuccess) e = allow_long_rows_lds_fixed_width<16>();
    if (e == hipSuccess) e = allow_long_rows_lds_fixed_width<32>();
    if (e == hipSuccess) e = allow_long_rows_lds_fixed_width<64>();
    return e;
}

// What a stored element costs a row of the block-per-row kernel, by tile width (ns, measured on a 200 000-element
// row): the chain itself does not depend on the width, but a wider tile means a shorter chunk (a tile buffer holds
// 6144 floats), and with two chunks in flight a short chunk no longer covers the memory round trip.  Two blocks
// share a compute unit; they slow each other down by about what the second one adds, so the model counts one.
struct LongTileCost { int tile; double ns_per_element; };
constexpr LongTileCost kLongTileCosts[] = {{16, 5.5}, {32, 6.8}, {64, 14.7}};
constexpr double kComputeUnits = 256.0;

template <int VEC>
hipError_t launch_long_rows(const LongArgs &a, int64_t nrows, int64_t longest, int64_t elems, hipStream_t st) {
    LongArgs args = a;
    // Every feature's chain is its own, so a row can be cut along the features into tiles of 16 .. 64 floats, one
    // block each.  The launch lasts as long as the longest row's block, or as long as all blocks take on all compute
    // units (rows are handed out longest first): the tile width is the one for which the larger of the two is smallest.
    int tile = kLongTileCosts[0].tile;
    double best = 0.0;
    for (const LongTileCost &c : kLongTileCosts) {
        const double tiles = (double)((a.feat + c.tile - 1) / c.tile);
        const double longest_row = (double)longest * c.ns_per_element;
        const double all_rows = (double)elems * tiles * c.ns_per_element / kComputeUnits;
        const double lasts = std::max(longest_row, all_rows);
        if (best == 0.0 || lasts < best) {
            best = lasts;
            tile = c.tile;
        }
    }
    if (tile > a.feat) tile = a.feat;
    args.tile = tile;
    const int vpr = tile / VEC;
    int chunk = kLongMaxChunk;
    if (chunk * vpr > 256 * kLongLoads) chunk = 256 * kLongLoads / vpr;
    if (chunk * tile > kLongTileFloats) chunk = kLongTileFloats / tile;
    chunk &= ~3;  // the chain reads a chunk's elements four at a time, 16-byte aligned
    args.chunk = chunk;
    const unsigned tiles = (unsigned)((a.feat + tile - 1) / tile);
    const int slots = chunk * vpr;  // vectors of a whole chunk; 256 threads fetch them in NL rounds
    args.tiles = (int)tiles;
    if (nrows * (int64_t)tiles >= (int64_t(1) << 31)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)(nrows * (int64_t)tiles));
    const dim3 block((unsigned)(kLongFetchThreads + 64));  // fetch waves + the chain wave
    if (VEC == 4 && slots > 1024 && a.feat % tile == 0 && tile >= 16 && (tile & (tile - 1)) == 0) {
        // every tile has the same power-of-two width: the instance that knows it at compile time
#define GNNAGG_LONG_FIXED(W)                                                                                     \
    if (tile == W)                                                                                               \
        hipLaunchKernelGGL((spmm_long_rows_kernel<4, 8, W>), grid, block, kLongSmemBytes, st, args)
        GNNAGG_LONG_FIXED(16);
        GNNAGG_LONG_FIXED(32);
        GNNAGG_LONG_FIXED(64);
#undef GNNAGG_LONG_FIXED
        return hipGetLastError();
    }
    if (slots <= 256) hipLaunchKernelGGL((spmm_long_rows_kernel<VEC, 1>), grid, block, kLongSmemBytes, st, args);
    else if (slots <= 512) hipLaunchKernelGGL((spmm_long_rows_kernel<VEC, 2>), grid, block, kLongSmemBytes, st, args);
    else if (slots <= 1024) hipLaunchKernelGGL((spmm_long_rows_kernel<VEC, 4>), grid, block, kLongSmemBytes, st, args);
    else hipLaunchKernelGGL((spmm_long_rows_kernel<VEC, 8>), grid, block, kLongSmemBytes, st, args);
    return hipGetLastError();
}

template <typename IdxT, int MODE>
hipError_t dispatch_tasks(const Shape &s, const SpmmArgs &a, Regions rpg, hipStream_t st) {
    if (s.vec == 4) return dispatch_shape<4, IdxT, MODE>(s, a, rpg, st);
    if (s.vec == 2) return dispatch_shape<2, IdxT, MODE>(s, a, rpg, st);
    return dispatch_shape<1, IdxT, MODE>(s, a, rpg, st);
}

// ------------------------------------------------------------------ plan kernels
// Degree class of a row: class c (c < kEmptyClass) holds the rows with
// ceil(log2(length)) == kEmptyClass - 1 - c, i.e. classes run from the LONGEST rows
// (small c) to single-element rows; the last class holds the empty rows.
constexpr int kEmptyClass = 41;
constexpr int kNumClasses = kEmptyClass + 1;
constexpr int kClassBits = 6;

struct ClassifyOut {
    unsigned long long class_count[kNumClasses];
    unsigned long long max_deg;
    unsigned int bad_rowptr;  // rowptr decreasing somewhere
    unsigned int bad_col;     // a column index outside [0, cols)
};

__host__ __device__ __forceinline__ int degree_class(int64_t deg) {
    if (deg <= 0) return kEmptyClass;
    int clog = 0;  // ceil(log2(deg))
    while ((int64_t(1) << clog) < deg) ++clog;
    return kEmptyClass - 1 - clog;
}

// (a grid of at most kClassifyBlocks blocks walks the rows: what every block adds to the handful of global counters
// at its end is a same-address atomic, and one per 256 rows made this kernel last 0.66 ms at 7 M rows)
constexpr int kClassifyBlocks = 1024;

__global__ __launch_bounds__(256) void classify_rows_kernel(const int64_t *__restrict__ rowptr, int rows,
                                                            uint32_t *__restrict__ key, int32_t *__restrict__ rowid,
                                                            ClassifyOut *__restrict__ out) {
    __shared__ unsigned int hist[kNumClasses];
    __shared__ unsigned long long smax;
    if (threadIdx.x < kNumClasses) hist[threadIdx.x] = 0;
    if (threadIdx.x == 0) smax = 0;
    __syncthreads();
    const int lane = (int)threadIdx.x & 63;
    unsigned long long longest = 0;
    const int64_t stride = (int64_t)gridDim.x * 256;
    // (every thread of a block makes the same number of rounds: the ballots below want whole waves)
    for (int64_t base = (int64_t)blockIdx.x * 256; base < rows; base += stride) {
        const int64_t r = base + (int64_t)threadIdx.x;
        int c = -1;  // the row's class; -1: no row, or a row whose rowptr runs backwards
        if (r < rows) {
            const int64_t d = rowptr[r + 1] - rowptr[r];
            if (d < 0) {
                atomicOr(&out->bad_rowptr, 1u);
                key[r] = (uint32_t)kEmptyClass;
            } else {
                c = degree_class(d);
                key[r] = (uint32_t)c;
                if ((unsigned long long)d > longest) longest = (unsigned long long)d;
            }
            rowid[r] = (int32_t)r;
        }
        // per wave one LDS atomic per class that occurs in it (its lanes found by ballots over the class's bits)
        uint64_t same = __builtin_amdgcn_ballot_w64(c >= 0);
#pragma unroll
        for (int b = 0; b < kClassBits; ++b) {
            const uint64_t has = __builtin_amdgcn_ballot_w64(((c >> b) & 1) != 0);
            same &= ((c >> b) & 1) ? has : ~has;
        }
        if (c >= 0 && (same & ((uint64_t(1) << lane) - 1)) == 0) atomicAdd(&hist[c], (unsigned int)__popcll(same));
    }
    longest = wave_max_u64(longest);
    if (lane == 0 && longest) atomicMax(&smax, longest);
    __syncthreads();
    if (threadIdx.x < kNumClasses && hist[threadIdx.x])
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

// task[t] = (first element, length, row) of the t-th row of the degree-ordered schedule
__global__ __launch_bounds__(256) void build_tasks_kernel(const int64_t *__restrict__ rowptr,
                                                          const int32_t *__restrict__ perm, int rows,
                                                          RowTask *__restrict__ task) {
    const int t = (int)blockIdx.x * 256 + (int)threadIdx.x;
    if (t >= rows) return;
    const int r = perm[t];
    const int64_t b = rowptr[r];
    RowTask d;
    d.start = b;
    d.len = (int32_t)(rowptr[r + 1] - b);
    d.row = r;
    task[t] = d;
}

}  // namespace
}  // namespace gnnagg

using namespace gnnagg;

struct gnnagg_plan {
    int64_t rows = 0, cols = 0, nnz = 0;
    int huge_thresh = 0;      // rows longer than this run in the block-per-row kernel
    int64_t nhuge = 0;        // such rows (the first nhuge tasks)
    int64_t huge_elems = 0;   // the stored elements in them (exact for up to 65536 such rows, else the class counts x the classes' upper ends)
    int long_thresh = 0;      // rows longer than this get a lane group of their own (head region)
    int64_t nlong = 0;        // such rows, the huge ones included (the first nlong tasks)
    int64_t nempty = 0;       // rows with no stored element (the last nempty entries of perm)
    int64_t max_deg = 0;
    int device = 0;
    int32_t *col32 = nullptr;   // [nnz]
    RowTask *task = nullptr;    // [rows] rows by degree class, longest first; ascending row id inside a class
    int64_t nshort = 0;       // rows of 1 .. kShortRowLen elements (the last non-empty tasks)
    // (measured on MI355X: 1, 2, 4, 8 or 16 rows per group move the boundary products by +-2 % and the local product by
    // less -- the memory system, not the hand-out of rows, is what bounds them; 2 is the best all round)
    int rows_per_group = 2;        // rows a lane group walks in the middle region
    int short_rows_per_group = 2;  // ... and in the tail region of the shortest rows (equal: one region)
    int lanes = 0, loads = 0;      // launch shape named by the options (0: chosen from the width)
    std::atomic<bool> busy{false}; // a call is being enqueued (the plan's events and side stream are in use)
    hipStream_t side = nullptr;          // the block-per-row kernel runs here, next to the main launch
    hipEvent_t fork = nullptr, join = nullptr;
    bool profile = false;
    bool profile_valid = false;
    hipEvent_t ev[4] = {nullptr, nullptr, nullptr, nullptr};  // call begin, main-kernel begin/end, call end
};

extern "C" int gnnagg_abi_version(void) { return GNNAGG_ABI_VERSION; }

extern "C" const char *gnnagg_last_error(void) { return last_error_slot().c_str(); }

// the plan-less operator's own handling of long rows (see gnnagg_spmm_csr_f32)
constexpr int64_t kScanMinRows = 16384;   // smaller matrices: one region, as they come
// (measured on MI355X, 2.45 M rows / 122 M elements at F = 100 and 7 M rows / 102 M elements at F = 128, ms:
//  no scanning 9.44 / 9.91; (length 256, 512 rows a group) 9.91 / 8.65; (256, 128) 7.93 / 8.68; (128, 128) 7.92 / 8.55;
//  (64, 64) 8.01 / 8.43; (32, 64) 9.15 / 8.46 -- the plan's own launch takes 7.9 / 7.8)
constexpr int kScanLongLen = 64;          // rows above this go to the scanning blocks
constexpr int kScanRowsPerGroup = 64;     // rows of rowptr a scanning lane group walks

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
    // col/value/mat may be null only for a matrix without stored elements, which this
    // entry point cannot tell (nnz is not an argument); they are not dereferenced then
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
        // No plan orders the rows by length here, so on a matrix of some size the launch's first blocks walk rowptr
        // and run the rows above the plan's own long-row threshold themselves: the longest chains start at once,
        // spread over the device, instead of wherever their row number puts them.  Allocates nothing.
        if (sparse_rows >= kScanMinRows) {
            a.long_len = kScanLongLen;
            a.scan_rows = kScanRowsPerGroup;
        }
        GNNAGG_HIP((dispatch_tasks<int64_t, kRowsNatural>(s, a, Regions{4, 4, 0}, st)));
        f_base += s.width();
    }
    return GNNAGG_OK;
}

static void plan_free(gnnagg_plan *p) {
    if (!p) return;
    (void)hipFree(p->col32);
    (void)hipFree(p->task);
    if (p->fork) (void)hipEventDestroy(p->fork);
    if (p->join) (void)hipEventDestroy(p->join);
    if (p->side) (void)hipStreamDestroy(p->side);
    for (hipEvent_t e : p->ev)
        if (e) (void)hipEventDestroy(e);
    delete p;
}

// Plans handed to gnnagg_plan_destroy wait here until the next plan is created: freeing device memory synchronises
// the whole device (and is illegal while a stream is being captured), which a destructor run by a garbage collector
// in the middle of a training step must not do.  Plan creation is set-up work that synchronises anyway.
static std::mutex retired_mutex;
static std::vector<gnnagg_plan *> retired_plans;

static void free_retired_plans(int device) {
    std::vector<gnnagg_plan *> mine;
    {
        std::lock_guard<std::mutex> hold(retired_mutex);
        for (size_t i = 0; i < retired_plans.size();) {
            if (retired_plans[i]->device == device) {
                mine.push_back(retired_plans[i]);
                retired_plans[i] = retired_plans.back();
                retired_plans.pop_back();
            } else {
                ++i;
            }
        }
    }
    if (mine.empty()) return;
    (void)hipDeviceSynchronize();  // whatever still reads their arrays finishes first
    for (gnnagg_plan *p : mine) plan_free(p);
}

extern "C" int gnnagg_plan_create(const int64_t *rowptr, const int64_t *col, int64_t rows, int64_t cols, int64_t nnz,
                                  void *stream, gnnagg_plan **plan_out) {
    return gnnagg_plan_create_ex(rowptr, col, rows, cols, nnz, nullptr, stream, plan_out);
}

// rows of at most this many elements form the tail region (more rows per lane group)
constexpr int kShortRowLen = 8;

extern "C" int gnnagg_plan_create_ex(const int64_t *rowptr, const int64_t *col, int64_t rows, int64_t cols, int64_t nnz,
                                     const gnnagg_plan_options *options, void *stream, gnnagg_plan **plan_out) {
    GNNAGG_REQUIRE(plan_out, "null plan_out");
    *plan_out = nullptr;
    gnnagg_plan_options opt{};
    if (options) opt = *options;
    GNNAGG_REQUIRE(opt.long_row_threshold >= 0 && opt.block_row_threshold >= 0 && opt.rows_per_group >= 0 &&
                       opt.short_rows_per_group >= 0 && opt.rows_per_group <= kMaxRowsPerGroup &&
                       opt.short_rows_per_group <= kMaxRowsPerGroup,
                   "plan options: thresholds must not be negative, rows per group lie in 0 .. %d", kMaxRowsPerGroup);
    GNNAGG_REQUIRE(opt.reserved[0] == 0 && opt.reserved[1] == 0, "plan options: the reserved fields must be 0");
    GNNAGG_REQUIRE((opt.lanes_per_row == 0 && opt.loads_per_lane == 0) || shape_exists(opt.lanes_per_row, opt.loads_per_lane),
                   "plan options: no row kernel with %d lanes per row and %d loads per lane", opt.lanes_per_row,
                   opt.loads_per_lane);
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
    p->long_thresh = opt.long_row_threshold > 0 ? opt.long_row_threshold : 256;
    // A row is handed to the block-per-row kernel only when its chain, fed by one lane
    // group (a few elements per microsecond), would outlast the whole launch: that
    // length grows with the matrix, about nnz / 4096 (measured on MI355X), floor 2048 (below it the
    // block-per-row kernel, 50 .. 85 stored elements per microsecond and row, no longer pays).
    int64_t huge_default = std::max<int64_t>(2048, nnz / 4096);
    if (huge_default > (1 << 30)) huge_default = 1 << 30;
    p->huge_thresh = opt.block_row_threshold > 0 ? std::max(opt.block_row_threshold, p->long_thresh) : (int)huge_default;
    if (opt.rows_per_group > 0) p->rows_per_group = opt.rows_per_group;
    if (opt.short_rows_per_group > 0) p->short_rows_per_group = opt.short_rows_per_group;
    p->lanes = opt.lanes_per_row;
    p->loads = opt.loads_per_lane;
    GNNAGG_HIP(hipGetDevice(&p->device));
    free_retired_plans(p->device);

    // rowptr end points (host check; also forces the inputs to be ready)
    int64_t ends[2] = {0, 0};
    GNNAGG_HIP(hipMemcpyAsync(&ends[0], rowptr, sizeof(int64_t), hipMemcpyDeviceToHost, st));
    GNNAGG_HIP(hipMemcpyAsync(&ends[1], rowptr + rows, sizeof(int64_t), hipMemcpyDeviceToHost, st));
    GNNAGG_HIP(hipStreamSynchronize(st));
    GNNAGG_REQUIRE(ends[0] == 0 && ends[1] == nnz, "rowptr[0]=%lld, rowptr[rows]=%lld do not match nnz=%lld",
                   (long long)ends[0], (long long)ends[1], (long long)nnz);

    GNNAGG_HIP(hipMalloc((void **)&p->col32, sizeof(int32_t) * (size_t)std::max<int64_t>(nnz, 1)));
    GNNAGG_HIP(hipMalloc((void **)&p->task, sizeof(RowTask) * (size_t)std::max<int64_t>(rows, 1)));

    DevBuf<ClassifyOut> d_out;
    GNNAGG_HIP(d_out.alloc(1));
    GNNAGG_HIP(hipMemsetAsync(d_out.p, 0, sizeof(ClassifyOut), st));

    ClassifyOut h_out{};
    if (rows > 0) {
        DevBuf<uint32_t> key_in, key_out;
        DevBuf<int32_t> row_in, perm;
        GNNAGG_HIP(key_in.alloc((size_t)rows));
        GNNAGG_HIP(key_out.alloc((size_t)rows));
        GNNAGG_HIP(row_in.alloc((size_t)rows));
        GNNAGG_HIP(perm.alloc((size_t)rows));
        hipLaunchKernelGGL(classify_rows_kernel, dim3(std::min<unsigned>(grid_for(rows, 256), kClassifyBlocks)), dim3(256), 0, st, rowptr, (int)rows,
                           key_in.p, row_in.p, d_out.p);
        GNNAGG_HIP(hipGetLastError());
        if (nnz > 0) {
            const unsigned g = (unsigned)std::min<int64_t>((nnz + 255) / 256, 1 << 20);
            hipLaunchKernelGGL(narrow_cols_kernel, dim3(g), dim3(256), 0, st, col, nnz, cols, p->col32, d_out.p);
            GNNAGG_HIP(hipGetLastError());
        }
        // stable sort of the rows by class: ascending row id inside a class
        bool in_b = false;
        if (int rc = sort_pairs_u32(key_in.p, key_out.p, reinterpret_cast<uint32_t *>(row_in.p),
                                    reinterpret_cast<uint32_t *>(perm.p), rows, kClassBits, st, &in_b))
            return rc;
        const int32_t *order = in_b ? perm.p : row_in.p;
        GNNAGG_HIP(hipMemcpyAsync(&h_out, d_out.p, sizeof(ClassifyOut), hipMemcpyDeviceToHost, st));
        GNNAGG_HIP(hipStreamSynchronize(st));
        if (!h_out.bad_rowptr && h_out.max_deg < (1ull << 31)) {  // row lengths are only meaningful for a monotone rowptr
            hipLaunchKernelGGL(build_tasks_kernel, dim3(grid_for(rows, 256)), dim3(256), 0, st, rowptr, order,
                               (int)rows, p->task);
            GNNAGG_HIP(hipGetLastError());
            GNNAGG_HIP(hipStreamSynchronize(st));  // perm is released on scope exit
        }
        GNNAGG_HIP(hipStreamSynchronize(st));
    }
    GNNAGG_REQUIRE(!h_out.bad_rowptr, "rowptr is not non-decreasing");
    GNNAGG_REQUIRE(!h_out.bad_col, "a column index lies outside [0, %lld)", (long long)cols);
    p->nempty = (int64_t)h_out.class_count[kEmptyClass];
    p->max_deg = (int64_t)h_out.max_deg;
    if (p->max_deg >= (int64_t(1) << 31))
        return fail(GNNAGG_ERR_UNSUPPORTED, "a row holds %lld stored elements (limit 2^31-1)", (long long)p->max_deg);
    // rows strictly longer than long_thresh: whole classes above the threshold's class
    const int thresh_class = degree_class(p->long_thresh);
    for (int c = 0; c < thresh_class; ++c) p->nlong += (int64_t)h_out.class_count[c];
    const int huge_class = degree_class(p->huge_thresh);
    for (int c = 0; c < huge_class; ++c) {
        p->nhuge += (int64_t)h_out.class_count[c];
        // class c holds the rows of ceil(log2(length)) == kEmptyClass - 1 - c
        const int64_t upper = std::min<int64_t>(int64_t(1) << (kEmptyClass - 1 - c), p->max_deg);
        p->huge_elems += (int64_t)h_out.class_count[c] * upper;
    }
    for (int c = degree_class(kShortRowLen); c < kEmptyClass; ++c) p->nshort += (int64_t)h_out.class_count[c];
    if (p->long_thresh < kShortRowLen) p->nshort = 0;  // (such rows sit in the head region then)
    if (p->nhuge > 0) {
        // the elements in those rows exactly, when the rows are few enough to look at (they head the schedule)
        if (p->nhuge <= 65536) {
            std::vector<RowTask> head((size_t)p->nhuge);
            GNNAGG_HIP(hipMemcpy(head.data(), p->task, head.size() * sizeof(RowTask), hipMemcpyDeviceToHost));
            p->huge_elems = 0;
            for (const RowTask &t : head) p->huge_elems += t.len;
        }
        GNNAGG_HIP(enable_long_rows_lds());
        GNNAGG_HIP(hipStreamCreateWithFlags(&p->side, hipStreamNonBlocking));
        GNNAGG_HIP(hipEventCreateWithFlags(&p->fork, hipEventDisableTiming));
        GNNAGG_HIP(hipEventCreateWithFlags(&p->join, hipEventDisableTiming));
    }

    guard.p = nullptr;
    *plan_out = p;
    return GNNAGG_OK;
}

extern "C" int gnnagg_plan_destroy(gnnagg_plan *plan) {
    if (!plan) return GNNAGG_OK;
    std::lock_guard<std::mutex> hold(retired_mutex);
    retired_plans.push_back(plan);
    return GNNAGG_OK;
}

extern "C" int gnnagg_plans_release(void) {
    int device = 0;
    GNNAGG_HIP(hipGetDevice(&device));
    free_retired_plans(device);
    return GNNAGG_OK;
}

extern "C" int gnnagg_plan_info(const gnnagg_plan *plan, int64_t *info) {
    GNNAGG_REQUIRE(plan && info, "null plan/info");
    info[0] = plan->rows;
    info[1] = plan->cols;
    info[2] = plan->nnz;
    info[3] = plan->nhuge;
    info[4] = plan->huge_thresh;
    info[5] = plan->nempty;
    info[6] = plan->max_deg;
    info[7] = plan->rows_per_group;
    info[8] = plan->nshort;
    info[9] = plan->short_rows_per_group;
    info[10] = plan->nlong;
    info[11] = plan->long_thresh;
    return GNNAGG_OK;
}

namespace gnnagg {
namespace {

// Marks a plan as in use for the duration of one enqueueing call (host side): a second call that arrives meanwhile
// is refused instead of re-recording the first one's events.
struct BusyGuard {
    gnnagg_plan *plan;
    bool mine;
    explicit BusyGuard(gnnagg_plan *p) : plan(p), mine(!p->busy.exchange(true, std::memory_order_acquire)) {}
    ~BusyGuard() {
        if (mine) plan->busy.store(false, std::memory_order_release);
    }
    BusyGuard(const BusyGuard &) = delete;
    BusyGuard &operator=(const BusyGuard &) = delete;
};

int plan_spmm(gnnagg_plan *plan, const float *value, const float *mat, int64_t ldx, float *out, int64_t ldd,
              int64_t feat, int accumulate, void *stream) {
    GNNAGG_REQUIRE(plan, "null plan");
    GNNAGG_REQUIRE(feat >= 0, "negative feature width");
    if (plan->rows == 0 || feat == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(out, "null out");
    GNNAGG_REQUIRE(plan->nnz == 0 || (value && mat), "null value/mat");
    if (int rc = check_feat(feat)) return rc;
    GNNAGG_REQUIRE(ldx >= feat && ldd >= feat && ldx < (int64_t(1) << 31) && ldd < (int64_t(1) << 31),
                   "row strides %lld / %lld must be at least the width %lld and below 2^31", (long long)ldx,
                   (long long)ldd, (long long)feat);
    hipStream_t st = static_cast<hipStream_t>(stream);
    BusyGuard in_use(plan);
    if (!in_use.mine)
        return fail(GNNAGG_ERR_INVALID, "this plan is in use by another call (two calls on one plan must not overlap: "
                                        "its events and side stream belong to one call at a time)");

    const int vec = pick_vec(feat, mat, out, ldx, ldd);
    // accumulate: empty rows keep their value, so they are not visited at all
    const int64_t nshort = plan->rows - plan->nlong - (accumulate ? plan->nempty : 0);
    // the tail region: the rows of at most kShortRowLen elements and, when every row is written, the empty ones
    const Regions regions{plan->rows_per_group, plan->short_rows_per_group,
                          plan->nshort + (accumulate ? 0 : plan->nempty)};
    if (plan->lanes > 0 && (int64_t)vec * plan->lanes * plan->loads < feat)
        return fail(GNNAGG_ERR_INVALID, "the plan's launch shape (%d lanes x %d loads x %d floats) does not cover %lld features",
                    plan->lanes, plan->loads, vec, (long long)feat);
    const bool prof = plan->profile;
    if (prof) {
        plan->profile_valid = false;
        GNNAGG_HIP(hipEventRecord(plan->ev[0], st));
    }
    if (plan->nhuge > 0) {
        // all feature tiles of the very long rows, one block each, on the plan's side
        // stream so that they run next to the main launch instead of in front of it
        GNNAGG_HIP(hipEventRecord(plan->fork, st));
        GNNAGG_HIP(hipStreamWaitEvent(plan->side, plan->fork, 0));
        LongArgs la{};
        la.task = plan->task;
        la.col = plan->col32;
        la.val = value;
        la.x = mat;
        la.dst = out;
        la.feat = (int)feat;
        la.ldx = (int)ldx;
        la.ldd = (int)ldd;
        la.accumulate = accumulate;
        if (vec == 4) GNNAGG_HIP(launch_long_rows<4>(la, plan->nhuge, plan->max_deg, plan->huge_elems, plan->side));
        else if (vec == 2) GNNAGG_HIP(launch_long_rows<2>(la, plan->nhuge, plan->max_deg, plan->huge_elems, plan->side));
        else GNNAGG_HIP(launch_long_rows<1>(la, plan->nhuge, plan->max_deg, plan->huge_elems, plan->side));
        GNNAGG_HIP(hipEventRecord(plan->join, plan->side));
    }
    for (int64_t f_base = 0; f_base < feat;) {
        const Shape s = pick_shape(vec, feat - f_base, plan->lanes, plan->loads);
        SpmmArgs a{};
        a.task = plan->task;
        a.col = plan->col32;
        a.val = value;
        a.x = mat;
        a.dst = out;
        a.feat = (int)feat;
        a.ldx = (int)ldx;
        a.ldd = (int)ldd;
        a.f_base = (int)f_base;
        a.accumulate = accumulate;
        // one launch over the rows, longest first; the rows above the long-row threshold
        // form the head region (one lane group per row).  The very longest rows went to
        // the block-per-row kernel above.
        if (plan->nlong + nshort - plan->nhuge > 0) {
            const bool timed = prof && f_base == 0;
            a.task = plan->task + plan->nhuge;
            a.ntasks = plan->nlong + nshort - plan->nhuge;
            a.head_tasks = plan->nlong - plan->nhuge;
            if (timed) GNNAGG_HIP(hipEventRecord(plan->ev[1], st));
            GNNAGG_HIP((dispatch_tasks<int32_t, kRowsPlanned>(s, a, regions, st)));
            if (timed) {
                GNNAGG_HIP(hipEventRecord(plan->ev[2], st));
                plan->profile_valid = true;
            }
        }
        f_base += s.width();
    }
    if (plan->nhuge > 0) GNNAGG_HIP(hipStreamWaitEvent(st, plan->join, 0));
    if (prof) GNNAGG_HIP(hipEventRecord(plan->ev[3], st));
    return GNNAGG_OK;
}

}  // namespace
}  // namespace gnnagg

extern "C" int gnnagg_plan_spmm_f32(gnnagg_plan *plan, const float *value, const float *mat, float *out, int64_t feat,
                                    int accumulate, void *stream) {
    return plan_spmm(plan, value, mat, feat, out, feat, feat, accumulate, stream);
}

extern "C" int gnnagg_plan_spmm_strided_f32(gnnagg_plan *plan, const float *value, const float *mat,
                                            int64_t mat_stride, float *out, int64_t out_stride, int64_t feat,
                                            int accumulate, void *stream) {
    return plan_spmm(plan, value, mat, mat_stride, out, out_stride, feat, accumulate, stream);
}

extern "C" int gnnagg_plan_spmm_two_sources_f32(gnnagg_plan *plan, const float *value, const float *mat,
                                                int64_t mat_stride, int64_t mat_rows, const float *mat2,
                                                int64_t mat2_stride, float *out, int64_t out_stride, int64_t feat,
                                                int accumulate, void *stream) {
    GNNAGG_REQUIRE(plan, "null plan");
    GNNAGG_REQUIRE(feat >= 0, "negative feature width");
    GNNAGG_REQUIRE(mat_rows >= 0 && mat_rows <= plan->cols, "the first source holds %lld rows, the matrix has %lld columns",
                   (long long)mat_rows, (long long)plan->cols);
    if (plan->rows == 0 || feat == 0) return GNNAGG_OK;
    if (int rc = check_feat(feat)) return rc;
    GNNAGG_REQUIRE(out, "null out");
    GNNAGG_REQUIRE(plan->nnz == 0 || (value && (mat || mat_rows == 0) && (mat2 || mat_rows == plan->cols)),
                   "null value/mat/mat2");
    GNNAGG_REQUIRE(mat_stride >= feat && mat2_stride >= feat && out_stride >= feat && mat_stride < (int64_t(1) << 31) &&
                       mat2_stride < (int64_t(1) << 31) && out_stride < (int64_t(1) << 31),
                   "row strides %lld / %lld / %lld must be at least the width %lld and below 2^31", (long long)mat_stride,
                   (long long)mat2_stride, (long long)out_stride, (long long)feat);
    // a source without rows is never addressed, but the surplus gathers of a row's last round read row 0 of the
    // first source: point it at the second one's rows then
    if (mat_rows == 0) mat = mat2;
    if (mat_rows == plan->cols) mat2 = mat, mat2_stride = mat_stride;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int vec = std::min(pick_vec(feat, mat, out, mat_stride, out_stride), pick_vec(feat, mat2, out, mat2_stride, out_stride));
    const Regions regions{plan->rows_per_group, plan->short_rows_per_group,
                          plan->nshort + (accumulate ? 0 : plan->nempty)};
    for (int64_t f_base = 0; f_base < feat;) {
        const Shape s = pick_shape(vec, feat - f_base);
        SpmmArgs a{};
        a.task = plan->task;  // every row runs in the lane-group kernel, the very longest included
        a.col = plan->col32;
        a.val = value;
        a.x = mat;
        a.ldx = (int)mat_stride;
        a.x2 = mat2;
        a.ldx2 = (int)mat2_stride;
        a.x_rows = (int)mat_rows;
        a.dst = out;
        a.ldd = (int)out_stride;
        a.feat = (int)feat;
        a.f_base = (int)f_base;
        a.accumulate = accumulate;
        a.ntasks = plan->rows - (accumulate ? plan->nempty : 0);
        a.head_tasks = plan->nlong;
        if (vec == 4) GNNAGG_HIP((dispatch_shape<4, int32_t, kRowsPlanned, kSrcDense2>(s, a, regions, st)));
        else if (vec == 2) GNNAGG_HIP((dispatch_shape<2, int32_t, kRowsPlanned, kSrcDense2>(s, a, regions, st)));
        else GNNAGG_HIP((dispatch_shape<1, int32_t, kRowsPlanned, kSrcDense2>(s, a, regions, st)));
        f_base += s.width();
    }
    return GNNAGG_OK;
}

// Local elements from dense fp32 rows, the rest of every row from a second source still in its exchange format.
static int plan_spmm_dense_then(gnnagg_plan *plan, const float *value, const int32_t *split, const float *mat,
                                int64_t mat_stride, int64_t mat_rows, const void *rows16, int64_t rows16_stride,
                                const uint8_t *packed, const float *params, const int32_t *row_code, int bits, float *out,
                                int64_t out_stride, int64_t feat, int accumulate, void *stream) {
    GNNAGG_REQUIRE(plan, "null plan");
    GNNAGG_REQUIRE(feat >= 0, "negative feature width");
    GNNAGG_REQUIRE(mat_rows >= 0 && mat_rows <= plan->cols, "the first source holds %lld rows, the matrix has %lld columns",
                   (long long)mat_rows, (long long)plan->cols);
    if (plan->rows == 0 || feat == 0) return GNNAGG_OK;
    if (int rc = check_feat(feat)) return rc;
    if (feat % 4 != 0)
        return fail(GNNAGG_ERR_UNSUPPORTED, "rows in an exchange format need a width that is a multiple of 4 (got %lld)",
                    (long long)feat);
    GNNAGG_REQUIRE(out && split, "null out/split");
    const bool quant = packed != nullptr;
    GNNAGG_REQUIRE(plan->nnz == 0 || (value && mat && (quant ? (params && row_code) : rows16 != nullptr)),
                   "null value/mat/second source");
    if (quant) GNNAGG_REQUIRE(bits == 2 || bits == 4 || bits == 8, "bits must be 2, 4 or 8 (got %d)", bits);
    GNNAGG_REQUIRE(mat_stride >= feat && mat_stride % 4 == 0 && mat_stride < (int64_t(1) << 31) && out_stride >= feat &&
                       out_stride % 4 == 0 && out_stride < (int64_t(1) << 31) &&
                       (quant || (rows16_stride >= feat && rows16_stride % 4 == 0 && rows16_stride < (int64_t(1) << 31))),
                   "row strides must be multiples of 4, at least the width and below 2^31");
    GNNAGG_REQUIRE((reinterpret_cast<uintptr_t>(mat) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 &&
                       (reinterpret_cast<uintptr_t>(rows16) & 7) == 0 && (reinterpret_cast<uintptr_t>(packed) & 3) == 0 &&
                       (reinterpret_cast<uintptr_t>(params) & 7) == 0,
                   "fp32 rows must be 16-byte aligned, bf16 rows and parameters 8-byte aligned, packed bytes 4-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const Regions regions{plan->rows_per_group, plan->short_rows_per_group,
                          plan->nshort + (accumulate ? 0 : plan->nempty)};
    for (int64_t f_base = 0; f_base < feat;) {
        const Shape s = pick_shape(4, feat - f_base);
        SpmmArgs a{};
        a.task = plan->task;  // every row runs in the lane-group kernel, the very longest included
        a.col = plan->col32;
        a.val = value;
        a.split = split;
        a.x = mat;
        a.ldx = (int)mat_stride;
        a.x_rows = (int)mat_rows;
        a.x2 = static_cast<const float *>(rows16);
        a.ldx2 = (int)rows16_stride;
        a.qdata = packed;
        a.qparams = params;
        a.qcode = row_code;
        a.qbits = bits;
        a.dst = out;
        a.ldd = (int)out_stride;
        a.feat = (int)feat;
        a.f_base = (int)f_base;
        a.accumulate = accumulate;
        a.ntasks = plan->rows - (accumulate ? plan->nempty : 0);
        a.head_tasks = plan->nlong;
        if (quant) GNNAGG_HIP((dispatch_shape<4, int32_t, kRowsPlanned, kSrcDenseThenQuant>(s, a, regions, st)));
        else GNNAGG_HIP((dispatch_shape<4, int32_t, kRowsPlanned, kSrcDenseThenBf16>(s, a, regions, st)));
        f_base += s.width();
    }
    return GNNAGG_OK;
}

extern "C" int gnnagg_plan_spmm_dense_then_bf16_f32(gnnagg_plan *plan, const float *value, const int32_t *split,
                                                    const float *mat, int64_t mat_stride, int64_t mat_rows,
                                                    const uint16_t *mat2_bf16, int64_t mat2_stride, float *out,
                                                    int64_t out_stride, int64_t feat, int accumulate, void *stream) {
    GNNAGG_REQUIRE(plan == nullptr || plan->nnz == 0 || mat2_bf16, "null mat2_bf16");
    return plan_spmm_dense_then(plan, value, split, mat, mat_stride, mat_rows, mat2_bf16, mat2_stride, nullptr, nullptr,
                                nullptr, 0, out, out_stride, feat, accumulate, stream);
}

extern "C" int gnnagg_plan_spmm_dense_then_quantized_f32(gnnagg_plan *plan, const float *value, const int32_t *split,
                                                         const float *mat, int64_t mat_stride, int64_t mat_rows,
                                                         const uint8_t *packed, const float *params,
                                                         const int32_t *row_code, int bits, float *out,
                                                         int64_t out_stride, int64_t feat, int accumulate, void *stream) {
    GNNAGG_REQUIRE(plan == nullptr || plan->nnz == 0 || packed, "null packed");
    return plan_spmm_dense_then(plan, value, split, mat, mat_stride, mat_rows, nullptr, feat, packed, params, row_code,
                                bits, out, out_stride, feat, accumulate, stream);
}

extern "C" int gnnagg_plan_spmm_packed_f32(gnnagg_plan *plan, const float *value, const float *y_packed,
                                           const uint32_t *header, float *out, int64_t feat, int accumulate,
                                           void *stream) {
    GNNAGG_REQUIRE(plan, "null plan");
    const int hw = gnnagg_packed_header_words(feat);
    if (hw == 0)
        return fail(GNNAGG_ERR_UNSUPPORTED, "packed source rows exist for widths 32, 64, 128, 256 (got %lld)",
                    (long long)feat);
    if (plan->rows == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(out, "null out");
    GNNAGG_REQUIRE(plan->nnz == 0 || (value && y_packed && header), "null value/y_packed/header");
    GNNAGG_REQUIRE((reinterpret_cast<uintptr_t>(out) & 15) == 0 && (reinterpret_cast<uintptr_t>(y_packed) & 3) == 0,
                   "packed SpMM needs a 16-byte aligned output");
    SpmmArgs a{};
    a.task = plan->task;  // every row runs in the lane-group kernel, the very longest included
    a.col = plan->col32;
    a.val = value;
    a.x = y_packed;
    a.hdr = header;
    a.hdr_words = hw;
    a.dst = out;
    a.feat = (int)feat;
    a.f_base = 0;
    a.accumulate = accumulate;
    a.ntasks = plan->rows - (accumulate ? plan->nempty : 0);
    a.head_tasks = plan->nlong;
    const Regions regions{plan->rows_per_group, plan->short_rows_per_group,
                          plan->nshort + (accumulate ? 0 : plan->nempty)};
    GNNAGG_HIP(launch_packed(a, regions, static_cast<hipStream_t>(stream)));
    return GNNAGG_OK;
}

static int plan_spmm_quantized(gnnagg_plan *plan, const float *value, const uint8_t *packed, const float *params,
                               const int32_t *row_code, const int64_t *elem_code, float *out, int64_t out_stride,
                               int64_t feat, int bits, int accumulate, void *stream) {
    GNNAGG_REQUIRE(plan, "null plan");
    GNNAGG_REQUIRE(bits == 2 || bits == 4 || bits == 8, "bits must be 2, 4 or 8 (got %d)", bits);
    GNNAGG_REQUIRE(feat >= 0, "negative feature width");
    if (plan->rows == 0 || feat == 0) return GNNAGG_OK;
    if (int rc = check_feat(feat)) return rc;
    if (feat % 4 != 0)
        return fail(GNNAGG_ERR_UNSUPPORTED, "quantised source rows need a width that is a multiple of 4 (got %lld)",
                    (long long)feat);
    GNNAGG_REQUIRE(out, "null out");
    GNNAGG_REQUIRE(plan->nnz == 0 || (value && packed && params && (row_code || elem_code)),
                   "null value/packed/params/row codes");
    GNNAGG_REQUIRE(out_stride >= feat && out_stride % 4 == 0 && out_stride < (int64_t(1) << 31),
                   "output row stride %lld must be a multiple of 4, at least the width and below 2^31",
                   (long long)out_stride);
    GNNAGG_REQUIRE((reinterpret_cast<uintptr_t>(out) & 15) == 0 && (reinterpret_cast<uintptr_t>(packed) & 3) == 0 &&
                       (reinterpret_cast<uintptr_t>(params) & 7) == 0,
                   "quantised SpMM needs a 16-byte aligned output, 4-byte aligned bytes and 8-byte aligned parameters");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const Regions regions{plan->rows_per_group, plan->short_rows_per_group,
                          plan->nshort + (accumulate ? 0 : plan->nempty)};
    for (int64_t f_base = 0; f_base < feat;) {
        const Shape s = pick_shape(4, feat - f_base);
        SpmmArgs a{};
        a.task = plan->task;  // every row runs in the lane-group kernel, the very longest included
        a.col = elem_code ? static_cast<const void *>(elem_code) : static_cast<const void *>(plan->col32);
        a.val = value;
        a.qdata = packed;
        a.qparams = params;
        a.qcode = row_code;
        a.qbits = bits;
        a.dst = out;
        a.ldd = (int)out_stride;
        a.feat = (int)feat;
        a.f_base = (int)f_base;
        a.accumulate = accumulate;
        a.ntasks = plan->rows - (accumulate ? plan->nempty : 0);
        a.head_tasks = plan->nlong;
        if (elem_code) GNNAGG_HIP((dispatch_shape<4, int64_t, kRowsPlanned, kSrcQuant>(s, a, regions, st)));
        else GNNAGG_HIP((dispatch_shape<4, int32_t, kRowsPlanned, kSrcQuant>(s, a, regions, st)));
        f_base += s.width();
    }
    return GNNAGG_OK;
}

extern "C" int gnnagg_plan_spmm_quantized_f32(gnnagg_plan *plan, const float *value, const uint8_t *packed,
                                              const float *params, const int32_t *row_code, float *out,
                                              int64_t out_stride, int64_t feat, int bits, int accumulate, void *stream) {
    GNNAGG_REQUIRE(plan == nullptr || plan->nnz == 0 || row_code, "null row_code");
    return plan_spmm_quantized(plan, value, packed, params, row_code, nullptr, out, out_stride, feat, bits, accumulate,
                               stream);
}

extern "C" int gnnagg_plan_spmm_quantized_elements_f32(gnnagg_plan *plan, const float *value, const uint8_t *packed,
                                                       const float *params, const int64_t *elem_code, float *out,
                                                       int64_t out_stride, int64_t feat, int bits, int accumulate,
                                                       void *stream) {
    GNNAGG_REQUIRE(plan == nullptr || plan->nnz == 0 || elem_code, "null elem_code");
    return plan_spmm_quantized(plan, value, packed, params, nullptr, elem_code, out, out_stride, feat, bits, accumulate,
                               stream);
}

extern "C" int gnnagg_plan_spmm_bf16_f32(gnnagg_plan *plan, const float *value, const void *mat, int mat_is_bf16,
                                         int64_t mat_stride, void *out, int out_is_bf16, int64_t out_stride,
                                         int64_t feat, int accumulate, void *stream) {
    GNNAGG_REQUIRE(plan, "null plan");
    GNNAGG_REQUIRE(feat >= 0, "negative feature width");
    GNNAGG_REQUIRE(mat_is_bf16 || out_is_bf16, "neither operand is bf16: use gnnagg_plan_spmm_strided_f32");
    if (plan->rows == 0 || feat == 0) return GNNAGG_OK;
    if (int rc = check_feat(feat)) return rc;
    if (feat % 4 != 0)
        return fail(GNNAGG_ERR_UNSUPPORTED, "bf16 rows need a width that is a multiple of 4 (got %lld)", (long long)feat);
    if (out_is_bf16 && accumulate)
        return fail(GNNAGG_ERR_UNSUPPORTED, "bf16 result rows are written, not accumulated onto (accumulate must be 0)");
    GNNAGG_REQUIRE(out, "null out");
    GNNAGG_REQUIRE(plan->nnz == 0 || (value && mat), "null value/mat");
    GNNAGG_REQUIRE(mat_stride >= feat && mat_stride % 4 == 0 && mat_stride < (int64_t(1) << 31) && out_stride >= feat &&
                       out_stride % 4 == 0 && out_stride < (int64_t(1) << 31),
                   "row strides (%lld, %lld) must be multiples of 4, at least the width and below 2^31",
                   (long long)mat_stride, (long long)out_stride);
    // a lane moves four values at a time: 8 bytes of a bf16 row, 16 of an fp32 row
    GNNAGG_REQUIRE((reinterpret_cast<uintptr_t>(mat) & (mat_is_bf16 ? 7 : 15)) == 0 &&
                       (reinterpret_cast<uintptr_t>(out) & (out_is_bf16 ? 7 : 15)) == 0,
                   "bf16 rows must be 8-byte aligned, fp32 rows 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const Regions regions{plan->rows_per_group, plan->short_rows_per_group,
                          plan->nshort + (accumulate ? 0 : plan->nempty)};
    for (int64_t f_base = 0; f_base < feat;) {
        const Shape s = pick_shape(4, feat - f_base);
        SpmmArgs a{};
        a.task = plan->task;  // every row runs in the lane-group kernel, the very longest included
        a.col = plan->col32;
        a.val = value;
        a.x = static_cast<const float *>(mat);
        a.ldx = (int)mat_stride;
        a.dst = static_cast<float *>(out);
        a.ldd = (int)out_stride;
        a.dst_bf16 = out_is_bf16 ? 1 : 0;
        a.feat = (int)feat;
        a.f_base = (int)f_base;
        a.accumulate = accumulate;
        a.ntasks = plan->rows - (accumulate ? plan->nempty : 0);
        a.head_tasks = plan->nlong;
        if (mat_is_bf16)
            GNNAGG_HIP((dispatch_shape<4, int32_t, kRowsPlanned, kSrcBf16>(s, a, regions, st)));
        else
            GNNAGG_HIP((dispatch_shape<4, int32_t, kRowsPlanned, kSrcDense>(s, a, regions, st)));
        f_base += s.width();
    }
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
