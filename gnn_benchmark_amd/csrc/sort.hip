// Set-up time sorting and run detection on the device, hand-written for gfx950 (64-lane waves): a stable LSD radix
// sort of (key, 32-bit payload) pairs, an exclusive scan, and the run structure of a sorted list (unique values,
// counts, inverse).  They serve the format builders (COO -> CSR, CSR -> transposed CSR), the plan's ordering of rows
// by length, and the index-map builders of data_manager/DataProcessor.py, which the reference writes as per-edge
// Python loops over sorted lists (self_benchmark/a64fx/data_manager/DataProcessor.py:39-53, :238-246, :434-444).
//
// Radix sort, one pass per 8 bits of key, least significant first; a pass is three launches:
//   1. histogram: a block counts the digits of its tile of kTile keys (LDS atomics) into hist[digit][block];
//   2. exclusive scan of hist in (digit, block) order: where each block's keys of each digit start in the output;
//   3. scatter: the block ranks its tile's keys by digit, in input order (per-wave LDS counters; eight ballots give
//      the lanes of a wave that hold the same digit), brings them to their place in the tile through LDS, and writes
//      the tile out digit by digit, so that a digit's keys leave as one run of neighbouring addresses.  Equal keys
//      keep their input order: the sort is stable, which is what makes repeated (row, col) pairs keep their order
//      and what the reference's known-answer vectors need of its argsort.
#include "sort.h"

#include <algorithm>

namespace gnnagg {
namespace {

constexpr int kRadixBits = 8;
constexpr int kBins = 1 << kRadixBits;
constexpr int kKeysPerThread = 32;
constexpr int kTile = 256 * kKeysPerThread;
constexpr int kXcds = 8;  // gfx950: eight accelerator dies, each with its own L2

// ------------------------------------------------------------------ exclusive scan of uint32 (sums below 2^32)
constexpr int kScanPerThread = 8;
constexpr int kScanTile = 256 * kScanPerThread;

__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
    const int lane = (int)__lane_id();
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t up = (uint32_t)__shfl_up((int)v, d, 64);
        if (lane >= d) v += up;
    }
    return v;
}

// sum of the block's values in front of this thread's; *total: the block's sum (valid in every thread)
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t mine, uint32_t *total) {
    __shared__ uint32_t wave_sum[4];
    const int lane = (int)threadIdx.x & 63, wave = (int)threadIdx.x >> 6;
    const uint32_t incl = wave_inclusive_scan(mine);
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    uint32_t before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        if (w < wave) before += wave_sum[w];
        all += wave_sum[w];
    }
    __syncthreads();
    *total = all;
    return before + incl - mine;
}

__global__ __launch_bounds__(256) void scan_tile_sums_kernel(const uint32_t *__restrict__ in, int64_t n,
                                                             uint32_t *__restrict__ tile_sum) {
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanPerThread;
    uint32_t s = 0;
#pragma unroll
    for (int k = 0; k < kScanPerThread; ++k)
        if (base + k < n) s += in[base + k];
    uint32_t total;
    (void)block_exclusive_scan(s, &total);
    if (threadIdx.x == 0) tile_sum[blockIdx.x] = total;
}

// one block: exclusive scan of the tile sums in place, 256 at a time with a running carry
__global__ __launch_bounds__(256) void scan_sums_kernel(uint32_t *__restrict__ tile_sum, int64_t tiles) {
    uint32_t carry = 0;
    for (int64_t base = 0; base < tiles; base += 256) {
        const int64_t i = base + threadIdx.x;
        const uint32_t v = i < tiles ? tile_sum[i] : 0;
        uint32_t total;
        const uint32_t before = block_exclusive_scan(v, &total);
        if (i < tiles) tile_sum[i] = carry + before;
        carry += total;
    }
}

// (in and out may be the same array: a block reads its tile before it writes it)
__global__ __launch_bounds__(256) void scan_apply_kernel(const uint32_t *in, int64_t n,
                                                         const uint32_t *__restrict__ tile_before, uint32_t *out) {
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanPerThread;
    uint32_t v[kScanPerThread];
    uint32_t s = 0;
#pragma unroll
    for (int k = 0; k < kScanPerThread; ++k) {
        v[k] = base + k < n ? in[base + k] : 0;
        s += v[k];
    }
    uint32_t total;
    uint32_t run = tile_before[blockIdx.x] + block_exclusive_scan(s, &total);
#pragma unroll
    for (int k = 0; k < kScanPerThread; ++k) {
        if (base + k < n) out[base + k] = run;
        run += v[k];
    }
}

}  // namespace

namespace {

int64_t scan_tiles(int64_t n) { return (n + kScanTile - 1) / kScanTile; }

// the scan with the caller's array for the tile sums (scan_tiles(n) entries); enqueues only
int exclusive_scan_into(const uint32_t *in, uint32_t *out, int64_t n, uint32_t *tile_sums, hipStream_t st) {
    const int64_t tiles = scan_tiles(n);
    hipLaunchKernelGGL(scan_tile_sums_kernel, dim3((unsigned)tiles), dim3(256), 0, st, in, n, tile_sums);
    GNNAGG_HIP(hipGetLastError());
    hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(256), 0, st, tile_sums, tiles);
    GNNAGG_HIP(hipGetLastError());
    hipLaunchKernelGGL(scan_apply_kernel, dim3((unsigned)tiles), dim3(256), 0, st, in, n, tile_sums, out);
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

}  // namespace

// out[i] = in[0] + ... + in[i - 1] (in == out is fine).  Allocates the tile sums; returns when the scan is done.
int exclusive_scan_u32(const uint32_t *in, uint32_t *out, int64_t n, hipStream_t st) {
    if (n <= 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(scan_tiles(n) < (int64_t(1) << 31), "scan of more than 2^42 values");
    DevBuf<uint32_t> sums;
    GNNAGG_HIP(sums.alloc((size_t)scan_tiles(n)));
    if (int rc = exclusive_scan_into(in, out, n, sums.p, st)) return rc;
    GNNAGG_HIP(hipStreamSynchronize(st));  // the tile sums are released on scope exit
    return GNNAGG_OK;
}

namespace {

// ------------------------------------------------------------------ radix sort
template <typename KeyT>
__global__ __launch_bounds__(256) void radix_histogram_kernel(const KeyT *__restrict__ key, int64_t n, int shift,
                                                              uint32_t *__restrict__ hist, int64_t blocks) {
    __shared__ uint32_t bins[kBins];
    bins[threadIdx.x] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kTile + threadIdx.x;
#pragma unroll
    for (int r = 0; r < kKeysPerThread; ++r) {
        const int64_t i = base + (int64_t)r * 256;
        if (i < n) atomicAdd(&bins[(int)((key[i] >> shift) & (kBins - 1))], 1u);
    }
    __syncthreads();
    hist[(int64_t)threadIdx.x * blocks + blockIdx.x] = bins[threadIdx.x];
}

// One pass's scatter.  A block takes its tile in index order, wave w the keys [w * kTile / 4, (w + 1) * kTile / 4) in
// rounds of 64.  (1) Each wave ranks its keys against its own LDS counters, no block barrier: a key's rank in its wave
// is the counter of its digit + the lower lanes of this round that hold the same digit (eight ballots).  (2) From the
// four waves' counters: where each digit starts in the tile, and where each wave's keys of it do.  (3) The keys go to
// their place in the tile through LDS, so that (4) thread t writes position t + 256 j of the sorted tile: keys of one
// digit leave as one run of neighbouring addresses (kTile / 256 keys on average) instead of one by one.  (5) The
// payloads take the same way through the same LDS array, to the addresses step 4 kept.
template <typename KeyT>
__global__ __launch_bounds__(256) void radix_scatter_kernel(const KeyT *__restrict__ key_in,
                                                            const uint32_t *__restrict__ val_in, int64_t n, int shift,
                                                            const uint32_t *__restrict__ start, int64_t blocks,
                                                            KeyT *__restrict__ key_out, uint32_t *__restrict__ val_out) {
    __shared__ KeyT sorted[kTile];
    __shared__ uint32_t count[4][kBins];  // per wave: keys of each digit so far; after step 2: where they start
    __shared__ uint32_t out_base[kBins];  // output address of the digit's first key of this tile - its place in the tile
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // Workgroups go to the eight XCDs in turn; each XCD gets a stretch of neighbouring tiles, so that the runs two
    // neighbouring tiles write to one digit's region, which adjoin, meet in one L2 instead of two.
    const int64_t per_xcd = (int64_t)(gridDim.x / kXcds);
    const int64_t tile = (int64_t)(blockIdx.x % kXcds) * per_xcd + (int64_t)(blockIdx.x / kXcds);
    if (tile >= blocks) return;
    const int64_t tile_base = tile * kTile;
    const int live_keys = (int)std::min<int64_t>(kTile, n - tile_base);
#pragma unroll
    for (int w = 0; w < 4; ++w) count[w][tid] = 0;
    KeyT k[kKeysPerThread];
    uint32_t v[kKeysPerThread];
    uint32_t rank[kKeysPerThread];
    const int mine = wave * (kTile / 4) + lane;  // this thread's key of round r: tile position mine + 64 r
#pragma unroll
    for (int r = 0; r < kKeysPerThread; ++r) {
        const int at = mine + 64 * r;
        k[r] = at < live_keys ? key_in[tile_base + at] : KeyT(0);
        v[r] = at < live_keys ? val_in[tile_base + at] : 0u;
    }
    __syncthreads();
    uint32_t *my_count = count[wave];
#pragma unroll
    for (int r = 0; r < kKeysPerThread; ++r) {
        const bool live = mine + 64 * r < live_keys;  // dead keys are the tile's last ones
        const int digit = (int)((k[r] >> shift) & (kBins - 1));
        uint64_t same = __builtin_amdgcn_ballot_w64(live);
#pragma unroll
        for (int b = 0; b < kRadixBits; ++b) {
            const uint64_t has = __builtin_amdgcn_ballot_w64(((digit >> b) & 1) != 0);
            same &= ((digit >> b) & 1) ? has : ~has;
        }
        const uint32_t below = (uint32_t)__popcll(same & ((uint64_t(1) << lane) - 1));
        // the wave's LDS accesses execute in program order: this read sees the last round's update
        const uint32_t before = my_count[digit];
        __builtin_amdgcn_wave_barrier();
        if (live && below == 0) my_count[digit] = before + (uint32_t)__popcll(same);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        rank[r] = before + below;
    }
    __syncthreads();
    {   // digit `tid`
        const uint32_t c0 = count[0][tid], c1 = count[1][tid], c2 = count[2][tid], c3 = count[3][tid];
        uint32_t total;
        const uint32_t first = block_exclusive_scan(c0 + c1 + c2 + c3, &total);
        count[0][tid] = first;
        count[1][tid] = first + c0;
        count[2][tid] = first + c0 + c1;
        count[3][tid] = first + c0 + c1 + c2;
        out_base[tid] = start[(int64_t)tid * blocks + tile] - first;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kKeysPerThread; ++r) {
        const int digit = (int)((k[r] >> shift) & (kBins - 1));
        rank[r] += my_count[digit];  // now the key's place in the sorted tile
        if (mine + 64 * r < live_keys) sorted[rank[r]] = k[r];
    }
    __syncthreads();
    uint32_t to[kKeysPerThread];
#pragma unroll
    for (int j = 0; j < kKeysPerThread; ++j) {
        const int p = tid + 256 * j;
        if (p < live_keys) {
            const KeyT key = sorted[p];
            to[j] = out_base[(int)((key >> shift) & (kBins - 1))] + (uint32_t)p;
            key_out[to[j]] = key;
        }
    }
    __syncthreads();
    uint32_t *sorted_val = reinterpret_cast<uint32_t *>(sorted);
#pragma unroll
    for (int r = 0; r < kKeysPerThread; ++r)
        if (mine + 64 * r < live_keys) sorted_val[rank[r]] = v[r];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kKeysPerThread; ++j) {
        const int p = tid + 256 * j;
        if (p < live_keys) val_out[to[j]] = sorted_val[p];
    }
}

size_t align_up(size_t bytes) { return (bytes + 255) & ~size_t(255); }

size_t sort_hist_bytes(int64_t n) { return align_up((size_t)((n + kTile - 1) / kTile) * kBins * sizeof(uint32_t)); }
size_t sort_sums_bytes(int64_t n) {
    return align_up((size_t)scan_tiles((n + kTile - 1) / kTile * kBins) * sizeof(uint32_t));
}

template <typename KeyT>
int radix_sort_pairs(KeyT *key_a, KeyT *key_b, uint32_t *val_a, uint32_t *val_b, int64_t n, int bits, hipStream_t st,
                     bool *result_in_b, void *workspace) {
    *result_in_b = false;
    if (n <= 0 || bits <= 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(n < (int64_t(1) << 32), "radix sort of more than 2^32-1 pairs");
    const int64_t blocks = (n + kTile - 1) / kTile;
    DevBuf<char> own;
    if (!workspace) {
        GNNAGG_HIP(own.alloc(sort_pairs_workspace_bytes(n)));
        workspace = own.p;
    }
    uint32_t *hist = static_cast<uint32_t *>(workspace);
    uint32_t *sums = reinterpret_cast<uint32_t *>(static_cast<char *>(workspace) + sort_hist_bytes(n));
    KeyT *kin = key_a, *kout = key_b;
    uint32_t *vin = val_a, *vout = val_b;
    for (int shift = 0; shift < bits; shift += kRadixBits) {
        hipLaunchKernelGGL((radix_histogram_kernel<KeyT>), dim3((unsigned)blocks), dim3(256), 0, st, kin, n, shift,
                           hist, blocks);
        GNNAGG_HIP(hipGetLastError());
        if (int rc = exclusive_scan_into(hist, hist, blocks * kBins, sums, st)) return rc;
        const int64_t scatter_grid = (blocks + kXcds - 1) / kXcds * kXcds;
        hipLaunchKernelGGL((radix_scatter_kernel<KeyT>), dim3((unsigned)scatter_grid), dim3(256), 0, st, kin, vin, n, shift,
                           hist, blocks, kout, vout);
        GNNAGG_HIP(hipGetLastError());
        std::swap(kin, kout);
        std::swap(vin, vout);
        *result_in_b = !*result_in_b;
    }
    if (own.p) GNNAGG_HIP(hipStreamSynchronize(st));  // its own workspace is released on scope exit
    return GNNAGG_OK;
}

}  // namespace

size_t sort_pairs_workspace_bytes(int64_t n) { return n > 0 ? sort_hist_bytes(n) + sort_sums_bytes(n) : 0; }

int sort_pairs_u64(uint64_t *key_a, uint64_t *key_b, uint32_t *val_a, uint32_t *val_b, int64_t n, int bits,
                   hipStream_t st, bool *result_in_b, void *workspace) {
    return radix_sort_pairs<uint64_t>(key_a, key_b, val_a, val_b, n, bits, st, result_in_b, workspace);
}

int sort_pairs_u32(uint32_t *key_a, uint32_t *key_b, uint32_t *val_a, uint32_t *val_b, int64_t n, int bits,
                   hipStream_t st, bool *result_in_b, void *workspace) {
    return radix_sort_pairs<uint32_t>(key_a, key_b, val_a, val_b, n, bits, st, result_in_b, workspace);
}

namespace {

// ------------------------------------------------------------------ argsort / runs of a sorted list
__global__ void fill_u32_kernel(uint32_t *p, int count, uint32_t v) {
    if ((int)threadIdx.x < count) p[threadIdx.x] = v;
}

__global__ __launch_bounds__(256) void argsort_prepare_kernel(const int64_t *__restrict__ x, int64_t n,
                                                              uint64_t *__restrict__ key, uint32_t *__restrict__ idx,
                                                              unsigned long long *__restrict__ max_key,
                                                              unsigned int *__restrict__ negative) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    unsigned long long m = 0;
    bool neg = false;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const int64_t v = x[i];
        neg |= v < 0;
        key[i] = (uint64_t)v;
        idx[i] = (uint32_t)i;
        if (v > 0 && (unsigned long long)v > m) m = (unsigned long long)v;
    }
    // one atomic per block, not per thread: all of them land on one address
    __shared__ unsigned long long wave_m[4];
    __shared__ unsigned int wave_neg[4];
    m = wave_max_u64(m);
    const bool any_neg = __builtin_amdgcn_ballot_w64(neg) != 0;
    if ((threadIdx.x & 63) == 0) {
        wave_m[threadIdx.x >> 6] = m;
        wave_neg[threadIdx.x >> 6] = any_neg ? 1u : 0u;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w) m = wave_m[w] > m ? wave_m[w] : m;
        if (m) atomicMax(max_key, m);
        if (wave_neg[0] | wave_neg[1] | wave_neg[2] | wave_neg[3]) atomicOr(negative, 1u);
    }
}

__global__ __launch_bounds__(256) void argsort_finish_kernel(const uint64_t *__restrict__ key,
                                                             const uint32_t *__restrict__ idx, int64_t n,
                                                             int64_t *__restrict__ perm, int64_t *__restrict__ sorted) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    perm[i] = (int64_t)idx[i];
    if (sorted) sorted[i] = (int64_t)key[i];
}

// flag[i] = 1 where a run starts: i == 0, x[i] != x[i - 1], or i is one of the forced starts
__global__ __launch_bounds__(256) void run_flags_kernel(const int64_t *__restrict__ x, int64_t n,
                                                        uint32_t *__restrict__ flag) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    flag[i] = (i == 0 || x[i] != x[i - 1]) ? 1u : 0u;
}

__global__ __launch_bounds__(256) void force_starts_kernel(const int64_t *__restrict__ starts, int64_t count, int64_t n,
                                                           uint32_t *__restrict__ flag) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    const int64_t s = starts[i];
    if (s >= 0 && s < n) flag[s] = 1u;
}

// before[i] = runs that start in front of position i (exclusive scan of the flags).  The run of position i is
// before[i] + flag[i] - 1; a run's first position writes its value, and its start for the counts.
__global__ __launch_bounds__(256) void run_outputs_kernel(const int64_t *__restrict__ x, const uint32_t *__restrict__ flag,
                                                          const uint32_t *__restrict__ before, int64_t n,
                                                          int64_t *__restrict__ uniq, int64_t *__restrict__ inverse,
                                                          int64_t *__restrict__ run_start) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int64_t run = (int64_t)before[i] + (int64_t)flag[i] - 1;
    if (inverse) inverse[i] = run;
    if (flag[i]) {
        if (uniq) uniq[run] = x[i];
        if (run_start) run_start[run] = i;
    }
}

__global__ __launch_bounds__(256) void run_counts_kernel(const int64_t *__restrict__ run_start, int64_t runs, int64_t n,
                                                         int64_t *__restrict__ counts) {
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= runs) return;
    counts[r] = (r + 1 < runs ? run_start[r + 1] : n) - run_start[r];
}

}  // namespace
}  // namespace gnnagg

using namespace gnnagg;

namespace {

// The temporaries of one call, carved out of the caller's workspace or, without one, out of one allocation of the
// call's own (released when the call returns, which then has to wait for its kernels).
struct Carver {
    char *at = nullptr;
    DevBuf<char> own;
    int open(void *workspace, int64_t workspace_bytes, size_t need) {
        if (workspace) {
            GNNAGG_REQUIRE(workspace_bytes >= (int64_t)need, "workspace smaller than the *_workspace_bytes of this size");
            GNNAGG_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15) == 0, "workspace not 16-byte aligned");
            at = static_cast<char *>(workspace);
        } else {
            GNNAGG_HIP(own.alloc(need));
            at = own.p;
        }
        return GNNAGG_OK;
    }
    template <typename T>
    T *take(size_t count) {
        T *p = reinterpret_cast<T *>(at);
        at += align_up(count * sizeof(T));
        return p;
    }
};

size_t argsort_bytes(int64_t n) {
    return 2 * align_up((size_t)n * 8) + 2 * align_up((size_t)n * 4) + align_up(16) + sort_pairs_workspace_bytes(n);
}
size_t runs_bytes(int64_t n) {
    return 2 * align_up((size_t)n * 4) + align_up((size_t)n * 8) + align_up((size_t)scan_tiles(n) * 4);
}

}  // namespace

extern "C" int64_t gnnagg_argsort_workspace_bytes(int64_t n) { return n > 0 ? (int64_t)argsort_bytes(n) : 0; }
extern "C" int64_t gnnagg_runs_workspace_bytes(int64_t n) { return n > 0 ? (int64_t)runs_bytes(n) : 0; }

extern "C" int gnnagg_argsort_i64(const int64_t *x, int64_t n, int64_t *perm, int64_t *sorted, void *workspace,
                                  int64_t workspace_bytes, void *stream) {
    GNNAGG_REQUIRE(n >= 0, "negative size");
    if (n == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(x && perm, "null x/perm");
    if (n >= (int64_t(1) << 32)) return fail(GNNAGG_ERR_UNSUPPORTED, "argsort of more than 2^32-1 values");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Carver ws;
    if (int rc = ws.open(workspace, workspace_bytes, argsort_bytes(n))) return rc;
    uint64_t *key_a = ws.take<uint64_t>((size_t)n), *key_b = ws.take<uint64_t>((size_t)n);
    uint32_t *idx_a = ws.take<uint32_t>((size_t)n), *idx_b = ws.take<uint32_t>((size_t)n);
    unsigned long long *flags = ws.take<unsigned long long>(2);  // [0] the largest key, [1] whether a key was negative
    void *sort_ws = ws.take<char>(sort_pairs_workspace_bytes(n));
    const unsigned grid = (unsigned)std::min<int64_t>((n + 255) / 256, 256 * 4);
    hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, st, reinterpret_cast<uint32_t *>(flags), 4, 0u);
    hipLaunchKernelGGL(argsort_prepare_kernel, dim3(grid), dim3(256), 0, st, x, n, key_a, idx_a, flags,
                       reinterpret_cast<unsigned int *>(flags + 1));
    GNNAGG_HIP(hipGetLastError());
    unsigned long long h[2] = {0, 0};
    GNNAGG_HIP(hipMemcpyAsync(h, flags, sizeof(h), hipMemcpyDeviceToHost, st));
    GNNAGG_HIP(hipStreamSynchronize(st));
    GNNAGG_REQUIRE((h[1] & 0xffffffffull) == 0, "argsort takes non-negative keys (node ids, positions)");
    const int bits = h[0] ? ceil_log2_u64(h[0] + 1) : 1;
    bool in_b = false;
    if (int rc = sort_pairs_u64(key_a, key_b, idx_a, idx_b, n, bits, st, &in_b, sort_ws)) return rc;
    hipLaunchKernelGGL(argsort_finish_kernel, dim3(grid_for(n, 256)), dim3(256), 0, st, in_b ? key_b : key_a,
                       in_b ? idx_b : idx_a, n, perm, sorted);
    GNNAGG_HIP(hipGetLastError());
    if (ws.own.p) GNNAGG_HIP(hipStreamSynchronize(st));
    return GNNAGG_OK;
}

extern "C" int gnnagg_runs_i64(const int64_t *x, int64_t n, const int64_t *forced_starts, int64_t forced_count,
                               int64_t *uniq, int64_t *inverse, int64_t *counts, int64_t *runs_out, void *workspace,
                               int64_t workspace_bytes, void *stream) {
    GNNAGG_REQUIRE(n >= 0 && forced_count >= 0, "negative size");
    GNNAGG_REQUIRE(runs_out, "null runs_out");
    *runs_out = 0;
    if (n == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(x, "null x");
    GNNAGG_REQUIRE(forced_count == 0 || forced_starts, "null forced_starts");
    if (n >= (int64_t(1) << 32)) return fail(GNNAGG_ERR_UNSUPPORTED, "run detection over more than 2^32-1 values");
    hipStream_t st = static_cast<hipStream_t>(stream);
    Carver ws;
    if (int rc = ws.open(workspace, workspace_bytes, runs_bytes(n))) return rc;
    uint32_t *flag = ws.take<uint32_t>((size_t)n), *before = ws.take<uint32_t>((size_t)n);
    int64_t *run_start = ws.take<int64_t>((size_t)n);
    uint32_t *sums = ws.take<uint32_t>((size_t)scan_tiles(n));
    hipLaunchKernelGGL(run_flags_kernel, dim3(grid_for(n, 256)), dim3(256), 0, st, x, n, flag);
    GNNAGG_HIP(hipGetLastError());
    if (forced_count > 0) {
        hipLaunchKernelGGL(force_starts_kernel, dim3(grid_for(forced_count, 256)), dim3(256), 0, st, forced_starts,
                           forced_count, n, flag);
        GNNAGG_HIP(hipGetLastError());
    }
    if (int rc = exclusive_scan_into(flag, before, n, sums, st)) return rc;
    uint32_t last[2] = {0, 0};
    GNNAGG_HIP(hipMemcpyAsync(&last[0], before + (n - 1), sizeof(uint32_t), hipMemcpyDeviceToHost, st));
    GNNAGG_HIP(hipMemcpyAsync(&last[1], flag + (n - 1), sizeof(uint32_t), hipMemcpyDeviceToHost, st));
    GNNAGG_HIP(hipStreamSynchronize(st));  // the number of runs sizes the last launch and is what the call returns
    const int64_t runs = (int64_t)last[0] + (int64_t)last[1];
    hipLaunchKernelGGL(run_outputs_kernel, dim3(grid_for(n, 256)), dim3(256), 0, st, x, flag, before, n, uniq, inverse,
                       run_start);
    GNNAGG_HIP(hipGetLastError());
    if (counts) {
        hipLaunchKernelGGL(run_counts_kernel, dim3(grid_for(runs, 256)), dim3(256), 0, st, run_start, runs, n, counts);
        GNNAGG_HIP(hipGetLastError());
    }
    if (ws.own.p) GNNAGG_HIP(hipStreamSynchronize(st));
    *runs_out = runs;
    return GNNAGG_OK;
}
