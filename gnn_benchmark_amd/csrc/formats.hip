// Sparse-format construction on the device (setup-time): COO -> CSR, CSR -> transposed
// CSR, and the boundary-row gather.  gfx950 only.

#include <algorithm>
#include <type_traits>

#include "common.h"
#include "sort.h"

namespace gnnagg {
namespace {

// key = row << col_bits | col ; idx = position
__global__ __launch_bounds__(256) void pack_keys_kernel(const int64_t *__restrict__ row,
                                                        const int64_t *__restrict__ col, int64_t nnz, int64_t rows,
                                                        int64_t cols, int col_bits, uint64_t *__restrict__ key,
                                                        uint32_t *__restrict__ idx, unsigned int *__restrict__ bad) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= nnz) return;
    const int64_t r = row[e], c = col[e];
    if (r < 0 || r >= rows || c < 0 || c >= cols) {
        atomicOr(bad, 1u);
        key[e] = 0;
    } else {
        key[e] = ((uint64_t)r << col_bits) | (uint64_t)c;
    }
    idx[e] = (uint32_t)e;
}

__global__ __launch_bounds__(256) void unpack_sorted_kernel(const uint64_t *__restrict__ key,
                                                            const uint32_t *__restrict__ idx,
                                                            const float *__restrict__ value, int64_t nnz,
                                                            int col_bits, int64_t *__restrict__ col_out,
                                                            float *__restrict__ value_out) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= nnz) return;
    col_out[e] = (int64_t)(key[e] & ((uint64_t(1) << col_bits) - 1));
    if (value_out) value_out[e] = value[idx[e]];
}

// ptr[r] = number of sorted keys whose major index (key >> shift) is < r, r in [0, n]
__global__ __launch_bounds__(256) void major_ptr_kernel(const uint64_t *__restrict__ key, int64_t nnz, int shift,
                                                        int64_t n, int64_t *__restrict__ ptr) {
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r > n) return;
    int64_t lo = 0, hi = nnz;  // first position with major >= r
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if ((int64_t)(key[mid] >> shift) < r) lo = mid + 1; else hi = mid;
    }
    ptr[r] = lo;
}

// key = col << row_bits | row for every stored element of a CSR matrix; idx = position.  The row of element e is the
// last row r with rowptr[r] <= e.  A block owns 256 consecutive elements: two threads find the rows of its first and
// last element by binary search in rowptr, the block copies that stretch of rowptr to LDS (when it is at most kSpan
// rows: rows without elements can make it long) and every thread searches there instead of in memory.
constexpr int kSpan = 1024;

__device__ __forceinline__ int64_t last_row_at_or_before(const int64_t *__restrict__ rowptr, int64_t lo, int64_t hi,
                                                         int64_t e) {
    while (hi - lo > 1) {  // invariant: rowptr[lo] <= e, and hi is past the answer
        const int64_t mid = (lo + hi) >> 1;
        if (rowptr[mid] <= e) lo = mid; else hi = mid;
    }
    return lo;
}

__global__ __launch_bounds__(256) void pack_transposed_keys_kernel(const int64_t *__restrict__ rowptr,
                                                                   const int64_t *__restrict__ col, int64_t rows,
                                                                   int64_t cols, int64_t nnz, int row_bits,
                                                                   uint64_t *__restrict__ key,
                                                                   uint32_t *__restrict__ idx,
                                                                   unsigned int *__restrict__ bad) {
    __shared__ int64_t s_ptr[kSpan];
    __shared__ int64_t s_first, s_last;
    const int64_t e0 = (int64_t)blockIdx.x * 256;
    const int64_t e = e0 + threadIdx.x;
    if (threadIdx.x == 0) s_first = last_row_at_or_before(rowptr, 0, rows, e0);
    if (threadIdx.x == 64) s_last = last_row_at_or_before(rowptr, 0, rows, e0 + 255 < nnz ? e0 + 255 : nnz - 1);
    __syncthreads();
    const int64_t first = s_first, last = s_last;
    const int span = last - first + 1 <= kSpan ? (int)(last - first + 1) : 0;  // 0: too long for LDS
    for (int i = (int)threadIdx.x; i < span; i += 256) s_ptr[i] = rowptr[first + i];
    __syncthreads();
    if (e >= nnz) return;
    int64_t row;
    if (span) {
        int lo = 0, hi = span;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (s_ptr[mid] <= e) lo = mid; else hi = mid;
        }
        row = first + lo;
    } else {
        row = last_row_at_or_before(rowptr, first, last + 1, e);
    }
    const int64_t c = col[e];
    if (c < 0 || c >= cols) {
        atomicOr(bad, 1u);
        key[e] = 0;
    } else {
        key[e] = ((uint64_t)c << row_bits) | (uint64_t)row;
    }
    idx[e] = (uint32_t)e;
}

// out[i, :] = src[index[i], :].  A group of G lanes (G * VEC floats cover a row, or one pass of it)
// owns four rows at a time: their indices, then their vectors, are requested back to back before
// anything is stored.  Source rows come through normal loads (a boundary row usually goes to
// several peers, so it is asked for again soon); the result is written once, with streaming stores.
// OUT16 (VEC == 4 only): the rows are stored as bf16, rounded as the tensor copy rounds them.
template <int VEC, int G, bool OUT16>
__global__ __launch_bounds__(256) void gather_rows_kernel(const float *__restrict__ src, int64_t src_rows,
                                                          const int64_t *__restrict__ index,
                                                          void *__restrict__ out, int64_t n_index, int feat_vec) {
    static_assert(!OUT16 || VEC == 4, "bf16 rows are stored four values at a time");
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    using out_t = typename std::conditional<OUT16, u32x2, vec_t>::type;
    constexpr int kGroups = 256 / G;
    constexpr int kRows = 4;
    const int l = (int)threadIdx.x % G;
    const int group = (int)threadIdx.x / G;
    const int64_t step = (int64_t)gridDim.x * kGroups * kRows;
    for (int64_t base = ((int64_t)blockIdx.x * kGroups + group) * kRows; base < n_index; base += step) {
        const vec_t *s[kRows];
        out_t *d[kRows];
        bool ok[kRows], inside[kRows];
#pragma unroll
        for (int u = 0; u < kRows; ++u) {
            ok[u] = base + u < n_index;
            const int64_t r = ok[u] ? __builtin_nontemporal_load(index + base + u) : 0;
            // an index outside the source is never dereferenced: row 0 is read in its place and NaN is stored
            inside[u] = (uint64_t)r < (uint64_t)src_rows;
            s[u] = reinterpret_cast<const vec_t *>(src) + (inside[u] ? (size_t)r : 0) * (size_t)feat_vec;
            d[u] = reinterpret_cast<out_t *>(out) + (size_t)(base + u) * (size_t)feat_vec;
        }
        for (int f = l; f < feat_vec; f += G) {
            vec_t v[kRows];
#pragma unroll
            for (int u = 0; u < kRows; ++u)
                if (ok[u]) v[u] = s[u][f];
#pragma unroll
            for (int u = 0; u < kRows; ++u) {
                if (!ok[u]) continue;
                const vec_t w = inside[u] ? v[u] : v[u] * __builtin_nanf("");
                if constexpr (OUT16) {
                    u32x2 r;
                    r.x = (uint32_t)bf16_bits(w[0]) | ((uint32_t)bf16_bits(w[1]) << 16);
                    r.y = (uint32_t)bf16_bits(w[2]) | ((uint32_t)bf16_bits(w[3]) << 16);
                    __builtin_nontemporal_store(r, d[u] + f);
                } else {
                    __builtin_nontemporal_store(w, d[u] + f);
                }
            }
        }
    }
}

// any (index[i] >> shift) outside [0, bound): the lowest such position found by a block goes to *first_bad
template <typename T>
__global__ __launch_bounds__(256) void check_index_kernel(const T *__restrict__ index, int64_t count, int shift,
                                                          int64_t bound, unsigned long long *__restrict__ first_bad) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    unsigned long long bad = ~0ull;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += stride) {
        const int64_t v = (int64_t)index[i] >> shift;
        if ((v < 0 || v >= bound) && (unsigned long long)i < bad) bad = (unsigned long long)i;
    }
    if (bad != ~0ull) atomicMin(first_bad, bad);
}

template <int VEC, bool OUT16 = false>
hipError_t launch_gather_rows(const float *src, int64_t src_rows, const int64_t *index, void *out, int64_t n_index,
                              int feat_vec, hipStream_t st) {
    int g = 8;
    while (g < 64 && g < feat_vec) g *= 2;
    const int64_t rows_per_block = (256 / g) * 4;
    const int64_t need = (n_index + rows_per_block - 1) / rows_per_block;
    const unsigned grid = (unsigned)(need < 256 * 32 ? need : 256 * 32);
    if (g == 8) hipLaunchKernelGGL((gather_rows_kernel<VEC, 8, OUT16>), dim3(grid), dim3(256), 0, st, src, src_rows, index, out, n_index, feat_vec);
    else if (g == 16) hipLaunchKernelGGL((gather_rows_kernel<VEC, 16, OUT16>), dim3(grid), dim3(256), 0, st, src, src_rows, index, out, n_index, feat_vec);
    else if (g == 32) hipLaunchKernelGGL((gather_rows_kernel<VEC, 32, OUT16>), dim3(grid), dim3(256), 0, st, src, src_rows, index, out, n_index, feat_vec);
    else hipLaunchKernelGGL((gather_rows_kernel<VEC, 64, OUT16>), dim3(grid), dim3(256), 0, st, src, src_rows, index, out, n_index, feat_vec);
    return hipGetLastError();
}

// stable sort of the (key, position) pairs by the low `bits` bits of the key; where the result lies comes back in
// *key_sorted / *idx_sorted (one of the two array pairs)
int sort_keys(uint64_t *key_a, uint64_t *key_b, uint32_t *idx_a, uint32_t *idx_b, int64_t n, int bits, hipStream_t st,
              uint64_t **key_sorted, uint32_t **idx_sorted) {
    bool in_b = false;
    if (int rc = sort_pairs_u64(key_a, key_b, idx_a, idx_b, n, bits, st, &in_b)) return rc;
    *key_sorted = in_b ? key_b : key_a;
    *idx_sorted = in_b ? idx_b : idx_a;
    return GNNAGG_OK;
}

}  // namespace
}  // namespace gnnagg

using namespace gnnagg;

static int check_format_sizes(int64_t rows, int64_t cols, int64_t nnz) {
    GNNAGG_REQUIRE(rows >= 0 && cols >= 0 && nnz >= 0, "negative size");
    if (rows >= (int64_t(1) << 31) - 1 || cols >= (int64_t(1) << 31) - 1 || nnz >= (int64_t(1) << 31) - 1)
        return fail(GNNAGG_ERR_UNSUPPORTED, "format limits: rows, cols, nnz < 2^31-1 (got %lld, %lld, %lld)",
                    (long long)rows, (long long)cols, (long long)nnz);
    return GNNAGG_OK;
}

extern "C" int gnnagg_coo_to_csr(const int64_t *row, const int64_t *col, const float *value, int64_t nnz, int64_t rows,
                                 int64_t cols, int64_t *rowptr, int64_t *col_out, float *value_out, void *stream) {
    if (int rc = check_format_sizes(rows, cols, nnz)) return rc;
    GNNAGG_REQUIRE(rowptr, "null rowptr");
    GNNAGG_REQUIRE(nnz == 0 || (row && col && col_out), "null row/col/col_out");
    GNNAGG_REQUIRE((value == nullptr) == (value_out == nullptr), "value and value_out must both be given or both be null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (nnz == 0) {
        GNNAGG_HIP(hipMemsetAsync(rowptr, 0, sizeof(int64_t) * (size_t)(rows + 1), st));
        GNNAGG_HIP(hipStreamSynchronize(st));
        return GNNAGG_OK;
    }
    const int col_bits = std::max(1, ceil_log2_u64((uint64_t)std::max<int64_t>(cols, 1)));
    const int row_bits = std::max(1, ceil_log2_u64((uint64_t)std::max<int64_t>(rows, 1)));
    DevBuf<uint64_t> key_in, key_out;
    DevBuf<uint32_t> idx_in, idx_out;
    DevBuf<unsigned int> bad;
    GNNAGG_HIP(key_in.alloc((size_t)nnz));
    GNNAGG_HIP(key_out.alloc((size_t)nnz));
    GNNAGG_HIP(idx_in.alloc((size_t)nnz));
    GNNAGG_HIP(idx_out.alloc((size_t)nnz));
    GNNAGG_HIP(bad.alloc(1));
    GNNAGG_HIP(hipMemsetAsync(bad.p, 0, sizeof(unsigned int), st));
    hipLaunchKernelGGL(pack_keys_kernel, dim3(grid_for(nnz, 256)), dim3(256), 0, st, row, col, nnz, rows, cols, col_bits,
                       key_in.p, idx_in.p, bad.p);
    GNNAGG_HIP(hipGetLastError());
    unsigned int h_bad = 0;
    GNNAGG_HIP(hipMemcpyAsync(&h_bad, bad.p, sizeof(unsigned int), hipMemcpyDeviceToHost, st));
    GNNAGG_HIP(hipStreamSynchronize(st));
    GNNAGG_REQUIRE(!h_bad, "a row/col index lies outside [0,%lld) x [0,%lld)", (long long)rows, (long long)cols);
    uint64_t *key_sorted = nullptr;
    uint32_t *idx_sorted = nullptr;
    if (int rc = sort_keys(key_in.p, key_out.p, idx_in.p, idx_out.p, nnz, col_bits + row_bits, st, &key_sorted, &idx_sorted))
        return rc;
    hipLaunchKernelGGL(unpack_sorted_kernel, dim3(grid_for(nnz, 256)), dim3(256), 0, st, key_sorted, idx_sorted, value,
                       nnz, col_bits, col_out, value_out);
    GNNAGG_HIP(hipGetLastError());
    hipLaunchKernelGGL(major_ptr_kernel, dim3(grid_for(rows + 1, 256)), dim3(256), 0, st, key_sorted, nnz, col_bits, rows,
                       rowptr);
    GNNAGG_HIP(hipGetLastError());
    GNNAGG_HIP(hipStreamSynchronize(st));
    return GNNAGG_OK;
}

extern "C" int gnnagg_csr_transpose(const int64_t *rowptr, const int64_t *col, const float *value, int64_t rows,
                                    int64_t cols, int64_t nnz, int64_t *colptr, int64_t *row_t, float *value_t,
                                    void *stream) {
    if (int rc = check_format_sizes(rows, cols, nnz)) return rc;
    GNNAGG_REQUIRE(rowptr && colptr, "null rowptr/colptr");
    GNNAGG_REQUIRE(nnz == 0 || (col && row_t), "null col/row_t");
    GNNAGG_REQUIRE((value == nullptr) == (value_t == nullptr), "value and value_t must both be given or both be null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (nnz == 0) {
        GNNAGG_HIP(hipMemsetAsync(colptr, 0, sizeof(int64_t) * (size_t)(cols + 1), st));
        GNNAGG_HIP(hipStreamSynchronize(st));
        return GNNAGG_OK;
    }
    int64_t ends[2] = {0, 0};
    GNNAGG_HIP(hipMemcpyAsync(&ends[0], rowptr, sizeof(int64_t), hipMemcpyDeviceToHost, st));
    GNNAGG_HIP(hipMemcpyAsync(&ends[1], rowptr + rows, sizeof(int64_t), hipMemcpyDeviceToHost, st));
    GNNAGG_HIP(hipStreamSynchronize(st));
    GNNAGG_REQUIRE(ends[0] == 0 && ends[1] == nnz, "rowptr[0]=%lld, rowptr[rows]=%lld do not match nnz=%lld",
                   (long long)ends[0], (long long)ends[1], (long long)nnz);
    const int col_bits = std::max(1, ceil_log2_u64((uint64_t)std::max<int64_t>(cols, 1)));
    const int row_bits = std::max(1, ceil_log2_u64((uint64_t)std::max<int64_t>(rows, 1)));
    DevBuf<uint64_t> key_in, key_out;
    DevBuf<uint32_t> idx_in, idx_out;
    DevBuf<unsigned int> bad;
    GNNAGG_HIP(key_in.alloc((size_t)nnz));
    GNNAGG_HIP(key_out.alloc((size_t)nnz));
    GNNAGG_HIP(idx_in.alloc((size_t)nnz));
    GNNAGG_HIP(idx_out.alloc((size_t)nnz));
    GNNAGG_HIP(bad.alloc(1));
    GNNAGG_HIP(hipMemsetAsync(bad.p, 0, sizeof(unsigned int), st));
    hipLaunchKernelGGL(pack_transposed_keys_kernel, dim3(grid_for(nnz, 256)), dim3(256), 0, st, rowptr, col, rows, cols,
                       nnz, row_bits, key_in.p, idx_in.p, bad.p);
    GNNAGG_HIP(hipGetLastError());
    unsigned int h_bad = 0;
    GNNAGG_HIP(hipMemcpyAsync(&h_bad, bad.p, sizeof(unsigned int), hipMemcpyDeviceToHost, st));
    GNNAGG_HIP(hipStreamSynchronize(st));
    GNNAGG_REQUIRE(!h_bad, "a column index lies outside [0,%lld)", (long long)cols);
    // (col, row) keys are unique per stored position up to repeated entries; the radix
    // sort is stable, so repeated (row, col) pairs keep their CSR order.
    uint64_t *key_sorted = nullptr;
    uint32_t *idx_sorted = nullptr;
    if (int rc = sort_keys(key_in.p, key_out.p, idx_in.p, idx_out.p, nnz, col_bits + row_bits, st, &key_sorted, &idx_sorted))
        return rc;
    hipLaunchKernelGGL(unpack_sorted_kernel, dim3(grid_for(nnz, 256)), dim3(256), 0, st, key_sorted, idx_sorted, value,
                       nnz, row_bits, row_t, value_t);
    GNNAGG_HIP(hipGetLastError());
    hipLaunchKernelGGL(major_ptr_kernel, dim3(grid_for(cols + 1, 256)), dim3(256), 0, st, key_sorted, nnz, row_bits, cols,
                       colptr);
    GNNAGG_HIP(hipGetLastError());
    GNNAGG_HIP(hipStreamSynchronize(st));
    return GNNAGG_OK;
}

extern "C" int gnnagg_gather_rows_f32(const float *src, int64_t src_rows, const int64_t *index, float *out,
                                      int64_t n_index, int64_t feat, void *stream) {
    GNNAGG_REQUIRE(n_index >= 0 && feat >= 0 && src_rows >= 0, "negative size");
    if (n_index == 0 || feat == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(src && index && out, "null src/index/out");
    GNNAGG_REQUIRE(src_rows > 0, "rows are asked of a source without rows");
    if (feat > (1 << 20)) return fail(GNNAGG_ERR_UNSUPPORTED, "feature width %lld above 2^20", (long long)feat);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uintptr_t bits = reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(out);
    if (feat % 4 == 0 && bits % 16 == 0)
        GNNAGG_HIP(launch_gather_rows<4>(src, src_rows, index, out, n_index, (int)(feat / 4), st));
    else if (feat % 2 == 0 && bits % 8 == 0)
        GNNAGG_HIP(launch_gather_rows<2>(src, src_rows, index, out, n_index, (int)(feat / 2), st));
    else
        GNNAGG_HIP(launch_gather_rows<1>(src, src_rows, index, out, n_index, (int)feat, st));
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

extern "C" int gnnagg_gather_rows_f32_bf16(const float *src, int64_t src_rows, const int64_t *index, void *out,
                                           int64_t n_index, int64_t feat, void *stream) {
    GNNAGG_REQUIRE(n_index >= 0 && feat >= 0 && src_rows >= 0, "negative size");
    if (n_index == 0 || feat == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(src && index && out, "null src/index/out");
    GNNAGG_REQUIRE(src_rows > 0, "rows are asked of a source without rows");
    if (feat > (1 << 20)) return fail(GNNAGG_ERR_UNSUPPORTED, "feature width %lld above 2^20", (long long)feat);
    if (feat % 4 != 0 || reinterpret_cast<uintptr_t>(src) % 16 != 0 || reinterpret_cast<uintptr_t>(out) % 8 != 0)
        return fail(GNNAGG_ERR_UNSUPPORTED,
                    "bf16 result rows need a width that is a multiple of 4 (got %lld), a 16-byte aligned source and "
                    "an 8-byte aligned result", (long long)feat);
    GNNAGG_HIP((launch_gather_rows<4, true>(src, src_rows, index, out, n_index, (int)(feat / 4),
                                            static_cast<hipStream_t>(stream))));
    return GNNAGG_OK;
}

extern "C" int gnnagg_check_index(const void *index, int elem_bytes, int64_t count, int shift, int64_t bound,
                                  void *stream) {
    GNNAGG_REQUIRE(elem_bytes == 4 || elem_bytes == 8, "index elements are 4 or 8 bytes wide (got %d)", elem_bytes);
    GNNAGG_REQUIRE(count >= 0 && bound >= 0 && shift >= 0 && shift < 8 * elem_bytes, "bad count / bound / shift");
    if (count == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(index, "null index");
    hipStream_t st = static_cast<hipStream_t>(stream);
    DevBuf<unsigned long long> first_bad;
    GNNAGG_HIP(first_bad.alloc(1));
    GNNAGG_HIP(hipMemsetAsync(first_bad.p, 0xff, sizeof(unsigned long long), st));
    const unsigned grid = (unsigned)std::min<int64_t>((count + 255) / 256, 256 * 16);
    if (elem_bytes == 8)
        hipLaunchKernelGGL(check_index_kernel<int64_t>, dim3(grid), dim3(256), 0, st, static_cast<const int64_t *>(index),
                           count, shift, bound, first_bad.p);
    else
        hipLaunchKernelGGL(check_index_kernel<int32_t>, dim3(grid), dim3(256), 0, st, static_cast<const int32_t *>(index),
                           count, shift, bound, first_bad.p);
    GNNAGG_HIP(hipGetLastError());
    unsigned long long h = ~0ull;
    GNNAGG_HIP(hipMemcpyAsync(&h, first_bad.p, sizeof(h), hipMemcpyDeviceToHost, st));
    GNNAGG_HIP(hipStreamSynchronize(st));
    GNNAGG_REQUIRE(h == ~0ull, "index %llu of %lld lies outside [0, %lld)%s", h, (long long)count, (long long)bound,
                   shift ? " (after the shift)" : "");
    return GNNAGG_OK;
}
