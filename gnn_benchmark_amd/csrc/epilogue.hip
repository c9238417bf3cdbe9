// Fused elementwise epilogue of a GCN layer around the aggregation path:
// y = relu(z / row_div + bias) * (keep ? scale : 0) and its gradient.  HBM-bound streaming
// kernels (one read and one write of the activation instead of five passes).  The
// per-row divisor carries the mean-aggregation normalisation (1/in-degree), moved behind
// the dense product: D^-1 (A X) W == D^-1 ((A X) W).  A second forward variant writes its
// output packed (non-zero values at the front of each row + bitmap header) for the next
// layer's aggregation to gather, and the backward can take that bitmap in place of the output.
#include "common.h"

namespace gnnagg {
namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned char u8x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float relu_keep(float z, float d, float b, unsigned char k, float scale) {
    const float a = z / d + b;
    const float r = a > 0.0f ? a : 0.0f;
    return k ? r * scale : 0.0f;
}

// n4 = rows * feat / 4 vectors; feat4 = feat / 4
__global__ __launch_bounds__(256) void bias_relu_dropout_v4_kernel(const f4 *__restrict__ z,
                                                                   const f4 *__restrict__ bias,
                                                                   const u8x4 *__restrict__ keep,
                                                                   const float *__restrict__ row_div, float scale,
                                                                   f4 *__restrict__ y, int64_t n4, int feat4) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
        const f4 v = __builtin_nontemporal_load(z + i);
        const int64_t row = i / feat4;
        const f4 b = bias[i - row * feat4];
        const float d = row_div ? row_div[row] : 1.0f;
        u8x4 k = {1, 1, 1, 1};
        if (keep) k = __builtin_nontemporal_load(keep + i);
        f4 r;
        r.x = relu_keep(v.x, d, b.x, k.x, scale);
        r.y = relu_keep(v.y, d, b.y, k.y, scale);
        r.z = relu_keep(v.z, d, b.z, k.z, scale);
        r.w = relu_keep(v.w, d, b.w, k.w, scale);
        __builtin_nontemporal_store(r, y + i);
    }
}

__global__ __launch_bounds__(256) void bias_relu_dropout_kernel(const float *__restrict__ z,
                                                                const float *__restrict__ bias,
                                                                const unsigned char *__restrict__ keep,
                                                                const float *__restrict__ row_div, float scale,
                                                                float *__restrict__ y, int64_t n, int feat) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const int64_t row = i / feat;
        y[i] = relu_keep(z[i], row_div ? row_div[row] : 1.0f, bias[i - row * feat], keep ? keep[i] : (unsigned char)1,
                         scale);
    }
}

// gz = (y > 0 ? g * scale : 0) / row_div   (y is the OUTPUT of the forward: it is 0 exactly
// where the unit was inactive or dropped)
__global__ __launch_bounds__(256) void relu_dropout_backward_v4_kernel(const f4 *__restrict__ g,
                                                                       const f4 *__restrict__ y,
                                                                       const float *__restrict__ row_div, float scale,
                                                                       f4 *__restrict__ gz, int64_t n4, int feat4) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
        const f4 gv = __builtin_nontemporal_load(g + i);
        const f4 yv = __builtin_nontemporal_load(y + i);
        const float d = row_div ? row_div[i / feat4] : 1.0f;
        f4 r;
        r.x = yv.x > 0.0f ? gv.x * scale / d : 0.0f;
        r.y = yv.y > 0.0f ? gv.y * scale / d : 0.0f;
        r.z = yv.z > 0.0f ? gv.z * scale / d : 0.0f;
        r.w = yv.w > 0.0f ? gv.w * scale / d : 0.0f;
        __builtin_nontemporal_store(r, gz + i);
    }
}

__global__ __launch_bounds__(256) void relu_dropout_backward_kernel(const float *__restrict__ g,
                                                                    const float *__restrict__ y,
                                                                    const float *__restrict__ row_div, float scale,
                                                                    float *__restrict__ gz, int64_t n, int feat) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        gz[i] = y[i] > 0.0f ? g[i] * scale / (row_div ? row_div[i / feat] : 1.0f) : 0.0f;
}

// Same gradient, organised by rows so that the bias gradient comes out of the same pass:
// block b owns rows [b*rows_per_block, +rows_per_block); thread t owns the column vector
// t % feat4 and walks the rows t / feat4, + 256 / feat4, ...  Its running sum of the
// gradient BEFORE the row division (that is d/d bias) is reduced over the threads of the
// same column vector in a fixed order and written to bias_partial[b, :].  Needs
// feat4 <= 256 and 256 % feat4 == 0.
// PACKED: the forward output is not there as a dense tensor; which units were active comes from
// the bitmap words of each row's header (hdr_words 32-bit words per row, bitmaps at the even ones).
template <bool PACKED>
__global__ __launch_bounds__(256) void relu_dropout_backward_rows_kernel(const f4 *__restrict__ g,
                                                                         const void *__restrict__ y_or_hdr,
                                                                         const float *__restrict__ row_div, float scale,
                                                                         f4 *__restrict__ gz,
                                                                         f4 *__restrict__ bias_partial, int64_t rows,
                                                                         int feat4, int rows_per_block, int hdr_words) {
    __shared__ f4 sums[256];
    const int t = (int)threadIdx.x;
    const int c = t % feat4;
    const int lanes = 256 / feat4;  // rows in flight per block step
    const int64_t r_begin = (int64_t)blockIdx.x * rows_per_block;
    int64_t r_end = r_begin + rows_per_block;
    if (r_end > rows) r_end = rows;
    f4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int64_t r = r_begin + t / feat4; r < r_end; r += lanes) {
        const int64_t i = r * feat4 + c;
        const f4 gv = __builtin_nontemporal_load(g + i);
        bool on[4];
        if (PACKED) {
            const uint32_t w = static_cast<const uint32_t *>(y_or_hdr)[r * hdr_words + 2 * (c >> 3)];
            const uint32_t nib = (w >> (4 * (c & 7))) & 15u;
            on[0] = nib & 1u;
            on[1] = nib & 2u;
            on[2] = nib & 4u;
            on[3] = nib & 8u;
        } else {
            const f4 yv = __builtin_nontemporal_load(static_cast<const f4 *>(y_or_hdr) + i);
            on[0] = yv.x > 0.0f;
            on[1] = yv.y > 0.0f;
            on[2] = yv.z > 0.0f;
            on[3] = yv.w > 0.0f;
        }
        const float d = row_div ? row_div[r] : 1.0f;
        f4 pre;
        pre.x = on[0] ? gv.x * scale : 0.0f;
        pre.y = on[1] ? gv.y * scale : 0.0f;
        pre.z = on[2] ? gv.z * scale : 0.0f;
        pre.w = on[3] ? gv.w * scale : 0.0f;
        acc += pre;
        f4 out;
        out.x = pre.x / d;
        out.y = pre.y / d;
        out.z = pre.z / d;
        out.w = pre.w / d;
        __builtin_nontemporal_store(out, gz + i);
    }
    sums[t] = acc;
    __syncthreads();
    if (t < feat4) {
        f4 total = sums[t];
        for (int k = 1; k < lanes; ++k) total += sums[t + k * feat4];
        bias_partial[(int64_t)blockIdx.x * feat4 + t] = total;
    }
}

// ---- packed activations -----------------------------------------------------------------
// The output of a ReLU + dropout layer is mostly zeros (about three in four in training).  A
// row can be stored with its non-zero values moved to the front (order kept; the tail of the
// row is left as it is) plus a small header: for every 32 features a pair of 32-bit words, the
// bitmap of those features and the number of non-zeros in front of them.  The row stride stays
// F, so no offsets are needed; a consumer that gathers such a row touches only the header
// (64 bytes at F = 256) and the non-zero values.  F = 4 * G with G lanes per row in {8, 16, 32, 64}.
constexpr int packed_header_words(int feat) { return 2 * (feat / 32); }

template <int G>
__global__ __launch_bounds__(256) void bias_relu_dropout_pack_kernel(const f4 *__restrict__ z,
                                                                     const f4 *__restrict__ bias,
                                                                     const u8x4 *__restrict__ keep,
                                                                     const float *__restrict__ row_div, float scale,
                                                                     float *__restrict__ yp, uint32_t *__restrict__ hdr,
                                                                     int64_t rows) {
    constexpr int F = 4 * G;
    constexpr int HW = packed_header_words(F);
    const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) / G;
    if (row >= rows) return;               // whole rows (lane groups) leave together
    const int l = (int)threadIdx.x & (G - 1);
    const int64_t i = row * G + l;
    const f4 v = __builtin_nontemporal_load(z + i);
    const f4 b = bias[l];
    const float d = row_div ? row_div[row] : 1.0f;
    u8x4 k = {1, 1, 1, 1};
    if (keep) k = __builtin_nontemporal_load(keep + i);
    float y[4];
    y[0] = relu_keep(v.x, d, b.x, k.x, scale);
    y[1] = relu_keep(v.y, d, b.y, k.y, scale);
    y[2] = relu_keep(v.z, d, b.z, k.z, scale);
    y[3] = relu_keep(v.w, d, b.w, k.w, scale);
    uint32_t nib = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) nib |= (y[e] > 0.0f ? 1u : 0u) << e;
    const int cnt = __popc(nib);
    int incl = cnt;                        // inclusive scan of the counts over the row's lanes
#pragma unroll
    for (int s = 1; s < G; s <<= 1) {
        const int t = __shfl_up(incl, s, G);
        if (l >= s) incl += t;
    }
    const int excl = incl - cnt;
    float *dst = yp + (size_t)row * F + excl;
    int at = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e)
        if (nib & (1u << e)) dst[at++] = y[e];

    uint32_t word = nib << (4 * (l & 7));  // eight lanes make one bitmap word
    word |= __shfl_xor(word, 1, G);
    word |= __shfl_xor(word, 2, G);
    word |= __shfl_xor(word, 4, G);
    if ((l & 7) == 0) {                    // this lane's exclusive count = non-zeros in front of its word
        uint2 pair;
        pair.x = word;
        pair.y = (uint32_t)excl;
        *reinterpret_cast<uint2 *>(hdr + row * HW + 2 * (l >> 3)) = pair;
    }
}

unsigned stream_grid(int64_t n_items) {
    const int64_t blocks = (n_items + 255) / 256;
    return (unsigned)(blocks < 256 * 64 ? (blocks > 0 ? blocks : 1) : 256 * 64);  // 64 blocks per CU, grid-stride
}

bool aligned16(const void *a, const void *b, const void *c) {
    return ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 15) == 0;
}

}  // namespace
}  // namespace gnnagg

using namespace gnnagg;

extern "C" int gnnagg_bias_relu_dropout_f32(const float *z, const float *bias, const uint8_t *keep,
                                            const float *row_div, float scale, float *y, int64_t rows, int64_t feat,
                                            void *stream) {
    GNNAGG_REQUIRE(rows >= 0 && feat >= 0, "negative size");
    if (rows == 0 || feat == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(z && bias && y, "null z/bias/y");
    if (feat > (1 << 20)) return fail(GNNAGG_ERR_UNSUPPORTED, "feature width %lld above 2^20", (long long)feat);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t n = rows * feat;
    if (feat % 4 == 0 && aligned16(z, bias, y) && (reinterpret_cast<uintptr_t>(keep) & 3) == 0) {
        hipLaunchKernelGGL(bias_relu_dropout_v4_kernel, dim3(stream_grid(n / 4)), dim3(256), 0, st,
                           reinterpret_cast<const f4 *>(z), reinterpret_cast<const f4 *>(bias),
                           reinterpret_cast<const u8x4 *>(keep), row_div, scale, reinterpret_cast<f4 *>(y), n / 4,
                           (int)(feat / 4));
    } else {
        hipLaunchKernelGGL(bias_relu_dropout_kernel, dim3(stream_grid(n)), dim3(256), 0, st, z, bias, keep, row_div,
                           scale, y, n, (int)feat);
    }
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

extern "C" int gnnagg_relu_dropout_backward_blocks(int64_t rows, int64_t feat) {
    if (rows <= 0 || feat <= 0 || feat % 4 != 0 || feat / 4 > 256 || 256 % (feat / 4) != 0) return 0;
    const int64_t target = 256 * 16;  // blocks: enough to fill the chip, few enough to sum cheaply
    const int64_t rpb = (rows + target - 1) / target;
    return (int)((rows + rpb - 1) / rpb);
}

extern "C" int gnnagg_relu_dropout_backward_f32(const float *grad_y, const float *y, const float *row_div, float scale,
                                                float *grad_z, float *bias_partial, int64_t rows, int64_t feat,
                                                void *stream) {
    GNNAGG_REQUIRE(rows >= 0 && feat >= 0, "negative size");
    if (rows == 0 || feat == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(grad_y && y && grad_z, "null grad_y/y/grad_z");
    if (feat > (1 << 20)) return fail(GNNAGG_ERR_UNSUPPORTED, "feature width %lld above 2^20", (long long)feat);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t count = rows * feat;
    if (bias_partial) {
        const int blocks = gnnagg_relu_dropout_backward_blocks(rows, feat);
        GNNAGG_REQUIRE(blocks > 0, "bias partial sums need feat %% 4 == 0 and 256 %% (feat / 4) == 0 (feat=%lld)",
                       (long long)feat);
        GNNAGG_REQUIRE(aligned16(grad_y, y, grad_z) && (reinterpret_cast<uintptr_t>(bias_partial) & 15) == 0,
                       "bias partial sums need 16-byte aligned operands");
        const int64_t rpb = (rows + blocks - 1) / blocks;
        hipLaunchKernelGGL(relu_dropout_backward_rows_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, st,
                           reinterpret_cast<const f4 *>(grad_y), static_cast<const void *>(y), row_div, scale,
                           reinterpret_cast<f4 *>(grad_z), reinterpret_cast<f4 *>(bias_partial), rows, (int)(feat / 4),
                           (int)rpb, 0);
        GNNAGG_HIP(hipGetLastError());
        return GNNAGG_OK;
    }
    if (feat % 4 == 0 && aligned16(grad_y, y, grad_z)) {
        hipLaunchKernelGGL(relu_dropout_backward_v4_kernel, dim3(stream_grid(count / 4)), dim3(256), 0, st,
                           reinterpret_cast<const f4 *>(grad_y), reinterpret_cast<const f4 *>(y), row_div, scale,
                           reinterpret_cast<f4 *>(grad_z), count / 4, (int)(feat / 4));
    } else {
        hipLaunchKernelGGL(relu_dropout_backward_kernel, dim3(stream_grid(count)), dim3(256), 0, st, grad_y, y, row_div,
                           scale, grad_z, count, (int)feat);
    }
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

extern "C" int gnnagg_packed_header_words(int64_t feat) {
    if (feat != 32 && feat != 64 && feat != 128 && feat != 256) return 0;
    return packed_header_words((int)feat);
}

extern "C" int gnnagg_bias_relu_dropout_pack_f32(const float *z, const float *bias, const uint8_t *keep,
                                                 const float *row_div, float scale, float *y_packed, uint32_t *header,
                                                 int64_t rows, int64_t feat, void *stream) {
    GNNAGG_REQUIRE(rows >= 0, "negative size");
    if (gnnagg_packed_header_words(feat) == 0)
        return fail(GNNAGG_ERR_UNSUPPORTED, "packed activations exist for widths 32, 64, 128, 256 (got %lld)",
                    (long long)feat);
    if (rows == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(z && bias && y_packed && header, "null z/bias/y_packed/header");
    GNNAGG_REQUIRE(aligned16(z, bias, bias) && (reinterpret_cast<uintptr_t>(keep) & 3) == 0 &&
                       (reinterpret_cast<uintptr_t>(y_packed) & 3) == 0,
                   "packed epilogue needs 16-byte aligned z / bias and a 4-byte aligned mask");
    GNNAGG_REQUIRE(rows < (int64_t(1) << 31), "too many rows");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int g = (int)(feat / 4);
    const unsigned blocks = grid_for(rows * g, 256);
#define GNNAGG_PACK(G)                                                                                          \
    if (g == G)                                                                                                 \
        hipLaunchKernelGGL(bias_relu_dropout_pack_kernel<G>, dim3(blocks), dim3(256), 0, st,                    \
                           reinterpret_cast<const f4 *>(z), reinterpret_cast<const f4 *>(bias),                 \
                           reinterpret_cast<const u8x4 *>(keep), row_div, scale, y_packed, header, rows)
    GNNAGG_PACK(8);
    GNNAGG_PACK(16);
    GNNAGG_PACK(32);
    GNNAGG_PACK(64);
#undef GNNAGG_PACK
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

extern "C" int gnnagg_relu_dropout_backward_packed_f32(const float *grad_y, const uint32_t *header, const float *row_div,
                                                       float scale, float *grad_z, float *bias_partial, int64_t rows,
                                                       int64_t feat, void *stream) {
    GNNAGG_REQUIRE(rows >= 0, "negative size");
    const int hw = gnnagg_packed_header_words(feat);
    if (hw == 0)
        return fail(GNNAGG_ERR_UNSUPPORTED, "packed activations exist for widths 32, 64, 128, 256 (got %lld)",
                    (long long)feat);
    if (rows == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(grad_y && header && grad_z && bias_partial, "null grad_y/header/grad_z/bias_partial");
    GNNAGG_REQUIRE(aligned16(grad_y, grad_z, bias_partial), "packed backward needs 16-byte aligned operands");
    const int blocks = gnnagg_relu_dropout_backward_blocks(rows, feat);
    const int64_t rpb = (rows + blocks - 1) / blocks;
    hipLaunchKernelGGL(relu_dropout_backward_rows_kernel<true>, dim3((unsigned)blocks), dim3(256), 0,
                       static_cast<hipStream_t>(stream), reinterpret_cast<const f4 *>(grad_y),
                       static_cast<const void *>(header), row_div, scale, reinterpret_cast<f4 *>(grad_z),
                       reinterpret_cast<f4 *>(bias_partial), rows, (int)(feat / 4), (int)rpb, hw);
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}
