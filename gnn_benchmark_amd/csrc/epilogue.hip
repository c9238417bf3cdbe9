// Fused elementwise epilogue of a GCN layer around the aggregation path:
// y = relu(z + bias) * (keep ? scale : 0) and its gradient.  HBM-bound streaming
// kernels (one read and one write of the activation instead of four passes).
#include "common.h"

namespace gnnagg {
namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned char u8x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float relu_keep(float z, float b, unsigned char k, float scale) {
    const float a = z + b;
    const float r = a > 0.0f ? a : 0.0f;
    return k ? r * scale : 0.0f;
}

// n4 = rows * feat / 4 vectors; feat4 = feat / 4
__global__ __launch_bounds__(256) void bias_relu_dropout_v4_kernel(const f4 *__restrict__ z,
                                                                   const f4 *__restrict__ bias,
                                                                   const u8x4 *__restrict__ keep, float scale,
                                                                   f4 *__restrict__ y, int64_t n4, int feat4) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
        const f4 v = __builtin_nontemporal_load(z + i);
        const f4 b = bias[i % feat4];
        u8x4 k = {1, 1, 1, 1};
        if (keep) k = __builtin_nontemporal_load(keep + i);
        f4 r;
        r.x = relu_keep(v.x, b.x, k.x, scale);
        r.y = relu_keep(v.y, b.y, k.y, scale);
        r.z = relu_keep(v.z, b.z, k.z, scale);
        r.w = relu_keep(v.w, b.w, k.w, scale);
        __builtin_nontemporal_store(r, y + i);
    }
}

__global__ __launch_bounds__(256) void bias_relu_dropout_kernel(const float *__restrict__ z,
                                                                const float *__restrict__ bias,
                                                                const unsigned char *__restrict__ keep, float scale,
                                                                float *__restrict__ y, int64_t n, int feat) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        y[i] = relu_keep(z[i], bias[i % feat], keep ? keep[i] : (unsigned char)1, scale);
}

// gz = y > 0 ? g * scale : 0   (y is the OUTPUT of the forward: it is 0 exactly where the
// unit was inactive or dropped)
__global__ __launch_bounds__(256) void relu_dropout_backward_v4_kernel(const f4 *__restrict__ g,
                                                                       const f4 *__restrict__ y, float scale,
                                                                       f4 *__restrict__ gz, int64_t n4) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
        const f4 gv = __builtin_nontemporal_load(g + i);
        const f4 yv = __builtin_nontemporal_load(y + i);
        f4 r;
        r.x = yv.x > 0.0f ? gv.x * scale : 0.0f;
        r.y = yv.y > 0.0f ? gv.y * scale : 0.0f;
        r.z = yv.z > 0.0f ? gv.z * scale : 0.0f;
        r.w = yv.w > 0.0f ? gv.w * scale : 0.0f;
        __builtin_nontemporal_store(r, gz + i);
    }
}

__global__ __launch_bounds__(256) void relu_dropout_backward_kernel(const float *__restrict__ g,
                                                                    const float *__restrict__ y, float scale,
                                                                    float *__restrict__ gz, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        gz[i] = y[i] > 0.0f ? g[i] * scale : 0.0f;
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

extern "C" int gnnagg_bias_relu_dropout_f32(const float *z, const float *bias, const uint8_t *keep, float scale,
                                            float *y, int64_t rows, int64_t feat, void *stream) {
    GNNAGG_REQUIRE(rows >= 0 && feat >= 0, "negative size");
    if (rows == 0 || feat == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(z && bias && y, "null z/bias/y");
    if (feat > (1 << 20)) return fail(GNNAGG_ERR_UNSUPPORTED, "feature width %lld above 2^20", (long long)feat);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t n = rows * feat;
    if (feat % 4 == 0 && aligned16(z, bias, y) && (reinterpret_cast<uintptr_t>(keep) & 3) == 0) {
        hipLaunchKernelGGL(bias_relu_dropout_v4_kernel, dim3(stream_grid(n / 4)), dim3(256), 0, st,
                           reinterpret_cast<const f4 *>(z), reinterpret_cast<const f4 *>(bias),
                           reinterpret_cast<const u8x4 *>(keep), scale, reinterpret_cast<f4 *>(y), n / 4,
                           (int)(feat / 4));
    } else {
        hipLaunchKernelGGL(bias_relu_dropout_kernel, dim3(stream_grid(n)), dim3(256), 0, st, z, bias, keep, scale, y, n,
                           (int)feat);
    }
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

extern "C" int gnnagg_relu_dropout_backward_f32(const float *grad_y, const float *y, float scale, float *grad_z,
                                                int64_t count, void *stream) {
    GNNAGG_REQUIRE(count >= 0, "negative size");
    if (count == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(grad_y && y && grad_z, "null grad_y/y/grad_z");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (count % 4 == 0 && aligned16(grad_y, y, grad_z)) {
        hipLaunchKernelGGL(relu_dropout_backward_v4_kernel, dim3(stream_grid(count / 4)), dim3(256), 0, st,
                           reinterpret_cast<const f4 *>(grad_y), reinterpret_cast<const f4 *>(y), scale,
                           reinterpret_cast<f4 *>(grad_z), count / 4);
    } else {
        hipLaunchKernelGGL(relu_dropout_backward_kernel, dim3(stream_grid(count)), dim3(256), 0, st, grad_y, y, scale,
                           grad_z, count);
    }
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}
