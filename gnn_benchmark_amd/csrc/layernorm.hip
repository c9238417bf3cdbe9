// The elementwise chain between two SAGE layers -- dropout, LayerNorm over the features,
// ReLU (model/DistSAGE.py:49-53) -- as one streaming pass each way.  HBM-bound: the forward
// reads the layer output and the keep mask once and writes the next layer's input once; the
// backward reads the incoming gradient, the saved layer output and the mask once, takes the
// row's moments again from the registers that hold it (nothing but the layer output is kept
// from the forward), writes the gradient once, and leaves the per-feature sums for the
// LayerNorm weight / bias gradients as per-block partial sums taken in a fixed order.
//
// One group of LPR lanes owns a row; a lane holds NV float4 of it (features 4*(l + k*LPR)...),
// so a row is read exactly once and both moments are taken from registers.  The output row may
// sit inside a wider row-major array (row stride in floats), and so may the incoming gradient:
// the next layer keeps [aggregated | own] features side by side.
#include <type_traits>

#include "common.h"

namespace gnnagg {
namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned char u8x4 __attribute__((ext_vector_type(4)));

template <int LPR>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int s = LPR / 2; s >= 1; s >>= 1) v += __shfl_xor(v, s, LPR);
    return v;  // the same value (same summation tree) on every lane of the group
}

// What both directions need of a row: the dropped-out input d, its moments, the normalised
// value xhat.  Kept in one place so that forward and backward decide "n > 0" from the same
// arithmetic.
template <int LPR, int NV>
struct RowState {
    f4 d[NV];
    bool ok[NV];
    float mean, rstd;

    __device__ __forceinline__ void load(const f4 *__restrict__ z, const u8x4 *__restrict__ keep, float scale,
                                         int64_t row, int feat4, int l) {
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int c = l + k * LPR;
            ok[k] = c < feat4;
            f4 v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (ok[k]) {
                const int64_t i = row * feat4 + c;
                v = __builtin_nontemporal_load(z + i);
                if (keep) {
                    const u8x4 m = __builtin_nontemporal_load(keep + i);
                    v.x = m.x ? v.x * scale : 0.0f;
                    v.y = m.y ? v.y * scale : 0.0f;
                    v.z = m.z ? v.z * scale : 0.0f;
                    v.w = m.w ? v.w * scale : 0.0f;
                }
            }
            d[k] = v;
        }
    }
    __device__ __forceinline__ void moments(float inv_feat, float eps) {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < NV; ++k) s += (d[k].x + d[k].y) + (d[k].z + d[k].w);  // zeros where !ok
        mean = group_sum<LPR>(s) * inv_feat;
        float q = 0.0f;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            if (!ok[k]) continue;
            const f4 e = d[k] - mean;
            q += (e.x * e.x + e.y * e.y) + (e.z * e.z + e.w * e.w);
        }
        const float var = group_sum<LPR>(q) * inv_feat;  // biased, as LayerNorm defines it
        rstd = 1.0f / __builtin_sqrtf(var + eps);
    }
    __device__ __forceinline__ f4 xhat(int k) const { return (d[k] - mean) * rstd; }
};

__device__ __forceinline__ f4 affine(const f4 xh, const f4 gamma, const f4 beta) {
    f4 n;
    n.x = __builtin_fmaf(xh.x, gamma.x, beta.x);
    n.y = __builtin_fmaf(xh.y, gamma.y, beta.y);
    n.z = __builtin_fmaf(xh.z, gamma.z, beta.z);
    n.w = __builtin_fmaf(xh.w, gamma.w, beta.w);
    return n;
}

template <int LPR, int NV>
__global__ __launch_bounds__(256) void dropout_layernorm_relu_kernel(const f4 *__restrict__ z,
                                                                     const u8x4 *__restrict__ keep, float scale,
                                                                     const f4 *__restrict__ gamma,
                                                                     const f4 *__restrict__ beta, float eps,
                                                                     float *__restrict__ y, int64_t ldy,
                                                                     int64_t rows, int feat4) {
    constexpr int kGroups = 256 / LPR;
    const int l = (int)threadIdx.x % LPR;
    const float inv_feat = 1.0f / (float)(4 * feat4);
    f4 gm[NV], bt[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int c = l + k * LPR;
        const f4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
        gm[k] = c < feat4 ? gamma[c] : zero;
        bt[k] = c < feat4 ? beta[c] : zero;
    }
    // whole lane groups stay or leave together: the shuffles inside never see a missing lane
    for (int64_t row = (int64_t)blockIdx.x * kGroups + (int)threadIdx.x / LPR; row < rows;
         row += (int64_t)gridDim.x * kGroups) {
        RowState<LPR, NV> st;
        st.load(z, keep, scale, row, feat4, l);
        st.moments(inv_feat, eps);
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            if (!st.ok[k]) continue;
            const f4 n = affine(st.xhat(k), gm[k], bt[k]);
            f4 r;
            r.x = n.x > 0.0f ? n.x : 0.0f;
            r.y = n.y > 0.0f ? n.y : 0.0f;
            r.z = n.z > 0.0f ? n.z : 0.0f;
            r.w = n.w > 0.0f ? n.w : 0.0f;
            __builtin_nontemporal_store(r, reinterpret_cast<f4 *>(y + row * ldy) + (l + k * LPR));
        }
    }
}

// Block b owns rows [b * rows_per_block, + rows_per_block); its lane groups walk them with a
// fixed stride, so a thread always meets the same features and can keep running sums of
// d/d gamma = g_n * xhat and d/d beta = g_n (g_n: the gradient behind the ReLU).  At the end
// the groups' sums are added in group order and written to partial[b, 0, :] / partial[b, 1, :].
template <int LPR, int NV>
__global__ __launch_bounds__(256) void dropout_layernorm_relu_backward_kernel(
    const float *__restrict__ g, int64_t ldg, const f4 *__restrict__ z, const u8x4 *__restrict__ keep, float scale,
    const f4 *__restrict__ gamma, const f4 *__restrict__ beta, float eps, f4 *__restrict__ gz,
    f4 *__restrict__ partial, int64_t rows, int feat4, int64_t rows_per_block) {
    constexpr int kGroups = 256 / LPR;
    __shared__ f4 sums[2][NV][256];
    const int t = (int)threadIdx.x;
    const int l = t % LPR;
    const float inv_feat = 1.0f / (float)(4 * feat4);
    const f4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    f4 gm[NV], bt[NV], acc_gamma[NV], acc_beta[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int c = l + k * LPR;
        gm[k] = c < feat4 ? gamma[c] : zero;
        bt[k] = c < feat4 ? beta[c] : zero;
        acc_gamma[k] = zero;
        acc_beta[k] = zero;
    }
    const int64_t r_begin = (int64_t)blockIdx.x * rows_per_block;
    int64_t r_end = r_begin + rows_per_block;
    if (r_end > rows) r_end = rows;
    for (int64_t row = r_begin + t / LPR; row < r_end; row += kGroups) {
        RowState<LPR, NV> st;
        st.load(z, keep, scale, row, feat4, l);
        st.moments(inv_feat, eps);
        f4 xh[NV], dxh[NV];
        float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            xh[k] = zero;
            dxh[k] = zero;
            if (!st.ok[k]) continue;
            xh[k] = st.xhat(k);
            const f4 n = affine(xh[k], gm[k], bt[k]);
            const f4 gv = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(g + row * ldg) + (l + k * LPR));
            f4 gn;
            gn.x = n.x > 0.0f ? gv.x : 0.0f;
            gn.y = n.y > 0.0f ? gv.y : 0.0f;
            gn.z = n.z > 0.0f ? gv.z : 0.0f;
            gn.w = n.w > 0.0f ? gv.w : 0.0f;
            acc_gamma[k] += gn * xh[k];
            acc_beta[k] += gn;
            dxh[k] = gn * gm[k];
            s1 += (dxh[k].x + dxh[k].y) + (dxh[k].z + dxh[k].w);
            const f4 p = dxh[k] * xh[k];
            s2 += (p.x + p.y) + (p.z + p.w);
        }
        const float m1 = group_sum<LPR>(s1) * inv_feat;
        const float m2 = group_sum<LPR>(s2) * inv_feat;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            if (!st.ok[k]) continue;
            f4 dd = (dxh[k] - m1 - xh[k] * m2) * st.rstd;  // gradient with respect to the dropped-out input
            const int64_t i = row * feat4 + (l + k * LPR);
            if (keep) {
                const u8x4 m = keep[i];  // second touch of these 4 bytes: served by the cache
                dd.x = m.x ? dd.x * scale : 0.0f;
                dd.y = m.y ? dd.y * scale : 0.0f;
                dd.z = m.z ? dd.z * scale : 0.0f;
                dd.w = m.w ? dd.w * scale : 0.0f;
            }
            __builtin_nontemporal_store(dd, gz + i);
        }
    }
    if (!partial) return;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        sums[0][k][t] = acc_gamma[k];
        sums[1][k][t] = acc_beta[k];
    }
    __syncthreads();
    if (t < LPR) {
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int c = t + k * LPR;
            if (c >= feat4) continue;
            f4 tg = sums[0][k][t], tb = sums[1][k][t];
            for (int q = 1; q < kGroups; ++q) {
                tg += sums[0][k][t + q * LPR];
                tb += sums[1][k][t + q * LPR];
            }
            partial[((int64_t)blockIdx.x * 2 + 0) * feat4 + c] = tg;
            partial[((int64_t)blockIdx.x * 2 + 1) * feat4 + c] = tb;
        }
    }
}

struct RowShape {
    int lpr, nv;
};

// lanes per row and float4 per lane for a width (feat % 4 == 0, feat <= 1024); lpr == 0: none
RowShape row_shape(int64_t feat) {
    if (feat <= 0 || feat % 4 != 0 || feat > 1024) return RowShape{0, 0};
    const int feat4 = (int)(feat / 4);
    for (int lpr = 8; lpr <= 64; lpr *= 2)
        if (feat4 <= lpr) return RowShape{lpr, 1};
    return RowShape{64, (feat4 + 63) / 64};
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename F>
bool for_shape(const RowShape s, F &&launch) {
#define GNNAGG_LN_SHAPE(L, N)                          \
    if (s.lpr == L && s.nv == N) {                     \
        launch(std::integral_constant<int, L>(), std::integral_constant<int, N>()); \
        return true;                                   \
    }
    GNNAGG_LN_SHAPE(8, 1)
    GNNAGG_LN_SHAPE(16, 1)
    GNNAGG_LN_SHAPE(32, 1)
    GNNAGG_LN_SHAPE(64, 1)
    GNNAGG_LN_SHAPE(64, 2)
    GNNAGG_LN_SHAPE(64, 3)
    GNNAGG_LN_SHAPE(64, 4)
#undef GNNAGG_LN_SHAPE
    return false;
}

}  // namespace
}  // namespace gnnagg

using namespace gnnagg;

extern "C" int gnnagg_dropout_layernorm_relu_blocks(int64_t rows, int64_t feat) {
    if (rows <= 0 || row_shape(feat).lpr == 0) return 0;
    const int64_t target = 256 * 16;  // blocks: enough to fill the chip, few enough to sum cheaply
    const int64_t rpb = (rows + target - 1) / target;
    return (int)((rows + rpb - 1) / rpb);
}

extern "C" int gnnagg_dropout_layernorm_relu_f32(const float *z, const uint8_t *keep, float scale, const float *gamma,
                                                 const float *beta, float eps, float *y, int64_t y_stride,
                                                 int64_t rows, int64_t feat, void *stream) {
    GNNAGG_REQUIRE(rows >= 0, "negative size");
    const RowShape s = row_shape(feat);
    if (s.lpr == 0)
        return fail(GNNAGG_ERR_UNSUPPORTED, "the fused LayerNorm pass takes widths that are multiples of 4 up to 1024 "
                    "(got %lld)", (long long)feat);
    if (rows == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(z && gamma && beta && y, "null z/gamma/beta/y");
    GNNAGG_REQUIRE(y_stride >= feat && y_stride % 4 == 0, "output row stride %lld must be a multiple of 4 and at least "
                   "the width", (long long)y_stride);
    GNNAGG_REQUIRE(aligned16(z) && aligned16(gamma) && aligned16(beta) && aligned16(y) &&
                       (reinterpret_cast<uintptr_t>(keep) & 3) == 0,
                   "the fused LayerNorm pass needs 16-byte aligned rows and a 4-byte aligned mask");
    const int feat4 = (int)(feat / 4);
    hipStream_t st = static_cast<hipStream_t>(stream);
    for_shape(s, [&](auto L, auto N) {
        constexpr int kGroups = 256 / decltype(L)::value;
        const int64_t need = (rows + kGroups - 1) / kGroups;
        const unsigned blocks = (unsigned)(need < 256 * 32 ? need : 256 * 32);
        hipLaunchKernelGGL((dropout_layernorm_relu_kernel<decltype(L)::value, decltype(N)::value>), dim3(blocks),
                           dim3(256), 0, st, reinterpret_cast<const f4 *>(z), reinterpret_cast<const u8x4 *>(keep),
                           scale, reinterpret_cast<const f4 *>(gamma), reinterpret_cast<const f4 *>(beta), eps, y,
                           y_stride, rows, feat4);
    });
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

extern "C" int gnnagg_dropout_layernorm_relu_backward_f32(const float *grad_y, int64_t grad_stride, const float *z,
                                                          const uint8_t *keep, float scale, const float *gamma,
                                                          const float *beta, float eps, float *grad_z,
                                                          float *partial, int64_t rows, int64_t feat, void *stream) {
    GNNAGG_REQUIRE(rows >= 0, "negative size");
    const RowShape s = row_shape(feat);
    if (s.lpr == 0)
        return fail(GNNAGG_ERR_UNSUPPORTED, "the fused LayerNorm pass takes widths that are multiples of 4 up to 1024 "
                    "(got %lld)", (long long)feat);
    if (rows == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(grad_y && z && gamma && beta && grad_z && partial, "null grad_y/z/gamma/beta/grad_z/partial");
    GNNAGG_REQUIRE(grad_stride >= feat && grad_stride % 4 == 0, "gradient row stride %lld must be a multiple of 4 and "
                   "at least the width", (long long)grad_stride);
    GNNAGG_REQUIRE(aligned16(grad_y) && aligned16(z) && aligned16(gamma) && aligned16(beta) && aligned16(grad_z) &&
                       aligned16(partial) && (reinterpret_cast<uintptr_t>(keep) & 3) == 0,
                   "the fused LayerNorm pass needs 16-byte aligned rows and a 4-byte aligned mask");
    const int blocks = gnnagg_dropout_layernorm_relu_blocks(rows, feat);
    const int64_t rpb = (rows + blocks - 1) / blocks;
    const int feat4 = (int)(feat / 4);
    hipStream_t st = static_cast<hipStream_t>(stream);
    for_shape(s, [&](auto L, auto N) {
        hipLaunchKernelGGL((dropout_layernorm_relu_backward_kernel<decltype(L)::value, decltype(N)::value>),
                           dim3((unsigned)blocks), dim3(256), 0, st, grad_y, grad_stride,
                           reinterpret_cast<const f4 *>(z), reinterpret_cast<const u8x4 *>(keep), scale,
                           reinterpret_cast<const f4 *>(gamma), reinterpret_cast<const f4 *>(beta), eps,
                           reinterpret_cast<f4 *>(grad_z), reinterpret_cast<f4 *>(partial), rows, feat4, rpb);
    });
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}
