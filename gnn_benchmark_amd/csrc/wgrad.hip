// Weight-gradient product of a GCN layer, W_grad[Fi, Fo] = X^T[Fi, N] @ G[N, Fo], for
// N in the millions and Fi, Fo <= 256: a reduction over the rows of two tall-skinny
// row-major matrices.  fp32 MFMA (v_mfma_f32_32x32x2f32): 2*N*Fi*Fo flop against the
// 157.3 TFLOP/s fp32 matrix peak, 4*N*(Fi+Fo) bytes against HBM.
//
// A block of four waves owns the whole Fi x Fo output (each wave a (32*WM) x (32*WN)
// corner, accumulators in AGPRs) for one contiguous slice of the rows, so X and G are
// read from memory exactly once.  kChunk rows of X and of G are one contiguous run of
// memory each; the block copies them with 16-byte loads into LDS (register-staged, the
// next chunk in flight behind the MFMAs of the current one, two LDS buffers, one barrier
// per chunk) and every wave picks its operands out of LDS.  Both operands are already in
// MFMA operand order there: for a fixed row r the A operand wants X[r][m] across lanes m
// and the B operand wants G[r][n] across lanes n, so no transpose is needed.  Per-slice
// partial outputs are added up in slice order by a second kernel (deterministic, no
// atomics).
#include "common.h"
#include "dense_tiles.h"

namespace gnnagg {
namespace {

template <int WM, int WN>
struct WgradShape {
    static constexpr int kLdx = 64 * WM + kLdsPad;
    static constexpr int kLdg = 64 * WN + kLdsPad;
    static constexpr int kVecX = WM * kChunk / 16;  // float4 per thread per chunk of X
    static constexpr int kVecG = WN * kChunk / 16;
    static constexpr int kSmemFloats = 2 * kChunk * (kLdx + kLdg) + 256 * 4;  // + 16 bytes per thread to dump into
};

template <int WM, int WN>
__global__ __launch_bounds__(256, 1) void wgrad_partial_kernel(const float *__restrict__ x,
                                                               const float *__restrict__ g,
                                                               float *__restrict__ partial, int64_t rows, int fi,
                                                               int fo, int ldx, int ldg, int64_t rows_per_block,
                                                               int aligned) {
    using S = WgradShape<WM, WN>;
    extern __shared__ __align__(16) float smem[];
    float *xs = smem;                              // [2][kChunk][kLdx]
    float *gs = smem + 2 * kChunk * S::kLdx;       // [2][kChunk][kLdg]
    float *dump = smem + 2 * kChunk * (S::kLdx + S::kLdg) + 4 * (int)threadIdx.x;

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;               // 2 x 2 waves over the output
    const int wm = wave >> 1, wn = wave & 1;
    const int kk = lane >> 5;                // which of the two rows of a k-pair this lane feeds
    const int idx = lane & 31;
    const int m0 = wm * 32 * WM, n0 = wn * 32 * WN;

    floatx16 acc[WM][WN];
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int b = 0; b < WN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    const int64_t r_begin = (int64_t)blockIdx.x * rows_per_block;
    int64_t r_end = r_begin + rows_per_block;
    if (r_end > rows) r_end = rows;
    const int64_t slice = r_begin < r_end ? r_end - r_begin : 0;
    // 16-byte copies need whole float4 per row and aligned bases; otherwise every chunk takes the
    // element-wise path below.
    const int64_t full = aligned ? slice / kChunk : 0;

    ChunkLoader<S::kVecX, S::kLdx> lx;
    ChunkLoader<S::kVecG, S::kLdg> lg;
    lx.init(tid, fi, ldx);
    lg.init(tid, fo, ldg);

    // Columns past fi / fo of an LDS row are never written: whatever they hold only reaches
    // accumulator entries that are never stored.
    auto multiply = [&](int buf) {
        const float *xa = xs + buf * kChunk * S::kLdx + kk * S::kLdx + m0 + idx;
        const float *gb = gs + buf * kChunk * S::kLdg + kk * S::kLdg + n0 + idx;
        // operands of k-pair s+1 are read from LDS while the MFMAs of k-pair s run
        float a[2][WM], b[2][WN];
        auto read = [&](int s, float (&av)[WM], float (&bv)[WN]) {
#pragma unroll
            for (int i = 0; i < WM; ++i) av[i] = xa[2 * s * S::kLdx + 32 * i];
#pragma unroll
            for (int j = 0; j < WN; ++j) bv[j] = gb[2 * s * S::kLdg + 32 * j];
        };
        read(0, a[0], b[0]);
#pragma unroll
        for (int s = 0; s < kChunk / 2; ++s) {
            if (s + 1 < kChunk / 2) read(s + 1, a[(s + 1) & 1], b[(s + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int j = 0; j < WN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s & 1][i], b[s & 1][j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // steady state: whole chunks, no masks; the next chunk's global loads are in flight behind
    // this chunk's MFMAs and land in the other LDS buffer
    if (full > 0) {
        const float *xc = x + (size_t)r_begin * (size_t)ldx;
        const float *gc = g + (size_t)r_begin * (size_t)ldg;
        const size_t xstep = (size_t)kChunk * (size_t)ldx, gstep = (size_t)kChunk * (size_t)ldg;
        lx.fetch(xc);
        lg.fetch(gc);
        lx.store_all(xs, dump);
        lg.store_all(gs, dump);
        __syncthreads();
        for (int64_t c = 1; c < full; ++c) {
            xc += xstep;
            gc += gstep;
            lx.fetch(xc);
            lg.fetch(gc);
            __builtin_amdgcn_sched_barrier(0);  // keep the loads ahead of the MFMAs
            multiply((int)((c - 1) & 1));
            lx.store_all(xs + (c & 1) * kChunk * S::kLdx, dump);
            lg.store_all(gs + (c & 1) * kChunk * S::kLdg, dump);
            __syncthreads();
        }
        multiply((int)((full - 1) & 1));
        __syncthreads();
    }
    // what is left: the slice's last, partial chunk, or every chunk when 16-byte copies are not possible
    for (int64_t r = r_begin + full * kChunk; r < r_end; r += kChunk) {
        const int left = (int)(r_end - r < kChunk ? r_end - r : kChunk);
        lx.fetch_tail(x + (size_t)r * (size_t)ldx, left * fi, aligned != 0);
        lg.fetch_tail(g + (size_t)r * (size_t)ldg, left * fo, aligned != 0);
        lx.store(xs, aligned != 0);
        lg.store(gs, aligned != 0);
        __syncthreads();
        multiply(0);
        __syncthreads();
    }

    // 32x32 accumulator layout: register r of lane l holds D[(r % 4) + 4 * (l / 32) + 8 * (r / 4)][l % 32]
    float *out = partial + (size_t)blockIdx.x * (size_t)fi * (size_t)fo;
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int b = 0; b < WN; ++b) {
            const int n = n0 + b * 32 + idx;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + a * 32 + (r & 3) + 4 * kk + 8 * (r >> 2);
                if (m < fi && n < fo) out[(size_t)m * fo + n] = acc[a][b][r];
            }
        }
}

// out[i] = sum over the slices of partial[slice][i], in a fixed order: eight threads share an output,
// thread s adds the slices s, s + 8, ... and the eight sums are added in order of s.  (A block covers 32
// outputs, so that even a 128 x 128 result is spread over 512 blocks.)
constexpr int kReduceOutputs = 32;
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const float *__restrict__ partial, float *__restrict__ out,
                                                           int blocks, int count) {
    __shared__ float part[8][kReduceOutputs];
    const int o = (int)threadIdx.x & (kReduceOutputs - 1);
    const int s = (int)threadIdx.x / kReduceOutputs;
    const int i = (int)blockIdx.x * kReduceOutputs + o;
    float acc = 0.0f;
    if (i < count)
        for (int b = s; b < blocks; b += 8) acc += partial[(size_t)b * count + i];
    part[s][o] = acc;
    __syncthreads();
    if (s == 0 && i < count) {
        float total = part[0][o];
#pragma unroll
        for (int k = 1; k < 8; ++k) total += part[k][o];
        out[i] = total;
    }
}

int wgrad_blocks(int64_t rows) {
    int64_t b = 256;  // one block of four waves per CU: each wave keeps a SIMD's MFMA unit busy
    if (b * 64 > rows) b = rows / 64 > 0 ? rows / 64 : 1;
    return (int)b;
}

}  // namespace
}  // namespace gnnagg

using namespace gnnagg;

extern "C" int64_t gnnagg_wgrad_workspace_bytes(int64_t rows, int64_t fi, int64_t fo) {
    if (rows <= 0 || fi <= 0 || fo <= 0 || fi > 256 || fo > 256) return 0;
    return (int64_t)wgrad_blocks(rows) * fi * fo * (int64_t)sizeof(float);
}

extern "C" int gnnagg_wgrad_f32(const float *x, const float *g, float *w_grad, void *workspace, int64_t rows, int64_t fi,
                                int64_t fo, void *stream) {
    return gnnagg_wgrad_strided_f32(x, fi, g, fo, w_grad, workspace, rows, fi, fo, stream);
}

extern "C" int gnnagg_wgrad_strided_f32(const float *x, int64_t x_stride, const float *g, int64_t g_stride,
                                        float *w_grad, void *workspace, int64_t rows, int64_t fi, int64_t fo,
                                        void *stream) {
    GNNAGG_REQUIRE(rows >= 0 && fi > 0 && fo > 0, "bad size");
    GNNAGG_REQUIRE(x_stride >= fi && g_stride >= fo && x_stride < (int64_t(1) << 27) && g_stride < (int64_t(1) << 27),
                   "row strides %lld / %lld must be at least the widths %lld / %lld and below 2^27",
                   (long long)x_stride, (long long)g_stride, (long long)fi, (long long)fo);
    if (fi > 256 || fo > 256)
        return fail(GNNAGG_ERR_UNSUPPORTED, "weight-gradient kernel handles Fi, Fo <= 256 (got %lld, %lld)", (long long)fi,
                    (long long)fo);
    GNNAGG_REQUIRE(w_grad, "null w_grad");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (rows == 0) {  // empty sum: the reduce kernel over zero partials writes zeros
        const int count0 = (int)(fi * fo);
        hipLaunchKernelGGL(wgrad_reduce_kernel, dim3((unsigned)((count0 + kReduceOutputs - 1) / kReduceOutputs)), dim3(256), 0, st,
                           static_cast<const float *>(nullptr), w_grad, 0, count0);
        GNNAGG_HIP(hipGetLastError());
        return GNNAGG_OK;
    }
    GNNAGG_REQUIRE(x && g && workspace, "null x/g/workspace");
    const int blocks = wgrad_blocks(rows);
    // whole chunks per block, so that only a slice's last chunk is partial
    const int64_t rpb = ((rows + blocks - 1) / blocks + kChunk - 1) / kChunk * kChunk;
    const int aligned = (fi % 4 == 0 && fo % 4 == 0 && x_stride % 4 == 0 && g_stride % 4 == 0 &&
                         (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(g) & 15) == 0)
                            ? 1
                            : 0;
    float *partial = static_cast<float *>(workspace);
    // wave corner = 32*WM x 32*WN, block = 2 x 2 waves
    const int wm = (int)((fi + 63) / 64), wn = (int)((fo + 63) / 64);
#define GNNAGG_WGRAD(M, N)                                                                                   \
    if (wm == M && wn == N) {                                                                                \
        constexpr size_t smem = (size_t)WgradShape<M, N>::kSmemFloats * sizeof(float);                       \
        GNNAGG_HIP(allow_lds(reinterpret_cast<const void *>(&wgrad_partial_kernel<M, N>), smem));           \
        hipLaunchKernelGGL((wgrad_partial_kernel<M, N>), dim3((unsigned)blocks), dim3(256), smem, st, x, g,  \
                           partial, rows, (int)fi, (int)fo, (int)x_stride, (int)g_stride, rpb, aligned);     \
    } else
    GNNAGG_WGRAD(1, 1) GNNAGG_WGRAD(1, 2) GNNAGG_WGRAD(1, 3) GNNAGG_WGRAD(1, 4) GNNAGG_WGRAD(2, 1) GNNAGG_WGRAD(2, 2)
    GNNAGG_WGRAD(2, 3) GNNAGG_WGRAD(2, 4) GNNAGG_WGRAD(3, 1) GNNAGG_WGRAD(3, 2) GNNAGG_WGRAD(3, 3) GNNAGG_WGRAD(3, 4)
    GNNAGG_WGRAD(4, 1) GNNAGG_WGRAD(4, 2) GNNAGG_WGRAD(4, 3) GNNAGG_WGRAD(4, 4) {
        return fail(GNNAGG_ERR_UNSUPPORTED, "no weight-gradient shape for Fi=%lld Fo=%lld", (long long)fi, (long long)fo);
    }
#undef GNNAGG_WGRAD
    GNNAGG_HIP(hipGetLastError());
    const int count = (int)(fi * fo);
    hipLaunchKernelGGL(wgrad_reduce_kernel, dim3((unsigned)((count + kReduceOutputs - 1) / kReduceOutputs)), dim3(256), 0, st, partial, w_grad,
                       blocks, count);
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}
