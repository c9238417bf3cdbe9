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
#include <mutex>

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

// What the MASKED form of the kernel does to G on its way into LDS: g is the gradient with respect
// to a layer's output y = relu(z) * keep * scale, z = (x @ w) / row_div + bias.  The kernel turns it
// into pre = (y > 0 ? g * scale : 0) (the gradient with respect to z; y is 0 exactly where the unit
// was inactive or dropped), adds pre up per column (the bias gradient), divides by row_div, uses
// the result as the G operand and also writes it out for the input-gradient product.
struct MaskArgs {
    const float *act;       // y [rows, fo], row stride ldact; with all_on: any readable row of fo floats, ldact = 0
    const float *row_div;   // [rows] or nullptr
    float *gz;              // out: [rows, fo] contiguous, or nullptr (not wanted)
    float *bias_partial;    // out: [blocks][kVecG * 256] float4, the per-thread column sums
    int ldact;
    float scale;
    int all_on;             // no ReLU / dropout behind the product: every entry counts
    // alternative to act: one bit per unit (set = the unit was active); the word of columns 32 v .. 32 v + 31 of row
    // r is bits[r * bits_stride + v * bits_step] (the header of packed activations: stride 2 * (fo / 32), step 2)
    const uint32_t *bits;
    int bits_stride, bits_step;
};

// MODE 0: plain product.  MODE 1: the masked form above.  MODE 2: only the column sums of g * scale ride along (no
// mask, no division, nothing written out): the bias gradient of a layer without ReLU / dropout behind its product.
// MODE 3: MODE 1 with the activity read from a bitmap (4 bytes per 32 units) instead of the activations themselves.
template <int WM, int WN, int MODE>
__global__ __launch_bounds__(256, 1) void wgrad_partial_kernel(const float *__restrict__ x,
                                                               const float *__restrict__ g,
                                                               float *__restrict__ partial, int64_t rows, int fi,
                                                               int fo, int ldx, int ldg, int64_t rows_per_block,
                                                               int aligned, const MaskArgs mk) {
    constexpr bool MASKED = MODE != 0;   // something rides along with G
    constexpr bool FULL = MODE == 1 || MODE == 3;  // ... the whole mask pass
    constexpr bool BITS = MODE == 3;               // ... with the activity from a bitmap
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

    // MASKED: the activations come in with the same loader shape as G; thread t's vector j always sits in
    // the same columns (the chunk is 16 whole rows), so its column sums stay in registers.
    ChunkLoader<MASKED ? S::kVecG : 1, S::kLdg> lc;
    floatx4 colsum[S::kVecG];
    float dreg[S::kVecG];
    int grow[S::kVecG];  // row of vector j inside a chunk
    int bit_word[S::kVecG], bit_shift[S::kVecG];  // BITS: where the vector's four activity bits sit in its row's words
    uint32_t breg[S::kVecG];
    if (MASKED) {
        if (FULL && !BITS) lc.init(tid, fo, mk.ldact);
#pragma unroll
        for (int j = 0; j < S::kVecG; ++j) {
            colsum[j] = floatx4{0.f, 0.f, 0.f, 0.f};
            grow[j] = lg.elem[j] / fo;
            const int col = lg.elem[j] % fo;
            bit_word[j] = (col >> 5) * mk.bits_step;
            bit_shift[j] = col & 31;
        }
    }
    // any readable float per row when there is no divisor (the value is not used then)
    const float *divp = FULL ? (mk.row_div ? mk.row_div : x) : nullptr;
    const int divstep = (FULL && mk.row_div) ? 1 : 0;
    auto fetch_divisors = [&](int64_t r, int64_t last) {  // rows r .. r+15, clamped to `last`
#pragma unroll
        for (int j = 0; j < S::kVecG; ++j) {
            int64_t row = r + grow[j];
            if (row > last) row = last;
            dreg[j] = divp[row * divstep];
            if (BITS) breg[j] = mk.bits[(size_t)row * (size_t)mk.bits_stride + bit_word[j]];
        }
    };
    // The same for the whole chunks of the steady state: no clamp, and 32-bit offsets from the slice's first row that
    // advance by one chunk per call (no 64-bit index arithmetic ahead of the MFMAs).
    const float *div_base = FULL ? divp + (size_t)r_begin * (size_t)divstep : nullptr;
    const uint32_t *bits_base = BITS ? mk.bits + (size_t)r_begin * (size_t)mk.bits_stride : nullptr;
    int div_off[S::kVecG], bits_off[S::kVecG];
#pragma unroll
    for (int j = 0; j < S::kVecG; ++j) {
        div_off[j] = MASKED ? grow[j] * divstep : 0;
        bits_off[j] = BITS ? grow[j] * mk.bits_stride + bit_word[j] : 0;
    }
    auto fetch_divisors_next = [&]() {
#pragma unroll
        for (int j = 0; j < S::kVecG; ++j) {
            dreg[j] = div_base[div_off[j]];
            div_off[j] += kChunk * divstep;
            if (BITS) {
                breg[j] = bits_base[bits_off[j]];
                bits_off[j] += kChunk * mk.bits_stride;
            }
        }
    };
    // turns vector j of lg.reg (g) into the G operand, with lc.reg = y; `valid` = number of values of the chunk that exist
    auto mask_piece = [&](int64_t r, int valid, int j) __attribute__((always_inline)) {
        const bool used = lg.lds_off[j] >= 0 && lg.elem[j] < valid;
        const floatx4 gv = lg.reg[j];
        floatx4 pre;
        if (!FULL) {  // column sums only: G itself stays the operand
            pre = used ? gv * mk.scale : floatx4{0.f, 0.f, 0.f, 0.f};
            colsum[j] += pre;
            return;
        }
        if (BITS) {
            const uint32_t nib = breg[j] >> bit_shift[j];
            pre.x = (used && (nib & 1u)) ? gv.x * mk.scale : 0.0f;
            pre.y = (used && (nib & 2u)) ? gv.y * mk.scale : 0.0f;
            pre.z = (used && (nib & 4u)) ? gv.z * mk.scale : 0.0f;
            pre.w = (used && (nib & 8u)) ? gv.w * mk.scale : 0.0f;
        } else {
            const floatx4 yv = lc.reg[j];
            const bool all = mk.all_on != 0;
            pre.x = (used && (all || yv.x > 0.0f)) ? gv.x * mk.scale : 0.0f;
            pre.y = (used && (all || yv.y > 0.0f)) ? gv.y * mk.scale : 0.0f;
            pre.z = (used && (all || yv.z > 0.0f)) ? gv.z * mk.scale : 0.0f;
            pre.w = (used && (all || yv.w > 0.0f)) ? gv.w * mk.scale : 0.0f;
        }
        colsum[j] += pre;
        const float inv = mk.row_div ? 1.0f / dreg[j] : 1.0f;
        pre *= inv;
        lg.reg[j] = pre;
        if (used && mk.gz)
            __builtin_nontemporal_store(pre, reinterpret_cast<floatx4 *>(mk.gz + (size_t)r * (size_t)fo + lg.elem[j]));
    };
    auto mask_g = [&](int64_t r, int valid) {
#pragma unroll
        for (int j = 0; j < S::kVecG; ++j) mask_piece(r, valid, j);
    };

    // Columns past fi / fo of an LDS row are never written: whatever they hold only reaches
    // accumulator entries that are never stored.
    // `between(s)` runs behind the MFMAs of k-pair s: work that does not depend on them executes in their shadow
    auto multiply_and = [&](int buf, auto between) __attribute__((always_inline)) {
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
            between(s);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto multiply = [&](int buf) { multiply_and(buf, [](int) {}); };

    // steady state: whole chunks, no masks; the next chunk's global loads are in flight behind
    // this chunk's MFMAs and land in the other LDS buffer
    if (full > 0) {
        const float *xc = x + (size_t)r_begin * (size_t)ldx;
        const float *gc = g + (size_t)r_begin * (size_t)ldg;
        const size_t xstep = (size_t)kChunk * (size_t)ldx, gstep = (size_t)kChunk * (size_t)ldg;
        const float *cc = MASKED ? mk.act + (size_t)r_begin * (size_t)mk.ldact : nullptr;
        const size_t cstep = MASKED ? (size_t)kChunk * (size_t)mk.ldact : 0;
        lx.fetch(xc);
        lg.fetch(gc);
        if (MASKED) {
            if (FULL) {
                if (!BITS) lc.fetch(cc);
                fetch_divisors_next();
            }
            mask_g(r_begin, kChunk * fo);
        }
        lx.store_all(xs, dump);
        lg.store_all(gs, dump);
        __syncthreads();
        for (int64_t c = 1; c < full; ++c) {
            xc += xstep;
            gc += gstep;
            lx.fetch(xc);
            lg.fetch(gc);
            if (MASKED) {
                cc += cstep;
                if (FULL) {
                    if (!BITS) lc.fetch(cc);
                    fetch_divisors_next();
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the loads ahead of the MFMAs
            if (MASKED) {
                // the chunk's MFMAs cover the flight of the loads; the mask work on what they brought runs in
                // the shadow of the last k-pair's MFMAs
                const int64_t r = r_begin + c * kChunk;
                multiply_and((int)((c - 1) & 1), [&](int s) __attribute__((always_inline)) {
                    if (s == kChunk / 2 - 1) mask_g(r, kChunk * fo);
                });
            } else {
                multiply((int)((c - 1) & 1));
            }
            __builtin_amdgcn_sched_barrier(0);
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
        if (MASKED) {  // the host only launches this form with 16-byte copies possible
            if (FULL) {
                if (!BITS) lc.fetch_tail(mk.act + (size_t)r * (size_t)mk.ldact, left * fo, true);
                fetch_divisors(r, r_end - 1);
            }
            mask_g(r, left * fo);
        }
        lx.store(xs, aligned != 0);
        lg.store(gs, aligned != 0);
        __syncthreads();
        multiply(0);
        __syncthreads();
    }

    if (MASKED) {
        floatx4 *bp = reinterpret_cast<floatx4 *>(mk.bias_partial) + (size_t)blockIdx.x * (S::kVecG * 256);
#pragma unroll
        for (int j = 0; j < S::kVecG; ++j) bp[j * 256 + tid] = colsum[j];
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

// bias[n] = sum over the blocks and over the 16 rows of a chunk of the per-thread column sums: the
// values of column n sit in the vectors number (4 * (n / 4) + r * fo) / 4, r < 16, of a chunk.  A block
// of 256 threads owns 16 columns; thread (r, c) adds up row r of column c over the blocks, and the
// 16 row sums of a column are then added in order of r.
__global__ __launch_bounds__(256) void wgrad_bias_reduce_kernel(const float *__restrict__ partial, float *__restrict__ bias,
                                                                int blocks, int vec_per_block, int fo) {
    __shared__ float part[kChunk][16];
    const int c = (int)threadIdx.x & 15, r = (int)threadIdx.x >> 4;
    const int n = (int)blockIdx.x * 16 + c;
    float s = 0.0f;
    if (n < fo) {
        const int v = (4 * (n / 4) + r * fo) / 4;
        for (int b = 0; b < blocks; ++b) s += partial[((size_t)b * vec_per_block + v) * 4 + (n & 3)];
    }
    part[r][c] = s;
    __syncthreads();
    if (r == 0 && n < fo) {
        float total = part[0][c];
#pragma unroll
        for (int k = 1; k < kChunk; ++k) total += part[k][c];
        bias[n] = total;
    }
}

// ---- bf16-input form ---------------------------------------------------------------------------
// The same product with both operands rounded to bf16 (round to nearest even) on their way into
// LDS and v_mfma_f32_32x32x8_bf16 (fp32 accumulation).  The matrix work is then a fraction of the
// time the operands take to stream in: this form is HBM-bound.  The MFMA wants, per lane, four
// consecutive ROWS of one column (the contraction runs over rows), so a chunk is staged
// transposed: a thread loads a 4 x 4 block (four rows, four columns: one float4 per row) and
// writes four 8-byte column pieces, [column][16 rows as bf16 + 8 bytes of padding].  Rows past
// the slice read the slice's last row and count as zeros, so there is no separate tail path.
constexpr int kLdh = 2 * kChunk + 8;  // bytes between staged columns

// SPLIT: fp32 accuracy on the same units -- every operand value is cut into three bf16 pieces (hi, mid, lo: three
// planes of the staging layout) and a product is the sum of six v_mfma_f32_32x32x16_bf16 (hi*hi, hi*mid, mid*hi,
// mid*mid, hi*lo, lo*hi; what is left out is below 2^-24 |x||g| per term).
template <int WM, int WN, bool MASKED, bool BITS, bool SPLIT = false>
__global__ __launch_bounds__(256, 1) void wgrad_bf16_partial_kernel(const float *__restrict__ x,
                                                                    const float *__restrict__ g,
                                                                    float *__restrict__ partial, int64_t rows, int fi,
                                                                    int fo, int ldx, int ldg, int64_t rows_per_block,
                                                                    const MaskArgs mk) {
    extern __shared__ __align__(16) float smem[];
    char *lds = reinterpret_cast<char *>(smem);
    constexpr int kPlaneBytes = (64 * WM + 64 * WN) * kLdh;
    constexpr int kBufBytes = (SPLIT ? 3 : 1) * kPlaneBytes;
    constexpr int kGOff = 64 * WM * kLdh;

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int kk = lane >> 5;
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
    const int64_t chunks = r_begin < r_end ? (r_end - r_begin + kChunk - 1) / kChunk : 0;

    // thread u owns the block (row-quad u / (width/4), column-quad u % (width/4)) of each operand's chunk;
    // threads past the 4 * (width/4) blocks repeat earlier ones (same values to the same place)
    const int xq = fi / 4, gq = fo / 4;
    const int ux = tid % (4 * xq), ug = tid % (4 * gq);
    const int x_rq = ux / xq, x_cq = ux % xq, g_rq = ug / gq, g_cq = ug % gq;
    const bool g_first = tid < 4 * gq;  // the one thread that accounts for its block of G
    const int x_dst = 4 * x_cq * kLdh + 8 * x_rq;
    const int g_dst = kGOff + 4 * g_cq * kLdh + 8 * g_rq;

    floatx4 xr[4], gr[4], yr[4];
    float dr[4];
    uint32_t br[4];  // BITS: the word that holds the activity bits of the block's four columns, per row
    const int b_word = ((4 * g_cq) >> 5) * mk.bits_step, b_shift = (4 * g_cq) & 31;
    floatx4 colsum = {0.f, 0.f, 0.f, 0.f};
    const float *divp = MASKED ? (mk.row_div ? mk.row_div : x) : nullptr;  // any readable float per row without a divisor
    const int64_t divstep = MASKED ? (mk.row_div ? 1 : ldx) : 0;
    auto fetch = [&](int64_t r0) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            int64_t rx = r0 + 4 * x_rq + c, rg = r0 + 4 * g_rq + c;
            if (rx >= r_end) rx = r_end - 1;
            if (rg >= r_end) rg = r_end - 1;
            xr[c] = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(x + (size_t)rx * (size_t)ldx + 4 * x_cq));
            gr[c] = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(g + (size_t)rg * (size_t)ldg + 4 * g_cq));
            if (MASKED) {
                if (BITS)
                    br[c] = mk.bits[(size_t)rg * (size_t)mk.bits_stride + b_word];
                else
                    yr[c] = __builtin_nontemporal_load(
                        reinterpret_cast<const floatx4 *>(mk.act + (size_t)rg * (size_t)mk.ldact + 4 * g_cq));
                dr[c] = divp[rg * divstep];
            }
        }
    };
    auto stage = [&](int64_t r0, int buf) {
        char *dst = lds + buf * kBufBytes;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const bool live_x = r0 + 4 * x_rq + c < r_end, live_g = r0 + 4 * g_rq + c < r_end;
            if (!live_x) xr[c] = floatx4{0.f, 0.f, 0.f, 0.f};
            if (MASKED) {
                const bool all = mk.all_on != 0;
                bool on[4];
                if (BITS) {
                    const uint32_t nib = br[c] >> b_shift;
                    on[0] = nib & 1u, on[1] = nib & 2u, on[2] = nib & 4u, on[3] = nib & 8u;
                } else {
                    on[0] = all || yr[c].x > 0.0f, on[1] = all || yr[c].y > 0.0f;
                    on[2] = all || yr[c].z > 0.0f, on[3] = all || yr[c].w > 0.0f;
                }
                floatx4 pre;
                pre.x = (live_g && on[0]) ? gr[c].x * mk.scale : 0.0f;
                pre.y = (live_g && on[1]) ? gr[c].y * mk.scale : 0.0f;
                pre.z = (live_g && on[2]) ? gr[c].z * mk.scale : 0.0f;
                pre.w = (live_g && on[3]) ? gr[c].w * mk.scale : 0.0f;
                if (g_first) colsum += pre;
                const float inv = mk.row_div ? 1.0f / dr[c] : 1.0f;
                pre *= inv;
                gr[c] = pre;
                if (live_g && g_first && mk.gz)
                    __builtin_nontemporal_store(
                        pre, reinterpret_cast<floatx4 *>(mk.gz + (size_t)(r0 + 4 * g_rq + c) * (size_t)fo + 4 * g_cq));
            } else if (!live_g) {
                gr[c] = floatx4{0.f, 0.f, 0.f, 0.f};
            }
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {  // column 4 q + c of the block: its four consecutive rows
            if (SPLIT) {
                shortx4 px[3], pg[3];
                split_bf16x3(xr[0][c], xr[1][c], xr[2][c], xr[3][c], px);
                split_bf16x3(gr[0][c], gr[1][c], gr[2][c], gr[3][c], pg);
#pragma unroll
                for (int q = 0; q < 3; ++q) {
                    *reinterpret_cast<shortx4 *>(dst + q * kPlaneBytes + x_dst + c * kLdh) = px[q];
                    *reinterpret_cast<shortx4 *>(dst + q * kPlaneBytes + g_dst + c * kLdh) = pg[q];
                }
            } else {
                *reinterpret_cast<shortx4 *>(dst + x_dst + c * kLdh) = to_bf16x4(xr[0][c], xr[1][c], xr[2][c], xr[3][c]);
                *reinterpret_cast<shortx4 *>(dst + g_dst + c * kLdh) = to_bf16x4(gr[0][c], gr[1][c], gr[2][c], gr[3][c]);
            }
        }
    };
    // Columns past fi / fo are never written: whatever they hold only reaches accumulator entries
    // that are never stored.
    auto multiply = [&](int buf) {
        const char *xa = lds + buf * kBufBytes + (m0 + idx) * kLdh + 8 * kk;
        const char *gb = lds + buf * kBufBytes + kGOff + (n0 + idx) * kLdh + 8 * kk;
        if (SPLIT) {
            // a lane feeds rows 4 kk .. 4 kk + 3 and 8 + 4 kk .. of its column to one 32x32x16 MFMA (both operands
            // in the same order, so the sum over the chunk's 16 rows is the same)
            auto piece8 = [](const char *at) {
                union {
                    shortx4 h[2];
                    bf16x8 v;
                } u;
                u.h[0] = *reinterpret_cast<const shortx4 *>(at);
                u.h[1] = *reinterpret_cast<const shortx4 *>(at + 16);
                return u.v;
            };
            bf16x8 a3[WM][3];
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int q = 0; q < 3; ++q) a3[i][q] = piece8(xa + q * kPlaneBytes + 32 * i * kLdh);
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                bf16x8 b3[3];
#pragma unroll
                for (int q = 0; q < 3; ++q) b3[q] = piece8(gb + q * kPlaneBytes + 32 * j * kLdh);
#pragma unroll
                for (int i = 0; i < WM; ++i) {  // smallest pieces first
                    floatx16 c = acc[i][j];
                    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3[i][2], b3[0], c, 0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3[i][0], b3[2], c, 0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3[i][1], b3[1], c, 0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3[i][1], b3[0], c, 0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3[i][0], b3[1], c, 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3[i][0], b3[0], c, 0, 0, 0);
                }
            }
            return;
        }
        shortx4 a[2][WM], b[2][WN];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
#pragma unroll
            for (int i = 0; i < WM; ++i) a[s][i] = *reinterpret_cast<const shortx4 *>(xa + 32 * i * kLdh + 16 * s);
#pragma unroll
            for (int j = 0; j < WN; ++j) b[s][j] = *reinterpret_cast<const shortx4 *>(gb + 32 * j * kLdh + 16 * s);
        }
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int j = 0; j < WN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a[s][i], b[s][j], acc[i][j], 0, 0, 0);
    };

    if (chunks > 0) {
        fetch(r_begin);
        stage(r_begin, 0);
        __syncthreads();
        for (int64_t c = 1; c < chunks; ++c) {
            const int64_t r0 = r_begin + c * kChunk;
            fetch(r0);
            __builtin_amdgcn_sched_barrier(0);  // keep the loads ahead of the MFMAs
            multiply((int)((c - 1) & 1));
            __builtin_amdgcn_sched_barrier(0);
            stage(r0, (int)(c & 1));
            __syncthreads();
        }
        multiply((int)((chunks - 1) & 1));
    }

    if (MASKED) reinterpret_cast<floatx4 *>(mk.bias_partial)[(size_t)blockIdx.x * 256 + tid] = g_first ? colsum : floatx4{0.f, 0.f, 0.f, 0.f};
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

// bias[n] for the bf16 form: thread u = rq * (fo/4) + cq of a block holds the sums of columns 4 cq .. 4 cq + 3 over
// the rows 4 rq .. 4 rq + 3 of every chunk.  One thread per column, blocks then row-quads in order.
__global__ __launch_bounds__(256) void wgrad_bias_reduce_quads_kernel(const float *__restrict__ partial,
                                                                      float *__restrict__ bias, int blocks, int fo) {
    const int n = (int)blockIdx.x * 256 + (int)threadIdx.x;
    if (n >= fo) return;
    const int gq = fo / 4;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    for (int b = 0; b < blocks; ++b)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) s[rq] += partial[((size_t)b * 256 + rq * gq + n / 4) * 4 + (n & 3)];
    bias[n] = (s[0] + s[1]) + (s[2] + s[3]);
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

extern "C" int gnnagg_wgrad_f32(const float *x, const float *g, float *w_grad, void *workspace, int64_t workspace_bytes,
                                int64_t rows, int64_t fi, int64_t fo, void *stream) {
    return gnnagg_wgrad_strided_f32(x, fi, g, fo, w_grad, workspace, workspace_bytes, rows, fi, fo, stream);
}

namespace {

int run_wgrad(const float *x, int64_t x_stride, const float *g, int64_t g_stride, float *w_grad, void *workspace,
              int64_t workspace_bytes, int64_t rows, int64_t fi, int64_t fo, void *stream, const MaskArgs *mask,
              float *bias_grad, int form = 0) {  // 0 fp32 MFMA, 1 operands rounded to bf16, 2 three bf16 pieces per operand (both masked only)
    GNNAGG_REQUIRE(form >= 0 && form <= 2, "product form is 0 (fp32), 1 (bf16 inputs) or 2 (bf16 x 3 pieces), got %d", form);
    GNNAGG_REQUIRE(form == 0 || mask, "the bf16 forms of the weight gradient come with the masked pass");
    const bool bf16 = form != 0;
    GNNAGG_REQUIRE(rows >= 0 && fi > 0 && fo > 0, "bad size");
    GNNAGG_REQUIRE(x_stride >= fi && g_stride >= fo && x_stride < (int64_t(1) << 27) && g_stride < (int64_t(1) << 27),
                   "row strides %lld / %lld must be at least the widths %lld / %lld and below 2^27",
                   (long long)x_stride, (long long)g_stride, (long long)fi, (long long)fo);
    if (fi > 256 || fo > 256)
        return fail(GNNAGG_ERR_UNSUPPORTED, "weight-gradient kernel handles Fi, Fo <= 256 (got %lld, %lld)", (long long)fi,
                    (long long)fo);
    GNNAGG_REQUIRE(w_grad, "null w_grad");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (rows == 0) {  // empty sums: the reduce kernels over zero partials write zeros
        const int count0 = (int)(fi * fo);
        hipLaunchKernelGGL(wgrad_reduce_kernel, dim3((unsigned)((count0 + kReduceOutputs - 1) / kReduceOutputs)), dim3(256),
                           0, st, static_cast<const float *>(nullptr), w_grad, 0, count0);
        if (mask)
            hipLaunchKernelGGL(wgrad_bias_reduce_kernel, dim3(grid_for(fo, 16)), dim3(256), 0, st,
                               static_cast<const float *>(nullptr), bias_grad, 0, 0, (int)fo);
        GNNAGG_HIP(hipGetLastError());
        return GNNAGG_OK;
    }
    GNNAGG_REQUIRE(x && g && workspace, "null x/g/workspace");
    const int blocks = wgrad_blocks(rows);
    {   // the kernels write one partial result per slice (and, masked, per-thread bias sums) into the workspace
        const int64_t need = mask ? gnnagg_wgrad_relu_dropout_backward_workspace_bytes(rows, fi, fo)
                                  : gnnagg_wgrad_workspace_bytes(rows, fi, fo);
        if (need <= 0)
            return fail(GNNAGG_ERR_UNSUPPORTED, "no weight-gradient kernel for rows=%lld Fi=%lld Fo=%lld%s", (long long)rows,
                        (long long)fi, (long long)fo, mask ? " with the masked pass (widths must be multiples of 4)" : "");
        GNNAGG_REQUIRE(workspace_bytes >= need,
                       "workspace of %lld bytes given, %lld needed for rows=%lld Fi=%lld Fo=%lld",
                       (long long)workspace_bytes, (long long)need, (long long)rows, (long long)fi, (long long)fo);
    }
    // whole chunks per block, so that only a slice's last chunk is partial
    const int64_t rpb = ((rows + blocks - 1) / blocks + kChunk - 1) / kChunk * kChunk;
    const int aligned = (fi % 4 == 0 && fo % 4 == 0 && x_stride % 4 == 0 && g_stride % 4 == 0 &&
                         (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(g) & 15) == 0)
                            ? 1
                            : 0;
    float *partial = static_cast<float *>(workspace);
    MaskArgs mk{};
    if (mask) {
        mk = *mask;
        if (!aligned || (!mk.bits && (mk.ldact % 4 != 0 || (reinterpret_cast<uintptr_t>(mk.act) & 15) != 0)) ||
            (reinterpret_cast<uintptr_t>(mk.gz) & 15) != 0)
            return fail(GNNAGG_ERR_UNSUPPORTED, "the masked weight gradient takes widths and row strides that are "
                                                "multiples of 4 floats and 16-byte aligned operands");
        mk.bias_partial = partial + (size_t)blocks * (size_t)fi * (size_t)fo;  // behind the partial weight gradients
    }
    // wave corner = 32*WM x 32*WN, block = 2 x 2 waves
    const int wm = (int)((fi + 63) / 64), wn = (int)((fo + 63) / 64);
    const bool sums_only = mask && mk.all_on && !mk.row_div && !mk.gz && !mk.bits;
#define GNNAGG_WGRAD_FORM(M, N, MASKED)                                                                         \
    {                                                                                                           \
        constexpr size_t smem = (size_t)WgradShape<M, N>::kSmemFloats * sizeof(float);                          \
        GNNAGG_HIP(allow_lds(reinterpret_cast<const void *>(&wgrad_partial_kernel<M, N, MASKED>), smem));       \
        hipLaunchKernelGGL((wgrad_partial_kernel<M, N, MASKED>), dim3((unsigned)blocks), dim3(256), smem, st, x, g, \
                           partial, rows, (int)fi, (int)fo, (int)x_stride, (int)g_stride, rpb, aligned, mk);    \
    }
#define GNNAGG_WGRAD_SPLIT(M, N, BITS)                                                                          \
    {                                                                                                           \
        constexpr size_t smem = (size_t)6 * (64 * M + 64 * N) * kLdh;                                            \
        GNNAGG_HIP(allow_lds(reinterpret_cast<const void *>(&wgrad_bf16_partial_kernel<M, N, true, BITS, true>), smem)); \
        hipLaunchKernelGGL((wgrad_bf16_partial_kernel<M, N, true, BITS, true>), dim3((unsigned)blocks), dim3(256), smem, st, \
                           x, g, partial, rows, (int)fi, (int)fo, (int)x_stride, (int)g_stride, rpb, mk);       \
    }
#define GNNAGG_WGRAD_BF16(M, N)                                                                                  \
    {                                                                                                           \
        constexpr size_t smem = (size_t)2 * (64 * M + 64 * N) * kLdh;                                            \
        if (form == 2 && mk.bits)                                                                               \
            GNNAGG_WGRAD_SPLIT(M, N, true)                                                                      \
        else if (form == 2)                                                                                     \
            GNNAGG_WGRAD_SPLIT(M, N, false)                                                                     \
        else if (mk.bits)                                                                                       \
            hipLaunchKernelGGL((wgrad_bf16_partial_kernel<M, N, true, true>), dim3((unsigned)blocks), dim3(256), smem, st, \
                               x, g, partial, rows, (int)fi, (int)fo, (int)x_stride, (int)g_stride, rpb, mk);   \
        else                                                                                                    \
            hipLaunchKernelGGL((wgrad_bf16_partial_kernel<M, N, true, false>), dim3((unsigned)blocks), dim3(256), smem, st, \
                               x, g, partial, rows, (int)fi, (int)fo, (int)x_stride, (int)g_stride, rpb, mk);   \
    }
#define GNNAGG_WGRAD(M, N)                          \
    if (wm == M && wn == N) {                       \
        if (bf16) GNNAGG_WGRAD_BF16(M, N)           \
        else if (mask && sums_only) GNNAGG_WGRAD_FORM(M, N, 2) \
        else if (mask && mk.bits) GNNAGG_WGRAD_FORM(M, N, 3) \
        else if (mask) GNNAGG_WGRAD_FORM(M, N, 1)   \
        else GNNAGG_WGRAD_FORM(M, N, 0)             \
    } else
    GNNAGG_WGRAD(1, 1) GNNAGG_WGRAD(1, 2) GNNAGG_WGRAD(1, 3) GNNAGG_WGRAD(1, 4) GNNAGG_WGRAD(2, 1) GNNAGG_WGRAD(2, 2)
    GNNAGG_WGRAD(2, 3) GNNAGG_WGRAD(2, 4) GNNAGG_WGRAD(3, 1) GNNAGG_WGRAD(3, 2) GNNAGG_WGRAD(3, 3) GNNAGG_WGRAD(3, 4)
    GNNAGG_WGRAD(4, 1) GNNAGG_WGRAD(4, 2) GNNAGG_WGRAD(4, 3) GNNAGG_WGRAD(4, 4) {
        return fail(GNNAGG_ERR_UNSUPPORTED, "no weight-gradient shape for Fi=%lld Fo=%lld", (long long)fi, (long long)fo);
    }
#undef GNNAGG_WGRAD
#undef GNNAGG_WGRAD_FORM
#undef GNNAGG_WGRAD_BF16
#undef GNNAGG_WGRAD_SPLIT
    GNNAGG_HIP(hipGetLastError());
    const int count = (int)(fi * fo);
    hipLaunchKernelGGL(wgrad_reduce_kernel, dim3((unsigned)((count + kReduceOutputs - 1) / kReduceOutputs)), dim3(256), 0,
                       st, partial, w_grad, blocks, count);
    if (mask && bf16)
        hipLaunchKernelGGL(wgrad_bias_reduce_quads_kernel, dim3(grid_for(fo, 256)), dim3(256), 0, st, mk.bias_partial,
                           bias_grad, blocks, (int)fo);
    else if (mask)
        hipLaunchKernelGGL(wgrad_bias_reduce_kernel, dim3(grid_for(fo, 16)), dim3(256), 0, st, mk.bias_partial, bias_grad,
                           blocks, wn * 256, (int)fo);
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

}  // namespace

extern "C" int gnnagg_wgrad_strided_f32(const float *x, int64_t x_stride, const float *g, int64_t g_stride,
                                        float *w_grad, void *workspace, int64_t workspace_bytes, int64_t rows,
                                        int64_t fi, int64_t fo, void *stream) {
    return run_wgrad(x, x_stride, g, g_stride, w_grad, workspace, workspace_bytes, rows, fi, fo, stream, nullptr, nullptr);
}

// ---- the entry point that allocates nothing -------------------------------------------------------------------
// The per-slice partial results of gnnagg_wgrad_f32 normally live in a workspace the caller allocates.  Callers that
// cannot allocate (code under HIP graph capture, serving loops) get the same kernels with the partial results in a
// file-scope device array instead.  256 slices x 256 x 256 outputs x 4 bytes = 64 MiB per GPU the library runs on,
// held until the process ends: every shape the kernels take (Fi, Fo <= 256) fits.
constexpr size_t kScratchFloats = (size_t)256 * 256 * 256;
static __device__ __align__(256) float scratch[kScratchFloats];

namespace {

// `scratch` above is a host-side stand-in for the symbol, not a device address; every GPU holds its own copy of
// the array at its own address, looked up once per device with that device current.
constexpr int kMaxDevices = 64;
float *scratch_ptr[kMaxDevices];
std::mutex scratch_mutex;

int scratch_of_current_device(float **out) {
    int dev = -1;
    GNNAGG_HIP(hipGetDevice(&dev));
    GNNAGG_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal %d outside 0..%d", dev, kMaxDevices - 1);
    std::lock_guard<std::mutex> hold(scratch_mutex);
    if (!scratch_ptr[dev]) {
        void *p = nullptr;
        GNNAGG_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        GNNAGG_REQUIRE(p, "no device address for the built-in scratch array on device %d", dev);
        scratch_ptr[dev] = static_cast<float *>(p);
    }
    *out = scratch_ptr[dev];
    return GNNAGG_OK;
}

}  // namespace

extern "C" int gnnagg_wgrad_noalloc_f32(const float *x, const float *g, float *w_grad, int64_t rows, int64_t fi,
                                        int64_t fo, void *stream) {
    GNNAGG_REQUIRE(rows >= 0 && fi > 0 && fo > 0, "bad size");
    const int64_t need = rows == 0 ? 0 : (int64_t)wgrad_blocks(rows) * fi * fo * (int64_t)sizeof(float);
    if (fi > 256 || fo > 256 || need > (int64_t)(kScratchFloats * sizeof(float)))
        return fail(GNNAGG_ERR_UNSUPPORTED,
                    "Fi=%lld Fo=%lld needs more than the %lld bytes of the built-in scratch array (Fi, Fo <= 256); "
                    "use gnnagg_wgrad_f32 with a workspace",
                    (long long)fi, (long long)fo, (long long)(kScratchFloats * sizeof(float)));
    float *partial = nullptr;
    const int rc = scratch_of_current_device(&partial);
    if (rc != GNNAGG_OK) return rc;
    // every slice writes all Fi x Fo of its partial results before the reduction reads them: nothing in the array
    // has to start at zero, whatever the previous call left there
    return run_wgrad(x, fi, g, fo, w_grad, partial, (int64_t)(kScratchFloats * sizeof(float)), rows, fi, fo, stream,
                     nullptr, nullptr);
}

extern "C" int64_t gnnagg_wgrad_relu_dropout_backward_workspace_bytes(int64_t rows, int64_t fi, int64_t fo) {
    if (rows <= 0 || fi <= 0 || fo <= 0 || fi > 256 || fo > 256 || fi % 4 != 0 || fo % 4 != 0) return 0;
    const int64_t wn = (fo + 63) / 64;
    return (int64_t)wgrad_blocks(rows) * (fi * fo + wn * 1024) * (int64_t)sizeof(float);
}

extern "C" int gnnagg_wgrad_relu_dropout_backward_f32(const float *x, int64_t x_stride, const float *grad_y,
                                                      int64_t grad_stride, const float *y, int64_t y_stride,
                                                      const float *row_div, float scale, float *grad_z, float *w_grad,
                                                      float *bias_grad, void *workspace, int64_t workspace_bytes, int64_t rows, int64_t fi,
                                                      int64_t fo, void *stream) {
    GNNAGG_REQUIRE(bias_grad, "null bias_grad");
    GNNAGG_REQUIRE(!y || (y_stride >= fo && y_stride < (int64_t(1) << 27)), "bad row stride of y");
    // without y the kernel reads the first row of g over and over in its place (row stride 0: a cache hit) and
    // ignores the values
    MaskArgs mk{y ? y : grad_y, row_div, grad_z, nullptr, (int)(y ? y_stride : 0), scale, y ? 0 : 1, nullptr, 0, 0};
    return run_wgrad(x, x_stride, grad_y, grad_stride, w_grad, workspace, workspace_bytes, rows, fi, fo, stream, &mk, bias_grad);
}

extern "C" int gnnagg_wgrad_relu_dropout_backward_bf16_f32(const float *x, int64_t x_stride, const float *grad_y,
                                                           int64_t grad_stride, const float *y, int64_t y_stride,
                                                           const float *row_div, float scale, float *grad_z,
                                                           float *w_grad, float *bias_grad, void *workspace, int64_t workspace_bytes, int64_t rows,
                                                           int64_t fi, int64_t fo, void *stream) {
    GNNAGG_REQUIRE(bias_grad, "null bias_grad");
    GNNAGG_REQUIRE(!y || (y_stride >= fo && y_stride < (int64_t(1) << 27)), "bad row stride of y");
    MaskArgs mk{y ? y : grad_y, row_div, grad_z, nullptr, (int)(y ? y_stride : 0), scale, y ? 0 : 1, nullptr, 0, 0};
    return run_wgrad(x, x_stride, grad_y, grad_stride, w_grad, workspace, workspace_bytes, rows, fi, fo, stream, &mk, bias_grad, 1);
}

extern "C" int gnnagg_wgrad_relu_dropout_backward_bf16x3_f32(const float *x, int64_t x_stride, const float *grad_y,
                                                             int64_t grad_stride, const float *y, int64_t y_stride,
                                                             const float *row_div, float scale, float *grad_z,
                                                             float *w_grad, float *bias_grad, void *workspace, int64_t workspace_bytes,
                                                             int64_t rows, int64_t fi, int64_t fo, void *stream) {
    GNNAGG_REQUIRE(bias_grad, "null bias_grad");
    GNNAGG_REQUIRE(!y || (y_stride >= fo && y_stride < (int64_t(1) << 27)), "bad row stride of y");
    MaskArgs mk{y ? y : grad_y, row_div, grad_z, nullptr, (int)(y ? y_stride : 0), scale, y ? 0 : 1, nullptr, 0, 0};
    return run_wgrad(x, x_stride, grad_y, grad_stride, w_grad, workspace, workspace_bytes, rows, fi, fo, stream, &mk, bias_grad, 2);
}

extern "C" int gnnagg_wgrad_relu_dropout_backward_from_header_f32(const float *x, int64_t x_stride, const float *grad_y,
                                                                  int64_t grad_stride, const uint32_t *header,
                                                                  const float *row_div, float scale, float *grad_z,
                                                                  float *w_grad, float *bias_grad, void *workspace, int64_t workspace_bytes,
                                                                  int64_t rows, int64_t fi, int64_t fo, int bf16_inputs,
                                                                  void *stream) {
    GNNAGG_REQUIRE(bias_grad, "null bias_grad");
    GNNAGG_REQUIRE(header || rows == 0, "null header");
    if (!(fo == 32 || fo == 64 || fo == 128 || fo == 256))
        return fail(GNNAGG_ERR_UNSUPPORTED, "packed activations exist for widths 32, 64, 128, 256 (got %lld)", (long long)fo);
    MaskArgs mk{nullptr, row_div, grad_z, nullptr, 0, scale, 0, header, (int)(2 * (fo / 32)), 2};
    return run_wgrad(x, x_stride, grad_y, grad_stride, w_grad, workspace, workspace_bytes, rows, fi, fo, stream, &mk, bias_grad,
                     bf16_inputs);
}
