// Dense layer product with the elementwise work behind it fused in,
//
//     Y[rows, N] = epilogue( A[rows, K] @ W[K, N] ),
//
// for rows in the millions and K, N <= 256 (fp32 MFMA, v_mfma_f32_32x32x2f32; 2*rows*K*N flop
// against the 157.3 TFLOP/s fp32 matrix peak).  The epilogue divides row r by row_div[r],
// adds the bias, applies ReLU and the dropout keep-bits while the result is still in the
// accumulators, so the layer needs no elementwise pass over its [rows, N] result.
//
// A block of four waves (2 x 2) owns 64*WM rows and all N <= 64*WN columns at a time and
// walks its share of the row tiles; two blocks share a CU, so that one block's epilogue
// overlaps the other's MFMAs.  The contraction runs in chunks of 16: 64*WM x 16 values of A
// (a 64-byte piece of each row) and 16 x N values of W are copied into LDS through registers,
// the next chunk -- of this tile or the next -- in flight behind the MFMAs of the current one.
// A is row-major with the contraction index contiguous, while the MFMA wants one contraction
// index per lane across 32 rows; each lane therefore reads four consecutive values of its row
// with one 16-byte LDS read and spends them on four MFMAs (lanes 0-31 hold k+0..3, lanes 32-63
// k+4..7 of each group of eight: the order of the contraction is permuted, the same way for
// both operands).  W is the MFMA's A operand, so the accumulators hold tiles of Y^T and a lane
// owns runs of four consecutive columns of one row of Y: 16-byte stores.
//
// The BF16 form rounds both operands to bf16 (round to nearest even, in hardware) on their way
// into LDS and multiplies with v_mfma_f32_32x32x8_bf16 (fp32 accumulation): a lane's four
// consecutive values of a row are then one 8-byte operand.  W is staged transposed for that
// ([column][k]): a thread loads a 4 x 4 block of it and writes four 8-byte column pieces.  The
// matrix work shrinks to a fraction of the time the operands take to stream in, so this form
// is HBM-bound (4 * rows * (K + N) bytes).
#include <type_traits>
#include <utility>

#include "common.h"
#include "dense_tiles.h"

namespace gnnagg {
namespace {

struct LinearArgs {
    const float *a;          // [rows, K], row stride lda
    const float *row_div;    // [rows] or nullptr
    const float *w;          // [K, N], row stride ldw
    const float *bias;       // [N] or nullptr
    const uint32_t *keep;    // [rows, ceil(N/32)] keep-bits or nullptr
    float *y;                // [rows, N], row stride ldy
    uint32_t *header;        // PACK: [rows, 2 * (N / 32)] (bitmap, non-zeros in front) pairs; y then holds each row's
                             // non-zero values at its front
    int64_t rows;
    int lda, ldw, ldy, k, n;
    float scale;             // dropout scale of the epilogue
    int relu;
};

// SPLIT form, LDS records: a row of A / a column of W is 32 bytes per plane, its 16 k in the order 0-3, 8-11 | 4-7,
// 12-15 (the 16 bytes a lane of either half-wave feeds to one MFMA sit together); rows / columns whose bit 3 is set
// hold the two halves swapped, and the columns of W are permuted inside each group of 32 (both so that the 16-byte
// reads of neighbouring lanes and the 8-byte writes of the staging threads spread over the banks).
__device__ inline int split_offset(int kq, int row) { return (16 * (kq & 1) + 8 * (kq >> 1)) ^ (16 * ((row >> 3) & 1)); }
__device__ inline int split_column(int col) { return (col & ~7) | ((col & 7) ^ ((col >> 3) & 3)); }

template <int WM, int WN>
struct LinearShape {
    static constexpr int kRows = 64 * WM;            // rows of A per block
    static constexpr int kLda = kChunk + 4;          // floats between staged rows: 16-byte reads of 8 rows hit 8 bank groups
    static constexpr int kLdb = 64 * WN + 8;         // rows four apart (the two half-waves) land on the other half of the banks
    static constexpr int kVecA = WM;                 // float4 per thread per chunk of A
    static constexpr int kVecB = WN * kChunk / 16;   // float4 per thread per chunk of W
    static constexpr int kBufFloats = kRows * kLda + kChunk * kLdb;
    static constexpr int kSmemFloats = 2 * kBufFloats + 256 * 4;
    // BF16 form: rows of A and columns of W staged as kChunk bf16 + 8 bytes of padding each
    static constexpr int kLdh = 2 * kChunk + 8;      // bytes between staged rows / columns
    static constexpr int kBufBytesH = (kRows + 64 * WN) * kLdh;
    static constexpr int kSmemBytesH = 2 * kBufBytesH;
    // SPLIT form: three bf16 planes (hi, mid, lo) of the rows of A and of the columns of W, 16 k = 32 bytes a record
    static constexpr int kPlaneA = kRows * 32;
    static constexpr int kPlaneW = 64 * WN * 32;
    static constexpr int kBufBytesS = 3 * (kPlaneA + kPlaneW);
    static constexpr int kSmemBytesS = 2 * kBufBytesS;
};

// SPLIT (BF16 == false): every fp32 operand value is cut into three bf16 pieces on its way into LDS and a product
// runs as six bf16 MFMAs (hi*hi, hi*mid, mid*hi, mid*mid, hi*lo, lo*hi; the pieces left out are below 2^-24 of
// |a||w|, the size of an fp32 rounding) accumulated in fp32 -- 192 MFMA cycles per 32 x 32 x 16 block of products
// instead of the fp32 MFMA's 512.
template <int WM, int WN, bool BF16, bool PACK, bool SPLIT = false>
__global__ __launch_bounds__(256, 2) void linear_kernel(const LinearArgs p) {
    static_assert(!(BF16 && SPLIT), "the split form stages fp32");
    static_assert(!SPLIT || kChunk == 16, "one 32x32x16 MFMA group per chunk");
    using S = LinearShape<WM, WN>;
    extern __shared__ __align__(16) float smem[];
    float *dump = smem + 2 * S::kBufFloats + 4 * (int)threadIdx.x;  // (fp32 form only)
    char *smem_h = reinterpret_cast<char *>(smem);                  // (BF16 form)
    // PACK: non-zeros of each tile row in the block's left column half, behind the staging buffers
    int *row_count = reinterpret_cast<int *>(smem_h + (BF16    ? (size_t)S::kSmemBytesH
                                                       : SPLIT ? (size_t)S::kSmemBytesS
                                                               : (size_t)S::kSmemFloats * sizeof(float)));

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int kk = lane >> 5;
    const int idx = lane & 31;
    const int m0 = wm * 32 * WM, n0 = wn * 32 * WN;
    const int64_t tiles = (p.rows + S::kRows - 1) / S::kRows;
    int64_t tile = blockIdx.x;
    if (tile >= tiles) return;

    // acc[i][j] is the 32 x 32 tile of Y^T whose columns (lanes) are rows m0 + 32 i .. of Y and whose
    // rows (registers) are columns n0 + 32 j .. of Y: a lane ends up with runs of four consecutive
    // columns of one row of Y, which it stores 16 bytes at a time.
    floatx16 acc[WM][WN];
    auto clear = [&]() {
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    };
    clear();

    // A: thread t moves the float4 number t + 256*j of a chunk, i.e. piece t%4 of row t/4 + 64*j of the
    // tile.  Rows past the end read the last row instead; their results are never stored.
    const float *ap[S::kVecA];
    int a_dst[S::kVecA];
#pragma unroll
    for (int j = 0; j < S::kVecA; ++j)
        a_dst[j] = BF16    ? ((tid >> 2) + 64 * j) * S::kLdh + 8 * (tid & 3)                          // bytes
                   : SPLIT ? ((tid >> 2) + 64 * j) * 32 + split_offset(tid & 3, tid >> 2)             // bytes
                           : ((tid >> 2) + 64 * j) * S::kLda + 4 * (tid & 3);                         // floats
    auto enter_tile = [&](int64_t t) {
#pragma unroll
        for (int j = 0; j < S::kVecA; ++j) {
            int64_t row = t * S::kRows + (tid >> 2) + 64 * j;
            if (row >= p.rows) row = p.rows - 1;
            ap[j] = p.a + (size_t)row * (size_t)p.lda + 4 * (tid & 3);
        }
    };
    floatx4 areg[S::kVecA];
    auto fetch_a = [&](int k0) {
#pragma unroll
        for (int j = 0; j < S::kVecA; ++j) areg[j] = *reinterpret_cast<const floatx4 *>(ap[j] + k0);
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int j = 0; j < S::kVecA; ++j) {
            if (BF16) {
                *reinterpret_cast<shortx4 *>(smem_h + buf * S::kBufBytesH + a_dst[j]) =
                    to_bf16x4(areg[j].x, areg[j].y, areg[j].z, areg[j].w);
            } else if (SPLIT) {
                shortx4 piece[3];
                split_bf16x3(areg[j].x, areg[j].y, areg[j].z, areg[j].w, piece);
#pragma unroll
                for (int q = 0; q < 3; ++q)
                    *reinterpret_cast<shortx4 *>(smem_h + buf * S::kBufBytesS + q * S::kPlaneA + a_dst[j]) = piece[q];
            } else
                *reinterpret_cast<floatx4 *>(smem + buf * S::kBufFloats + a_dst[j]) = areg[j];
        }
    };
    ChunkLoader<S::kVecB, S::kLdb> lw;
    if (!BF16 && !SPLIT) lw.init(tid, p.n, p.ldw);
    // BF16: thread u owns the 4 x 4 block (k-quad u / (n/4), column-quad u % (n/4)) of a chunk of W; threads
    // past the 4 * (n/4) blocks repeat earlier ones (same values to the same place)
    floatx4 wreg[4];
    int w_src = 0, w_dst = 0;
    int w_dst_split[4] = {0, 0, 0, 0};
    if (BF16) {
        const int nq = p.n / 4;
        const int u = tid % (4 * nq);
        w_src = 4 * (u / nq) * p.ldw + 4 * (u % nq);
        w_dst = S::kRows * S::kLdh + 4 * (u % nq) * S::kLdh + 8 * (u / nq);
    }
    if (SPLIT) {  // k-quads fastest: four neighbouring threads fill one column's record
        const int u = tid % p.n;
        const int kq = u & 3, cq = u >> 2;
        w_src = 4 * kq * p.ldw + 4 * cq;
#pragma unroll
        for (int c = 0; c < 4; ++c)
            w_dst_split[c] = 3 * S::kPlaneA + split_column(4 * cq + c) * 32 + split_offset(kq, 4 * cq + c);
    }
    auto fetch_w = [&](const float *wc) {
        if (BF16 || SPLIT) {
#pragma unroll
            for (int c = 0; c < 4; ++c) wreg[c] = *reinterpret_cast<const floatx4 *>(wc + w_src + c * p.ldw);
        } else {
            lw.fetch_cached(wc);
        }
    };
    auto store_w = [&](int buf) {
        if (BF16) {
            char *dst = smem_h + buf * S::kBufBytesH + w_dst;
#pragma unroll
            for (int c = 0; c < 4; ++c)  // column 4 q + c of the block: its four consecutive k
                *reinterpret_cast<shortx4 *>(dst + c * S::kLdh) = to_bf16x4(wreg[0][c], wreg[1][c], wreg[2][c], wreg[3][c]);
        } else if (SPLIT) {
            char *dst = smem_h + buf * S::kBufBytesS;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                shortx4 piece[3];
                split_bf16x3(wreg[0][c], wreg[1][c], wreg[2][c], wreg[3][c], piece);
#pragma unroll
                for (int q = 0; q < 3; ++q)
                    *reinterpret_cast<shortx4 *>(dst + q * S::kPlaneW + w_dst_split[c]) = piece[q];
            }
        } else {
            lw.store_all(smem + buf * S::kBufFloats + S::kRows * S::kLda, dump);
        }
    };

    // Columns past n of a staged row of W are never written: whatever they hold only reaches
    // accumulator entries that are never stored.
    auto multiply = [&](int buf) {
        if (BF16) {
            const char *ah = smem_h + buf * S::kBufBytesH + (m0 + idx) * S::kLdh + 8 * kk;
            const char *wh = smem_h + buf * S::kBufBytesH + S::kRows * S::kLdh + (n0 + idx) * S::kLdh + 8 * kk;
            shortx4 ha[2][WM], hb[2][WN];
            auto read = [&](int s) {
#pragma unroll
                for (int i = 0; i < WM; ++i) ha[s][i] = *reinterpret_cast<const shortx4 *>(ah + 32 * i * S::kLdh + 16 * s);
#pragma unroll
                for (int j = 0; j < WN; ++j) hb[s][j] = *reinterpret_cast<const shortx4 *>(wh + 32 * j * S::kLdh + 16 * s);
            };
            read(0);
            read(1);
#pragma unroll
            for (int s = 0; s < kChunk / 8; ++s) {
#pragma unroll
                for (int i = 0; i < WM; ++i)
#pragma unroll
                    for (int j = 0; j < WN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(hb[s][j], ha[s][i], acc[i][j], 0, 0, 0);
            }
            return;
        }
        if (SPLIT) {
            const int half = 16 * (kk ^ ((idx >> 3) & 1));
            const char *ab = smem_h + buf * S::kBufBytesS + (m0 + idx) * 32 + half;
            const char *wb = smem_h + buf * S::kBufBytesS + 3 * S::kPlaneA + (n0 + split_column(idx)) * 32 + half;
            bf16x8 a3[WM][3];
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int q = 0; q < 3; ++q)
                    a3[i][q] = *reinterpret_cast<const bf16x8 *>(ab + q * S::kPlaneA + 32 * i * 32);
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                bf16x8 b3[3];
#pragma unroll
                for (int q = 0; q < 3; ++q) b3[q] = *reinterpret_cast<const bf16x8 *>(wb + q * S::kPlaneW + 32 * j * 32);
#pragma unroll
                for (int i = 0; i < WM; ++i) {  // smallest pieces first
                    floatx16 c = acc[i][j];
                    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b3[2], a3[i][0], c, 0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b3[0], a3[i][2], c, 0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b3[1], a3[i][1], c, 0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b3[1], a3[i][0], c, 0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b3[0], a3[i][1], c, 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b3[0], a3[i][0], c, 0, 0, 0);
                }
            }
            return;
        }
        const float *as = smem + buf * S::kBufFloats + (m0 + idx) * S::kLda + 4 * kk;
        const float *bs = smem + buf * S::kBufFloats + S::kRows * S::kLda + 4 * kk * S::kLdb + n0 + idx;
        floatx4 av[2][WM];
        float bv[2][WN];
        auto read_a = [&](int h) {
#pragma unroll
            for (int i = 0; i < WM; ++i)
                av[h][i] = *reinterpret_cast<const floatx4 *>(as + 32 * i * S::kLda + 8 * h);
        };
        auto read_b = [&](int s) {
#pragma unroll
            for (int j = 0; j < WN; ++j) bv[s & 1][j] = bs[(8 * (s >> 2) + (s & 3)) * S::kLdb + 32 * j];
        };
        read_a(0);
        read_b(0);
#pragma unroll
        for (int s = 0; s < kChunk / 2; ++s) {
            if (s + 1 < kChunk / 2) read_b(s + 1);
            if (s == 2) read_a(1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int j = 0; j < WN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[s & 1][j], av[s >> 2][i][s & 3], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // 32x32 accumulator layout: register r of lane l holds D[(r % 4) + 4 * (l / 32) + 8 * (r / 4)][l % 32]
    const int words = (p.n + 31) / 32;  // keep-bit words per row
    // this lane's row divisors and keep-bit words: loaded when a tile starts, used when it ends
    float rdiv[WM];
    uint32_t kbits[WM][WN];
    auto load_divisors = [&](int64_t t) {
#pragma unroll
        for (int i = 0; i < WM; ++i) {
            const int64_t m = t * S::kRows + m0 + 32 * i + idx;
            const bool live = m < p.rows;
            rdiv[i] = (p.row_div && live) ? p.row_div[m] : 1.0f;
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                const int nt = n0 + 32 * j;
                kbits[i][j] = (p.keep && live && nt < p.n) ? p.keep[(size_t)m * (size_t)words + (nt >> 5)] : 0xffffffffu;
            }
        }
    };
    auto finish_tile_dense = [&](int64_t t) {
#pragma unroll
        for (int i = 0; i < WM; ++i) {
            const int64_t m = t * S::kRows + m0 + 32 * i + idx;
            const bool live = m < p.rows;
            const float inv = 1.0f / rdiv[i];
            float *yrow = p.y + (size_t)(live ? m : 0) * (size_t)p.ldy;
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                const int nt = n0 + 32 * j;
                const uint32_t bits = kbits[i][j] >> (4 * kk);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int n = nt + 8 * g + 4 * kk;
                    if (!live || n >= p.n) continue;
                    floatx4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                    // (acc * inv + bias as one fused multiply-add per value, here and in the packed form)
                    const floatx4 b4 = p.bias ? *reinterpret_cast<const floatx4 *>(p.bias + n) : floatx4{0.f, 0.f, 0.f, 0.f};
                    v.x = __builtin_fmaf(v.x, inv, b4.x);
                    v.y = __builtin_fmaf(v.y, inv, b4.y);
                    v.z = __builtin_fmaf(v.z, inv, b4.z);
                    v.w = __builtin_fmaf(v.w, inv, b4.w);
                    if (p.relu) {
                        v.x = fmaxf(v.x, 0.0f);
                        v.y = fmaxf(v.y, 0.0f);
                        v.z = fmaxf(v.z, 0.0f);
                        v.w = fmaxf(v.w, 0.0f);
                    }
                    v *= p.scale;
                    const uint32_t b = bits >> (8 * g);
                    v.x = (b & 1u) ? v.x : 0.0f;
                    v.y = (b & 2u) ? v.y : 0.0f;
                    v.z = (b & 4u) ? v.z : 0.0f;
                    v.w = (b & 8u) ? v.w : 0.0f;
                    *reinterpret_cast<floatx4 *>(yrow + n) = v;
                }
            }
        }
    };

    // PACK: the same values, but every row keeps only its non-zeros, moved to its front in column order, and a
    // header says where they belong: per 32 columns the bitmap of the non-zeros and the number of non-zeros in
    // front of them.  Four lanes share a row (two per wave: columns 8g + 4kk + c of each 32-column tile; the block's
    // two column halves in two waves), so ranks come from the tile bitmaps (exchanged between the two lanes), a
    // running count over the wave's tiles, and the left half's total handed to the right half through LDS.
    auto finish_tile_packed = [&](int64_t t) {
        uint32_t word[WM][WN];
#pragma unroll
        for (int i = 0; i < WM; ++i) {
            const int64_t m = t * S::kRows + m0 + 32 * i + idx;
            const bool live = m < p.rows;
            const float inv = 1.0f / rdiv[i];
            int total = 0;
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                const int nt = n0 + 32 * j;
                const uint32_t bits = kbits[i][j] >> (4 * kk);
                uint32_t mine = 0;
                floatx4 b4[4];
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    b4[g] = (p.bias && nt < p.n) ? *reinterpret_cast<const floatx4 *>(p.bias + nt + 8 * g + 4 * kk)
                                                 : floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int local = 8 * (r >> 2) + (r & 3);  // + 4 kk: this value's column inside the tile
                    float v = __builtin_fmaf(acc[i][j][r], inv, b4[r >> 2][r & 3]);
                    v = fmaxf(v, 0.0f) * p.scale;
                    if (!((bits >> local) & 1u) || !live || nt >= p.n) v = 0.0f;
                    acc[i][j][r] = v;
                    mine |= (v > 0.0f ? 1u : 0u) << local;
                }
                mine <<= 4 * kk;
                word[i][j] = mine | (uint32_t)__shfl_xor((int)mine, 32);
                total += __popc(word[i][j]);
            }
            if (wn == 0 && kk == 0) row_count[m0 + 32 * i + idx] = total;
        }
        __syncthreads();
        const int hw = 2 * (p.n / 32);
#pragma unroll
        for (int i = 0; i < WM; ++i) {
            const int64_t m = t * S::kRows + m0 + 32 * i + idx;
            if (m >= p.rows) continue;
            int front = wn == 1 ? row_count[m0 + 32 * i + idx] : 0;
            float *yrow = p.y + (size_t)m * (size_t)p.ldy;
            uint32_t *hrow = p.header + (size_t)m * (size_t)hw;
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                const int nt = n0 + 32 * j;
                if (nt >= p.n) continue;
                const uint32_t w = word[i][j];
                if (kk == 0) {
                    hrow[2 * (nt >> 5)] = w;
                    hrow[2 * (nt >> 5) + 1] = (uint32_t)front;
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int local = 8 * (r >> 2) + (r & 3) + 4 * kk;
                    if ((w >> local) & 1u) yrow[front + __popc(w & ((1u << local) - 1u))] = acc[i][j][r];
                }
                front += __popc(w);
            }
        }
    };
    auto finish_tile = [&](int64_t t) {
        if (PACK)
            finish_tile_packed(t);
        else
            finish_tile_dense(t);
    };

    // One stream of chunks over all tiles of this block: the first chunk of the next tile is in
    // flight behind the last MFMAs of the current one, and a tile's stores drain behind the next
    // tile's MFMAs.
    const int chunks = p.k / kChunk;
    const size_t wstep = (size_t)kChunk * (size_t)p.ldw;
    enter_tile(tile);
    load_divisors(tile);
    fetch_a(0);
    fetch_w(p.w);
    store_a(0);
    store_w(0);
    __syncthreads();
    int buf = 0;
    for (;;) {
        const float *wc = p.w;
        for (int c = 1; c < chunks; ++c) {
            wc += wstep;
            fetch_w(wc);
            fetch_a(c * kChunk);
            __builtin_amdgcn_sched_barrier(0);  // keep the loads ahead of the MFMAs
            multiply(buf);
            store_a(buf ^ 1);
            store_w(buf ^ 1);
            __syncthreads();
            buf ^= 1;
        }
        const int64_t done = tile;
        tile += gridDim.x;
        const bool more = tile < tiles;
        if (more) {
            enter_tile(tile);
            fetch_w(p.w);
            fetch_a(0);
        }
        __builtin_amdgcn_sched_barrier(0);
        multiply(buf);
        if (more) {
            store_a(buf ^ 1);
            store_w(buf ^ 1);
        }
        __builtin_amdgcn_sched_barrier(0);
        finish_tile(done);
        __builtin_amdgcn_sched_barrier(0);
        if (!more) break;
        load_divisors(tile);
        clear();
        __syncthreads();
        buf ^= 1;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// The bf16-input form with the waves of a block split by role, and W resident in LDS.
//
// In the kernel above every wave does everything, one phase after the other: it issues the global loads of the next
// chunk, multiplies the current one, converts what the loads brought and writes it to LDS.  With bf16 operands the
// matrix work is a fraction of the time the operands take to stream in, so what counts is how many bytes of A a compute
// unit keeps in flight.  Here one block of twelve waves owns a compute unit:
//   * all of W, rounded to bf16 and transposed ([chunk of 16 k][column][16 k]: 32 bytes a column, the two 16-byte halves
//     swapped for columns whose bit 3 is set so that sixteen neighbouring lanes read 64 distinct banks), is written to
//     LDS once when the block starts (K x 256 x 2 bytes: 128 KB at K = 256) and stays there -- per-chunk loads of W would
//     queue behind the deep stream of A in the compute unit's in-order vector-memory path (measured: 0.3-0.6 ms of 3.4);
//   * waves 0-7 multiply: 4 x 2 over a tile of 128 rows x 256 columns, 32 rows x 128 columns each.  They read their rows
//     of A as fp32 from LDS (16 floats per row and chunk), round them to bf16 in registers (v_cvt_pk_bf16_f32) and feed
//     v_mfma_f32_32x32x16_bf16; the two waves of a SIMD (w and w + 4) work half an iteration apart, one multiplying while
//     the other reads and converts;
//   * waves 8-11 stream A: a 64-byte piece of each of the tile's 128 rows per chunk, kStreamDepth chunks (64 KB) in
//     flight in their registers, written to a ring of three 8 KB LDS slots two chunks ahead of the multiplying waves.
// One barrier per chunk hands slots over.  The epilogue is the same arithmetic as above on the same accumulator layout.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kStreamRows = 128;
constexpr int kStreamDepth = 8;                    // chunks of A in flight in the loading waves' registers
constexpr int kStreamSlots = 3;                    // raw A slots in LDS: chunks q, q + 1 being read, q + 2 being written
constexpr int kStreamASlot = kStreamRows * 64;     // 8 KB: 128 rows x 16 fp32
constexpr int kStreamWChunk = 256 * 32;            // 8 KB: 256 columns x 16 bf16
constexpr int kStreamBias = 256 * 4;               // the bias (zeros when there is none), staged once per block
constexpr int kStreamMaxK = 256;                   // W resident: K * 512 bytes of LDS
inline size_t stream_smem_bytes(int k, bool pack) {
    return (size_t)(k / kChunk) * kStreamWChunk + kStreamSlots * kStreamASlot + kStreamBias + (pack ? kStreamRows * sizeof(int) : 0);
}

// f(integral_constant<int, 0>{}), ..., f(integral_constant<int, N - 1>{}): a loop whose index is a constant expression
template <int... Is, typename F>
__device__ __forceinline__ void static_for_each(std::integer_sequence<int, Is...>, F &&f) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_each(std::make_integer_sequence<int, N>{}, f);
}

template <bool PACK>
__global__ __launch_bounds__(768, 1) void linear_stream_bf16_kernel(const LinearArgs p) {
    extern __shared__ __align__(16) char lds[];
    const int nk = p.k / kChunk;
    char *wres = lds;                                   // nk chunks of W
    char *aring = lds + nk * kStreamWChunk;             // kStreamSlots chunks of A, fp32
    float *bias_lds = reinterpret_cast<float *>(aring + kStreamSlots * kStreamASlot);
    int *row_count = reinterpret_cast<int *>(bias_lds + 256);  // PACK: non-zeros of each tile row in columns 0-127
    const int tid = (int)threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t tiles = (p.rows + kStreamRows - 1) / kStreamRows;
    if ((int64_t)blockIdx.x >= tiles) return;
    const int my_tiles = (int)((tiles - blockIdx.x + gridDim.x - 1) / gridDim.x);
    const int total = my_tiles * nk;  // chunks this block walks through, tile after tile
    // the loading waves' loop is unrolled kStreamDepth times: everybody meets at `padded` + 1 barriers
    const int padded = (total + kStreamDepth - 1) / kStreamDepth * kStreamDepth;
    if (tid < 256) bias_lds[tid] = (p.bias && tid < p.n) ? p.bias[tid] : 0.0f;
    // W: unit u = (chunk, half of the chunk's k, group of four columns); eight 16-byte loads, four 16-byte LDS writes
    for (int u = tid; u < nk * 128; u += 768) {
        const int cg = u & 63, khalf = (u >> 6) & 1, c = u >> 7;
        // columns past n: any valid address; what they hold only reaches results that are never stored
        const float *src = p.w + (size_t)(kChunk * c + 8 * khalf) * (size_t)p.ldw + (4 * cg < p.n ? 4 * cg : 0);
        floatx4 wreg[8];
#pragma unroll
        for (int kr = 0; kr < 8; ++kr) wreg[kr] = *reinterpret_cast<const floatx4 *>(src + (size_t)kr * (size_t)p.ldw);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = 4 * cg + j;
            union {
                bf16x2 h[4];
                floatx4 v;
            } cv;
#pragma unroll
            for (int h = 0; h < 4; ++h) cv.h[h] = __builtin_convertvector(floatx2{wreg[2 * h][j], wreg[2 * h + 1][j]}, bf16x2);
            *reinterpret_cast<floatx4 *>(wres + c * kStreamWChunk + col * 32 + 16 * (khalf ^ ((col >> 3) & 1))) = cv.v;
        }
    }
    // (visible to the multiplying waves behind the first barrier below)

    if (wave < 8) {
        const int wr = wave >> 1, wc = wave & 1;
        const int m0 = 32 * wr, n0 = 128 * wc;
        const int kk = lane >> 5, idx = lane & 31;
        // raw A slot: 16-byte unit (row, piece) sits at row * 4 + (piece ^ ((row >> 2) & 3)): sixteen neighbouring lanes
        // (rows) reading the same piece hit 64 distinct banks
        int a_off[2];
        {
            const int row = m0 + idx, sw = (row >> 2) & 3;
            a_off[0] = (row * 4 + ((2 * kk) ^ sw)) * 16;
            a_off[1] = (row * 4 + ((2 * kk + 1) ^ sw)) * 16;
        }
        const int b_off = (n0 + idx) * 32 + 16 * (kk ^ ((idx >> 3) & 1));
        floatx16 acc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;
        bf16x8 a_op, b_op[4];
        auto read_convert = [&](int sa, int c) __attribute__((always_inline)) {
            const char *pa = aring + sa * kStreamASlot;
            const char *pw = wres + c * kStreamWChunk + b_off;
            const floatx4 r0 = *reinterpret_cast<const floatx4 *>(pa + a_off[0]);
            const floatx4 r1 = *reinterpret_cast<const floatx4 *>(pa + a_off[1]);
#pragma unroll
            for (int j = 0; j < 4; ++j) b_op[j] = *reinterpret_cast<const bf16x8 *>(pw + j * 1024);
            union {
                bf16x2 h[4];
                bf16x8 v;
            } u;
            u.h[0] = __builtin_convertvector(floatx2{r0.x, r0.y}, bf16x2);
            u.h[1] = __builtin_convertvector(floatx2{r0.z, r0.w}, bf16x2);
            u.h[2] = __builtin_convertvector(floatx2{r1.x, r1.y}, bf16x2);
            u.h[3] = __builtin_convertvector(floatx2{r1.z, r1.w}, bf16x2);
            a_op = u.v;
        };
        auto multiply = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b_op[j], a_op, acc[j], 0, 0, 0);
        };

        // 32x32 accumulator layout: register r of lane l holds D[(r % 4) + 4 * (l / 32) + 8 * (r / 4)][l % 32], D = a tile
        // of Y^T: this lane owns runs of four consecutive columns of row m0 + idx
        const int words = (p.n + 31) / 32;
        float rdiv = 1.0f;
        uint32_t kbits[4];
        auto load_divisors = [&](int s) __attribute__((always_inline)) {
            const int64_t m = ((int64_t)blockIdx.x + (int64_t)s * gridDim.x) * kStreamRows + m0 + idx;
            const bool live = m < p.rows;
            rdiv = (p.row_div && live) ? p.row_div[m] : 1.0f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int nt = n0 + 32 * j;
                kbits[j] = (p.keep && live && nt < p.n) ? p.keep[(size_t)m * (size_t)words + (nt >> 5)] : 0xffffffffu;
            }
        };
        auto finish_tile = [&](int s) __attribute__((always_inline)) {
            const int64_t m = ((int64_t)blockIdx.x + (int64_t)s * gridDim.x) * kStreamRows + m0 + idx;
            const bool live = m < p.rows;
            const float inv = 1.0f / rdiv;
            if (!PACK) {
                // branch-free but for the store itself: ReLU and keep-bits as selects
                float *yrow = p.y + (size_t)(live ? m : 0) * (size_t)p.ldy;
                const bool relu = p.relu != 0;
                auto act = [&](float a, float bias) __attribute__((always_inline)) {
                    const float z = __builtin_fmaf(a, inv, bias);  // (acc * inv + bias as one fused multiply-add, as above)
                    return (relu ? fmaxf(z, 0.0f) : z) * p.scale;
                };
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int nt = n0 + 32 * j;
                    const uint32_t bits = kbits[j] >> (4 * kk);
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int n = nt + 8 * g + 4 * kk;
                        const floatx4 b4 = *reinterpret_cast<const floatx4 *>(bias_lds + (n & 255));
                        const uint32_t b = bits >> (8 * g);
                        floatx4 v;
                        v.x = act(acc[j][4 * g], b4.x);
                        v.y = act(acc[j][4 * g + 1], b4.y);
                        v.z = act(acc[j][4 * g + 2], b4.z);
                        v.w = act(acc[j][4 * g + 3], b4.w);
                        v.x = (b & 1u) ? v.x : 0.0f;
                        v.y = (b & 2u) ? v.y : 0.0f;
                        v.z = (b & 4u) ? v.z : 0.0f;
                        v.w = (b & 8u) ? v.w : 0.0f;
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[j][4 * g + r] = 0.0f;
                        if (live && n < p.n) *reinterpret_cast<floatx4 *>(yrow + n) = v;
                    }
                }
                return;
            }
            // PACK: every row keeps only its non-zeros, moved to its front in column order, and a header says where
            // they belong (per 32 columns the bitmap of the non-zeros and the number of non-zeros in front of them).
            // Four lanes share a row: two per wave (columns 8g + 4kk + c of each 32-column tile) and the block's two
            // column halves in two waves; the left half's total reaches the right half through LDS.
            uint32_t word[4];
            int count = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int nt = n0 + 32 * j;
                const uint32_t bits = kbits[j] >> (4 * kk);
                uint32_t mine = 0;
                floatx4 b4[4];
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    b4[g] = *reinterpret_cast<const floatx4 *>(bias_lds + nt + 8 * g + 4 * kk);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int local = 8 * (r >> 2) + (r & 3);  // + 4 kk: this value's column inside the tile
                    float v = __builtin_fmaf(acc[j][r], inv, b4[r >> 2][r & 3]);
                    v = fmaxf(v, 0.0f) * p.scale;
                    if (!((bits >> local) & 1u) || !live || nt >= p.n) v = 0.0f;
                    acc[j][r] = v;
                    mine |= (v > 0.0f ? 1u : 0u) << local;
                }
                mine <<= 4 * kk;
                word[j] = mine | (uint32_t)__shfl_xor((int)mine, 32);
                count += __popc(word[j]);
            }
            if (wc == 0 && kk == 0) row_count[m0 + idx] = count;
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the count is in LDS
            __builtin_amdgcn_s_barrier();        // (every wave of the block, the loading ones included, meets here)
            int front = wc == 1 ? row_count[m0 + idx] : 0;
            if (live) {
                const int hw = 2 * (p.n / 32);
                float *yrow = p.y + (size_t)m * (size_t)p.ldy;
                uint32_t *hrow = p.header + (size_t)m * (size_t)hw;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int nt = n0 + 32 * j;
                    if (nt >= p.n) continue;
                    const uint32_t w = word[j];
                    if (kk == 0) {
                        hrow[2 * (nt >> 5)] = w;
                        hrow[2 * (nt >> 5) + 1] = (uint32_t)front;
                    }
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int local = 8 * (r >> 2) + (r & 3) + 4 * kk;
                        if ((w >> local) & 1u) yrow[front + __popc(w & ((1u << local) - 1u))] = acc[j][r];
                    }
                    front += __popc(w);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;
        };

        // `early` waves multiply chunk q first and then prepare chunk q + 1; the others prepare chunk q, then multiply it
        const bool early = wave < 4;
        __builtin_amdgcn_s_waitcnt(0xc07f);  // this wave's share of W and of the bias is in LDS
        __builtin_amdgcn_s_barrier();
        int q = 0, sa = 0;  // sa = q % kStreamSlots
        if (early) {
            read_convert(0, 0);
            for (int s = 0; s < my_tiles; ++s) {
                load_divisors(s);
                for (int c = 0; c < nk; ++c, ++q) {
                    multiply();
                    if (c + 1 == nk) finish_tile(s);
                    sa = sa + 1 == kStreamSlots ? 0 : sa + 1;
                    if (q + 1 < total) read_convert(sa, c + 1 == nk ? 0 : c + 1);
                    __builtin_amdgcn_s_barrier();
                }
            }
        } else {
            for (int s = 0; s < my_tiles; ++s) {
                load_divisors(s);
                for (int c = 0; c < nk; ++c, ++q) {
                    read_convert(sa, c);
                    sa = sa + 1 == kStreamSlots ? 0 : sa + 1;
                    multiply();
                    if (c + 1 == nk) finish_tile(s);
                    __builtin_amdgcn_s_barrier();
                }
            }
        }
        for (; q < padded; ++q) __builtin_amdgcn_s_barrier();
    } else {
        // ---- four waves stream A through their registers: two 16-byte pieces of every chunk per thread ----
        const int pt = tid - 512;
        int a_row[2], a_piece[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int u = e * 256 + pt;  // 16-byte unit of the chunk, also its place in the slot: row u / 4
            a_row[e] = u >> 2;
            a_piece[e] = (u & 3) ^ ((a_row[e] >> 2) & 3);
        }
        const int a_dst = pt * 16;
        int a_tile = 0, a_c = 0, a_q = 0;  // the next chunk to request
        const float *a_ptr[2];
        auto enter_tile = [&]() __attribute__((always_inline)) {
            const int64_t first = ((int64_t)blockIdx.x + (int64_t)a_tile * gridDim.x) * kStreamRows;
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                int64_t r = first + a_row[e];
                if (r >= p.rows) r = p.rows - 1;  // rows past the end read the last row; their results are never stored
                a_ptr[e] = p.a + (size_t)r * (size_t)p.lda + 4 * a_piece[e];
            }
        };
        enter_tile();
        floatx4 areg[kStreamDepth][2];
        auto fetch = [&](auto set) __attribute__((always_inline)) {
            constexpr int S = decltype(set)::value;
#pragma unroll
            for (int e = 0; e < 2; ++e) areg[S][e] = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(a_ptr[e] + kChunk * a_c));
            ++a_q;
            if (a_q < total) {  // past the end: the same chunk again, never used
                if (++a_c == nk) {
                    a_c = 0;
                    ++a_tile;
                    enter_tile();
                }
            }
        };
        auto store = [&](auto set, int slot) __attribute__((always_inline)) {
            constexpr int S = decltype(set)::value;
            char *dst = aring + slot * kStreamASlot + a_dst;
#pragma unroll
            for (int e = 0; e < 2; ++e) *reinterpret_cast<floatx4 *>(dst + e * 4096) = areg[S][e];
        };
        // chunks 0 .. kStreamDepth-1 into registers; chunks 0 and 1 into LDS and their sets refilled
        static_for<kStreamDepth>([&](auto set) __attribute__((always_inline)) { fetch(set); });
        store(std::integral_constant<int, 0>{}, 0);
        fetch(std::integral_constant<int, 0>{});
        store(std::integral_constant<int, 1>{}, 1);
        fetch(std::integral_constant<int, 1>{});
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS writes (A, W, bias) have landed
        __builtin_amdgcn_s_barrier();
        // iteration q: chunk q + 2 (set (q + 2) % kStreamDepth) goes to slot (q + 2) % kStreamSlots; the set takes chunk
        // q + 2 + kStreamDepth
        int slot = 2, c = 0;
        for (int q = 0; q < padded; q += kStreamDepth) {
            static_for<kStreamDepth>([&](auto ph) __attribute__((always_inline)) {
                constexpr int S = (decltype(ph)::value + 2) % kStreamDepth;
                store(std::integral_constant<int, S>{}, slot);
                fetch(std::integral_constant<int, S>{});
                slot = slot + 1 == kStreamSlots ? 0 : slot + 1;
                if (PACK && q + decltype(ph)::value < total && ++c == nk) {
                    c = 0;
                    __builtin_amdgcn_s_barrier();  // the multiplying waves' exchange of row counts
                }
                __builtin_amdgcn_s_waitcnt(0xc07f);
                __builtin_amdgcn_s_barrier();
            });
        }
    }
}

template <bool PACK>
int launch_linear_stream(const LinearArgs &p, hipStream_t st) {
    const size_t smem = stream_smem_bytes(p.k, PACK);
    GNNAGG_HIP(allow_lds(reinterpret_cast<const void *>(&linear_stream_bf16_kernel<PACK>), smem));
    int dev = 0, cus = 0;
    GNNAGG_HIP(hipGetDevice(&dev));
    GNNAGG_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int64_t tiles = (p.rows + kStreamRows - 1) / kStreamRows;
    const int64_t resident = (int64_t)(cus > 0 ? cus : 256);  // one block of twelve waves per compute unit
    const unsigned blocks = (unsigned)(tiles < resident ? tiles : resident);
    hipLaunchKernelGGL((linear_stream_bf16_kernel<PACK>), dim3(blocks), dim3(768), smem, st, p);
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

template <int WM, int WN, bool BF16, bool PACK, bool SPLIT>
int launch_linear(const LinearArgs &p, hipStream_t st) {
    using S = LinearShape<WM, WN>;
    constexpr size_t smem = (BF16    ? (size_t)S::kSmemBytesH
                             : SPLIT ? (size_t)S::kSmemBytesS
                                     : (size_t)S::kSmemFloats * sizeof(float)) +
                            (PACK ? S::kRows * sizeof(int) : 0);
    GNNAGG_HIP(allow_lds(reinterpret_cast<const void *>(&linear_kernel<WM, WN, BF16, PACK, SPLIT>), smem));
    int dev = 0, cus = 0;
    GNNAGG_HIP(hipGetDevice(&dev));
    GNNAGG_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int64_t tiles = (p.rows + S::kRows - 1) / S::kRows;
    const int64_t resident = 2 * (int64_t)(cus > 0 ? cus : 256);  // two blocks per CU, each walks its share of the tiles
    const unsigned blocks = (unsigned)(tiles < resident ? tiles : resident);
    hipLaunchKernelGGL((linear_kernel<WM, WN, BF16, PACK, SPLIT>), dim3(blocks), dim3(256), smem, st, p);
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

template <bool BF16, bool SPLIT>
int dispatch_linear(const LinearArgs &p, hipStream_t st) {
    if constexpr (BF16) {
        // the kernel with W resident in LDS: K * 512 bytes of it, and an int chunk counter
        const int64_t tiles = (p.rows + kStreamRows - 1) / kStreamRows;
        if (p.k <= kStreamMaxK && tiles * (p.k / kChunk) < (int64_t(1) << 30))
            return p.header ? launch_linear_stream<true>(p, st) : launch_linear_stream<false>(p, st);
    }
    if (p.header) {  // packed output: widths 32, 64, 128, 256
        switch ((p.n + 63) / 64) {
            case 1: return launch_linear<2, 1, BF16, true, SPLIT>(p, st);
            case 2: return launch_linear<2, 2, BF16, true, SPLIT>(p, st);
            default: return launch_linear<2, 4, BF16, true, SPLIT>(p, st);
        }
    }
    switch ((p.n + 63) / 64) {
        case 1: return launch_linear<2, 1, BF16, false, SPLIT>(p, st);
        case 2: return launch_linear<2, 2, BF16, false, SPLIT>(p, st);
        case 3: return launch_linear<2, 3, BF16, false, SPLIT>(p, st);
        default: return launch_linear<2, 4, BF16, false, SPLIT>(p, st);
    }
}

bool aligned16(const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; }

int check_linear(const LinearArgs &p) {
    if (p.rows < 0 || p.k <= 0 || p.n <= 0) return fail(GNNAGG_ERR_INVALID, "negative or empty sizes");
    if (p.k % kChunk != 0 || p.n % 4 != 0 || p.n > 256 || p.k > (1 << 20))
        return fail(GNNAGG_ERR_UNSUPPORTED, "fused layer product takes K %% 16 == 0, N %% 4 == 0, N <= 256 (got K=%d N=%d)",
                    p.k, p.n);
    if (p.lda < p.k || p.ldw < p.n || p.ldy < p.n)
        return fail(GNNAGG_ERR_INVALID, "row strides must be at least the widths");
    if (p.lda % 4 || p.ldw % 4 || p.ldy % 4 || !aligned16(p.a) || !aligned16(p.w) || !aligned16(p.y) ||
        !aligned16(p.bias))
        return fail(GNNAGG_ERR_UNSUPPORTED, "fused layer product takes 16-byte aligned operands and row strides");
    if (p.rows > 0 && (!p.a || !p.w || !p.y)) return fail(GNNAGG_ERR_INVALID, "null operand");
    return GNNAGG_OK;
}

// one thread per word: 32 consecutive mask bytes of a row
__global__ __launch_bounds__(256) void pack_keep_bits_kernel(const uint8_t *__restrict__ keep, uint32_t *__restrict__ bits,
                                                             int feat, int words, int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int64_t row = i / words;
    const int f0 = (int)(i - row * words) * 32;
    const uint8_t *src = keep + (size_t)row * feat + f0;
    uint32_t w = 0;
#pragma unroll 8
    for (int q = 0; q < 32; ++q)
        if (f0 + q < feat && src[q]) w |= 1u << q;
    bits[i] = w;
}

// the same for rows of whole words on a 16-byte boundary: the word's 32 bytes arrive as two 16-byte loads
__global__ __launch_bounds__(256) void pack_keep_bits_aligned_kernel(const uint4 *__restrict__ keep,
                                                                     uint32_t *__restrict__ bits, int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const uint4 lo = keep[2 * i], hi = keep[2 * i + 1];
    const uint32_t part[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    uint32_t w = 0;
#pragma unroll
    for (int p = 0; p < 8; ++p)
#pragma unroll
        for (int b = 0; b < 4; ++b)
            if ((part[p] >> (8 * b)) & 0xffu) w |= 1u << (4 * p + b);
    bits[i] = w;
}

}  // namespace
}  // namespace gnnagg

using namespace gnnagg;

extern "C" int gnnagg_linear_shape_supported(int64_t k, int64_t n) {
    return (k > 0 && n > 0 && k % kChunk == 0 && n % 4 == 0 && n <= 256 && k <= (1 << 20)) ? 1 : 0;
}

extern "C" int gnnagg_pack_keep_bits(const void *keep, uint32_t *bits, int64_t rows, int64_t feat, void *stream) {
    GNNAGG_REQUIRE(rows >= 0 && feat > 0 && feat < (1 << 30), "bad sizes");
    if (rows == 0) return GNNAGG_OK;
    GNNAGG_REQUIRE(keep && bits, "null keep/bits");
    const int words = (int)((feat + 31) / 32);
    const int64_t total = rows * words;
    if (feat % 32 == 0 && reinterpret_cast<uintptr_t>(keep) % 16 == 0)
        hipLaunchKernelGGL(pack_keep_bits_aligned_kernel, dim3(grid_for(total, 256)), dim3(256), 0,
                           static_cast<hipStream_t>(stream), static_cast<const uint4 *>(keep), bits, total);
    else
        hipLaunchKernelGGL(pack_keep_bits_kernel, dim3(grid_for(total, 256)), dim3(256), 0,
                           static_cast<hipStream_t>(stream), static_cast<const uint8_t *>(keep), bits, (int)feat, words,
                           total);
    GNNAGG_HIP(hipGetLastError());
    return GNNAGG_OK;
}

namespace {
// form: 0 fp32 MFMA, 1 operands rounded to bf16, 2 every fp32 operand as three bf16 pieces (six bf16 MFMAs per product)
int run_linear(int form, const float *x, int64_t x_stride, const float *w, int64_t w_stride, const float *bias,
               const uint32_t *keep_bits, const float *row_div, float scale, int relu, float *y, int64_t y_stride,
               uint32_t *header, int64_t rows, int64_t k, int64_t n, void *stream) {
    GNNAGG_REQUIRE(x_stride < (1 << 27) && w_stride < (1 << 27) && y_stride < (1 << 27) && k < (1 << 27) && n < (1 << 27),
                   "sizes and row strides must be below 2^27");
    LinearArgs p{x, row_div, w, bias, keep_bits, y, header, rows, (int)x_stride, (int)w_stride, (int)y_stride, (int)k,
                 (int)n, scale, relu};
    if (int rc = check_linear(p)) return rc;
    if (header && !(n == 32 || n == 64 || n == 128 || n == 256))
        return fail(GNNAGG_ERR_UNSUPPORTED, "packed activations exist for widths 32, 64, 128, 256 (got %lld)", (long long)n);
    if (header && (!relu || y_stride != n))
        return fail(GNNAGG_ERR_INVALID, "packed output follows a ReLU and has row stride n");
    if (rows == 0) return GNNAGG_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (form) {
        case 0: return dispatch_linear<false, false>(p, st);
        case 1: return dispatch_linear<true, false>(p, st);
        case 2: return dispatch_linear<false, true>(p, st);
        default: return fail(GNNAGG_ERR_INVALID, "product form is 0 (fp32), 1 (bf16 inputs) or 2 (bf16 x 3 pieces), got %d", form);
    }
}
}  // namespace

extern "C" int gnnagg_linear_bias_relu_dropout_f32(const float *x, int64_t x_stride, const float *w, int64_t w_stride,
                                                   const float *bias, const uint32_t *keep_bits, const float *row_div,
                                                   float scale, int relu, float *y, int64_t y_stride, int64_t rows,
                                                   int64_t k, int64_t n, void *stream) {
    return run_linear(0, x, x_stride, w, w_stride, bias, keep_bits, row_div, scale, relu, y, y_stride, nullptr, rows,
                      k, n, stream);
}

extern "C" int gnnagg_linear_bias_relu_dropout_bf16x3_f32(const float *x, int64_t x_stride, const float *w,
                                                          int64_t w_stride, const float *bias, const uint32_t *keep_bits,
                                                          const float *row_div, float scale, int relu, float *y,
                                                          int64_t y_stride, int64_t rows, int64_t k, int64_t n,
                                                          void *stream) {
    return run_linear(2, x, x_stride, w, w_stride, bias, keep_bits, row_div, scale, relu, y, y_stride, nullptr, rows,
                      k, n, stream);
}

extern "C" int gnnagg_linear_bias_relu_dropout_bf16_f32(const float *x, int64_t x_stride, const float *w,
                                                        int64_t w_stride, const float *bias, const uint32_t *keep_bits,
                                                        const float *row_div, float scale, int relu, float *y,
                                                        int64_t y_stride, int64_t rows, int64_t k, int64_t n,
                                                        void *stream) {
    return run_linear(1, x, x_stride, w, w_stride, bias, keep_bits, row_div, scale, relu, y, y_stride, nullptr, rows,
                      k, n, stream);
}

extern "C" int gnnagg_linear_bias_relu_dropout_pack_f32(const float *x, int64_t x_stride, const float *w, int64_t w_stride,
                                                        const float *bias, const uint32_t *keep_bits,
                                                        const float *row_div, float scale, float *y_packed,
                                                        uint32_t *header, int64_t rows, int64_t k, int64_t n,
                                                        int bf16_inputs, void *stream) {
    GNNAGG_REQUIRE(header || rows == 0, "null header");
    return run_linear(bf16_inputs, x, x_stride, w, w_stride, bias, keep_bits, row_div, scale, 1, y_packed, n, header,
                      rows, k, n, stream);
}
