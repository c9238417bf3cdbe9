/*
 * TEST INFRASTRUCTURE -- CPU oracle, not part of the product.
 *
 * Plain-C restatement of the reference's native aggregation operator.  Only
 * tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may load
 * this library; the product (gnn_benchmark_amd/) never does.
 *
 * Paths below are relative to /root/reference/self_benchmark/a64fx/.
 *
 * Pinning status of each function (what independently fixes its answers):
 *   oracle_spmm_f32              scipy CSR @ X and dense fp64 A @ X on the recipe of
 *                                tests/test_spmm.py:70-115; accumulate invariant
 *                                spmm(A,X,out0) == out0 + A@X; feature-width sweep
 *                                across the reference's 16/64-float block edges;
 *                                bit-for-bit against the compiled reference op
 *                                (oracle/_ref) wherever that is built.
 *   oracle_divide_work           closed form + brute force (tests/test_oracle_spmm.py).
 *   oracle_distribute_work_for_row
 *                                hand-worked small cases; the reference holds no
 *                                assertion for it (tests/test_spmm.py:60 only prints):
 *                                PARITY UNPINNED beyond those cases.  It balances CPU
 *                                threads and has no effect on results.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* model/ops/src/utils.cpp:3 */
static int divup(int x, int y) { return (x + y - 1) / y; }

/* model/ops/src/utils.cpp:6-16 -- even split of `total_work` over `num_threads`
 * (ceil(remaining / threads_left) per step; the last bound is forced to total). */
void oracle_divide_work(int32_t *work_range, int32_t total_work, int32_t num_threads) {
    int remain = total_work;
    work_range[0] = 0;
    for (int i = 0; i < num_threads; i++) {
        int chunk = divup(remain, num_threads - i);
        work_range[i + 1] = work_range[i] + chunk;
        remain -= chunk;
    }
    work_range[num_threads] = total_work;
}

/* model/ops/spmm_kernel.py:7-28 -- greedy split of rows over threads on the
 * per-row SUM OF VALUES (segment_csr(value, rowptr, "sum")), target total//T.
 * A bound is placed at row i (not i+1) when the running sum first exceeds the
 * target, and the running sum restarts from that row's own weight (:19-24).
 * Unset bounds stay at num_rows (:12,25).  fp32 arithmetic like the tensors the
 * reference loops over; exact whenever the values are small integers. */
void oracle_distribute_work_for_row(const int64_t *rowptr, const float *value, int64_t num_rows,
                                    int32_t num_threads, int32_t *row_splits) {
    float *w = (float *)malloc(sizeof(float) * (size_t)(num_rows > 0 ? num_rows : 1));
    double total_d = 0.0;
    for (int64_t r = 0; r < num_rows; r++) {
        float s = 0.0f;
        for (int64_t e = rowptr[r]; e < rowptr[r + 1]; e++) s += value[e];
        w[r] = s;
        total_d += (double)s;
    }
    float total = (float)total_d;
    float target = floorf(total / (float)num_threads); /* tensor // int on fp32 */
    for (int t = 0; t <= num_threads; t++) row_splits[t] = (int32_t)num_rows;
    row_splits[0] = 0;
    float cur = 0.0f;
    int tid = 0;
    for (int64_t i = 0; i < num_rows; i++) {
        cur += w[i];
        if (cur > target && tid < num_threads) {
            row_splits[tid + 1] = (int32_t)i;
            tid++;
            cur = w[i];
        }
    }
    row_splits[num_threads] = (int32_t)num_rows;
    free(w);
}

/* model/ops/src/spmm.cpp:468-480 with kernel_1xN (:24-60 / :68-143): for one row,
 * every output element starts from the value already in `out` (:32-35, :78-95),
 * receives one fused multiply-add per stored element in CSR order (:37-53, :97-126)
 * and is stored back (:56-59, :128-142).  The reference walks the feature axis in
 * blocks of 64 floats plus one masked corner block (:452-479); blocks are independent
 * lanes of the same recurrence, so the element-wise recurrence below is identical
 * bit for bit.  Address arithmetic is 64-bit here; the reference truncates it to
 * `int` (:38-39, :98-99), which is an overflow hazard, not a semantic. */
static void spmm_rows(const int64_t *rowptr, const int64_t *col, const float *value, const float *mat,
                      float *out, int64_t row_begin, int64_t row_end, int64_t feat) {
    for (int64_t m = row_begin; m < row_end; m++) {
        float *o = out + m * feat;
        const int64_t e0 = rowptr[m], e1 = rowptr[m + 1];
        for (int64_t e = e0; e < e1; e++) {
            const float a = value[e];
            const float *b = mat + col[e] * feat;
            for (int64_t n = 0; n < feat; n++) o[n] = fmaf(a, b[n], o[n]);
        }
    }
}

/* model/ops/src/spmm.cpp:327-507 (`computation_ops.spmm`).
 *   out[m,:] += sum_{e in row m} value[e] * mat[col[e],:]   for m in [0, sparse_rows)
 * Thread t owns rows [row_split[t], row_split[t+1]) (:421-422); a NULL split falls
 * back to divide_work over the rows (:399-403).  Returns 0, or -1 on bad arguments
 * (the reference asserts on rank/shape, :341-348). */
int oracle_spmm_f32(const int64_t *rowptr, const int64_t *col, const float *value, const float *mat,
                    float *out, int64_t sparse_rows, int64_t feat, const int32_t *row_split,
                    int32_t num_threads) {
    if (!rowptr || !out || sparse_rows < 0 || feat < 0 || num_threads < 1) return -1;
    if (sparse_rows == 0 || feat == 0) return 0;
    int32_t *own = NULL;
    if (row_split == NULL) {
        own = (int32_t *)malloc(sizeof(int32_t) * (size_t)(num_threads + 1));
        oracle_divide_work(own, (int32_t)sparse_rows, num_threads);
        row_split = own;
    }
#ifdef _OPENMP
#pragma omp parallel for schedule(static, 1) num_threads(num_threads)
#endif
    for (int t = 0; t < num_threads; t++) {
        spmm_rows(rowptr, col, value, mat, out, row_split[t], row_split[t + 1], feat);
    }
    free(own);
    return 0;
}

int oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* out[r][j] = fmaf(q[r][j], scale[r], zero_point[r]): the single-rounding multiply-add the
 * reference's dequantisation kernels use (svmla, quantization_arm.cpp:263-266).  Exact fmaf
 * from libm / the FMA unit; numpy has no fused multiply-add. */
void oracle_fma_rows_f32(const float *q, const float *scale, const float *zero_point, float *out,
                         int64_t rows, int64_t feat) {
    for (int64_t r = 0; r < rows; r++) {
        const float s = scale[r], z = zero_point[r];
        for (int64_t j = 0; j < feat; j++) out[r * feat + j] = fmaf(q[r * feat + j], s, z);
    }
}
