/*
 * gnn_agg.h -- C ABI of libgnnagg.so: the aggregation hot path of a full-batch,
 * graph-partitioned GCN/GraphSAGE trainer, written for AMD MI355X (gfx950).
 *
 * Every pointer is a DEVICE pointer unless its comment says "host".  `stream` is a
 * hipStream_t passed as void* (NULL = the default stream).  All entry points only
 * enqueue work on `stream` unless their comment says they synchronise.  They return
 * GNNAGG_OK or an error code; gnnagg_last_error() gives the message of the calling
 * thread's last failure.  Results are deterministic: no floating-point atomics are
 * used anywhere, so two runs on the same inputs are bit-identical.
 *
 * Reference paths cited below are relative to self_benchmark/a64fx/ of
 * zhuangbility111/GNN_benchmark.
 */
#ifndef GNN_AGG_H
#define GNN_AGG_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GNNAGG_OK 0
#define GNNAGG_ERR_INVALID 1     /* bad argument (null pointer, negative size, bad alignment, index out of range) */
#define GNNAGG_ERR_HIP 2         /* a HIP runtime call failed */
#define GNNAGG_ERR_UNSUPPORTED 3 /* sizes beyond what the kernels address (see each function) */

/* Raised whenever an exported prototype changes, an entry point goes away or the meaning of an argument changes
 * (2: `src_rows` in the row gathers, `workspace_bytes` in the weight-gradient entry points, 12 values from
 * gnnagg_plan_info; 3: the measurement probes left the library, gnnagg_plan_spmm_two_sources_f32 and gnnagg_plans_release came; 4: the two gnnagg_plan_spmm_dense_then_* entry points came; 5: gnnagg_argsort_i64 and gnnagg_runs_i64 came; 6: both take a workspace, gnnagg_argsort_workspace_bytes and
 * gnnagg_runs_workspace_bytes came).  Every binding compares it with
 * gnnagg_abi_version() of the library it loaded before the first call. */
#define GNNAGG_ABI_VERSION 6

/* Version of this ABI (GNNAGG_ABI_VERSION of the built library).  No reference counterpart. */
int gnnagg_abi_version(void);

/* Message of the calling thread's most recent failure ("" if none).  Host string,
 * valid until the next failing call on the same thread.  Replaces the c10::Error text
 * raised by CHECK_CPU / CHECK_INPUT (model/ops/src/utils.h:12-13). */
const char *gnnagg_last_error(void);

/* ---------------------------------------------------------------------------------
 * CSR SpMM, out[m,:] += sum_{e in row m} value[e] * mat[col[e],:]  for m < sparse_rows.
 *
 * Replaces `computation_ops.spmm(rowptr, col, value, mat, out, sparse_rows,
 * parallel_row_split, parallel_col_split)` = spmm_cpu_optimized_no_tile_v1
 * (model/ops/src/spmm.h:3-6, model/ops/src/spmm.cpp:327-507, bound at
 * model/ops/src/ops.cpp:23).  Same accumulate-into-`out` semantics (spmm.cpp:32-35,
 * :78-95) and the same int64/int64/fp32 CSR arrays.  The two CPU thread-split
 * arguments have no meaning on a GPU and are not part of this signature.
 *   rowptr int64 [sparse_rows+1], col int64 [nnz], value fp32 [nnz]
 *   mat    fp32 row-major [dense_rows, feat] (contiguous), out fp32 [sparse_rows, feat]
 * Each row is one fp32 FMA chain in CSR order starting from out[m,:], exactly the
 * recurrence of kernel_1xN (spmm.cpp:37-53).  Column indices are NOT range-checked
 * here (the reference does not check them either); use a plan for checked inputs.
 * ------------------------------------------------------------------------------- */
int gnnagg_spmm_csr_f32(const int64_t *rowptr, const int64_t *col, const float *value, const float *mat,
                        float *out, int64_t sparse_rows, int64_t feat, void *stream);

/* ---------------------------------------------------------------------------------
 * Cached schedule ("plan") of one sparse matrix.
 *
 * Replaces the per-matrix CPU work split the reference computes once and caches on
 * the sparse object: distribute_work_for_row + get/set_work_range[_for_transpose]
 * (model/ops/spmm_kernel.py:7-28, :48-57, :80-87).  On the GPU the cached object is a
 * degree-binned row schedule: rows ordered by degree class (powers of two of the row
 * length), longest rows first, and column indices narrowed to int32.  Rows above a
 * length threshold are fetched by a whole thread block each (gathers staged through
 * LDS), the rest by groups of 16-64 lanes.  Every row is
 * still one fp32 FMA chain in CSR order, so results are bit-identical to
 * gnnagg_spmm_csr_f32 and to the reference's CPU operator.
 *
 * gnnagg_plan_create reads rowptr/col on `stream`, validates them (rowptr[0]==0,
 * non-decreasing, rowptr[rows]==nnz, 0 <= col < cols) and SYNCHRONISES the stream; it
 * allocates device memory it owns.  The plan keeps no reference to rowptr/col after
 * it returns.  rows, cols < 2^31 and nnz < 2^40 (GNNAGG_ERR_UNSUPPORTED otherwise).
 * ------------------------------------------------------------------------------- */
typedef struct gnnagg_plan gnnagg_plan;

int gnnagg_plan_create(const int64_t *rowptr, const int64_t *col, int64_t rows, int64_t cols, int64_t nnz,
                       void *stream, gnnagg_plan **plan_out);

/* The same with the schedule's tuning values given explicitly (NULL, or a field left 0: the default).
 *   long_row_threshold   rows longer than this get a lane group of their own at the head of the launch (256)
 *   block_row_threshold  rows longer than this run in the block-per-row kernel (max(2048, nnz / 4096))
 *   rows_per_group       rows a lane group walks, one after the other, in the middle of the launch (2; at most 16)
 *   short_rows_per_group the same for the rows of at most 8 elements at the end of the launch (2; at most 16)
 *   lanes_per_row, loads_per_lane  launch shape of the row kernel instead of the one chosen from the feature
 *                        width: lanes x loads x (4, 2 or 1 floats, by alignment) must cover the width, else the
 *                        product calls return GNNAGG_ERR_INVALID.  Instances: 16x1, 16x2, 16x3, 32x1, 32x2, 64x1,
 *                        64x2, 64x3, 64x4, 64x5, 64x6, 64x8.
 * Results do not depend on any of them (every row stays one FMA chain); they only move time.  No counterpart
 * in the reference (its cached split depends on the thread count alone, model/ops/spmm_kernel.py:48-57). */
typedef struct gnnagg_plan_options {
    int32_t long_row_threshold;
    int32_t block_row_threshold;
    int32_t rows_per_group;
    int32_t short_rows_per_group;
    int32_t lanes_per_row;
    int32_t loads_per_lane;
    int32_t reserved[2]; /* must be 0 */
} gnnagg_plan_options;

int gnnagg_plan_create_ex(const int64_t *rowptr, const int64_t *col, int64_t rows, int64_t cols, int64_t nnz,
                          const gnnagg_plan_options *options, void *stream, gnnagg_plan **plan_out);

/* Gives a plan back (NULL is accepted).  Makes no HIP call and never synchronises -- safe from a destructor in the
 * middle of a training step or while a stream is being captured; work already enqueued with the plan runs to its
 * end.  The plan's device memory is released by the next gnnagg_plan_create[_ex] on the same device (set-up work
 * that synchronises anyway), after a device synchronisation. */
int gnnagg_plan_destroy(gnnagg_plan *plan);

/* Releases, now, the device memory of every plan of the current device that was handed to gnnagg_plan_destroy
 * (column indices narrowed to 32 bits and the row schedule: 4 bytes per stored element + 16 per row, about 0.5 GB
 * for a 7 M-row / 100 M-element matrix).  Synchronises the device first, so call it where that is safe -- the end
 * of graph set-up, between epochs -- and never while a stream is being captured.  A process that drops plans and
 * creates no new one on that device would otherwise keep their memory until it ends.  No reference counterpart. */
int gnnagg_plans_release(void);

/* out (+)= A @ mat through a plan.  `value` is the fp32 [nnz] array in the CSR order
 * the plan was built from.  accumulate != 0: out += A@mat (the reference semantics,
 * spmm.cpp:32-35).  accumulate == 0: out = A@mat, every row written (fuses the
 * `torch.zeros` the reference allocates before the local aggregation,
 * model/layers/aggregator.py:67-70, :167-170).  Allocates nothing and does not
 * synchronise the host.  A plan owns a few events (and, when it holds very long rows, a
 * side stream joined back into `stream` before the call returns), so two calls on the
 * SAME plan must not overlap: issue them on one stream, or order them yourself (a call that
 * arrives while another thread is still inside a call on the same plan returns
 * GNNAGG_ERR_INVALID).  Calls on different plans are independent. */
int gnnagg_plan_spmm_f32(gnnagg_plan *plan, const float *value, const float *mat, float *out, int64_t feat,
                         int accumulate, void *stream);

/* The same product for operands that are column blocks of wider row-major arrays: row r of
 * mat starts at mat + r * mat_stride, row r of out at out + r * out_stride (strides in
 * floats, each at least feat).  This is what lets a layer keep [A x | x] side by side in one
 * [rows, 2 * feat] array and run lin_neigh and lin_self (model/layers/sageconv.py:87-88) as
 * ONE dense product, without copying either half: the aggregation reads the right half and
 * writes the left one.  Results equal gnnagg_plan_spmm_f32 on contiguous copies bit for bit. */
int gnnagg_plan_spmm_strided_f32(gnnagg_plan *plan, const float *value, const float *mat, int64_t mat_stride,
                                 float *out, int64_t out_stride, int64_t feat, int accumulate, void *stream);

/* The same product with the dense operand in TWO arrays: column c of the matrix reads row c of mat for
 * c < mat_rows and row c - mat_rows of mat2 above (plan->cols - mat_rows rows; strides in floats).  This is what
 * lets the local aggregation and the aggregation of the received halo rows run as ONE launch, one FMA chain per
 * output row: build the plan over [A_local | A_from] (every row: its local elements, then its halo elements with
 * column + N_local -- the numbering the reference's raw-halo path gives halo nodes itself,
 * data_manager/DataProcessor.py:29-60) and pass the layer input as mat and recv_buf as mat2.  Each output row is
 * then written once instead of written by the local product and read and written again by the post-aggregation
 * (model/layers/aggregator.py:67-70 then :102), with the same chain, hence the same bits.  Every row runs in the
 * lane-group kernel (no block-per-row side launch).  Allocates nothing, no host synchronisation. */
int gnnagg_plan_spmm_two_sources_f32(gnnagg_plan *plan, const float *value, const float *mat, int64_t mat_stride,
                                     int64_t mat_rows, const float *mat2, int64_t mat2_stride, float *out,
                                     int64_t out_stride, int64_t feat, int accumulate, void *stream);

/* The one-launch product when the received rows are still in their exchange format (a 16-bit or quantised
 * exchange): the plan is over [A_local | A_from] as above, `split` int32 [rows] says how many of a row's leading
 * stored elements belong to A_local; those gather fp32 rows of mat, the others rows (column - mat_rows) of the
 * second source -- bf16 rows (mat2_bf16, stride in 16-bit values; what gnnagg_plan_spmm_bf16_f32 gathers), or the
 * packed bytes / parameters / row codes gnnagg_plan_spmm_quantized_f32 gathers.  Every output row is the FMA chain
 * of the local product continued by the one of the product from the exchange format, hence the same bits as those
 * two calls (model/layers/aggregator.py:70 then :85-104; backward :170 then :180-199).  feat a multiple of 4, fp32
 * rows 16-byte aligned.  A matrix whose rows all have split == their length is a plain product.  Allocate nothing,
 * no host synchronisation. */
int gnnagg_plan_spmm_dense_then_bf16_f32(gnnagg_plan *plan, const float *value, const int32_t *split, const float *mat,
                                         int64_t mat_stride, int64_t mat_rows, const uint16_t *mat2_bf16,
                                         int64_t mat2_stride, float *out, int64_t out_stride, int64_t feat,
                                         int accumulate, void *stream);
int gnnagg_plan_spmm_dense_then_quantized_f32(gnnagg_plan *plan, const float *value, const int32_t *split,
                                              const float *mat, int64_t mat_stride, int64_t mat_rows,
                                              const uint8_t *packed, const float *params, const int32_t *row_code,
                                              int bits, float *out, int64_t out_stride, int64_t feat, int accumulate,
                                              void *stream);

/* Host-side description of a plan, info[0..11] (host pointer):
 * rows, cols, nnz, rows handled by the block-per-row kernel (longer than the next
 * entry), that length threshold, rows with no stored element, largest row length, rows
 * handled per lane group, rows of at most 8 elements, rows per lane group for those, rows
 * with a lane group of their own (longer than the next entry), that length threshold. */
int gnnagg_plan_info(const gnnagg_plan *plan, int64_t *info);

/* Kernel timing of a plan, for benchmarks.  After gnnagg_plan_profile(plan, 1) every
 * gnnagg_plan_spmm_f32 call records HIP events on its stream around the whole call and
 * around its dominant kernel (the launch that walks the rows of the first feature tile;
 * the only launch unless the feature row is wider than one tile).
 * gnnagg_plan_profile_read SYNCHRONISES on the last recorded events and returns, in
 * milliseconds, ms[0] = that kernel, ms[1] = the whole call (all kernels), of the most
 * recent call (host pointer; -1 when nothing was recorded).  Replaces the std::chrono
 * prints the reference compiles in under `#define PROFILE` (spmm.cpp:12, :411-413,
 * :486-491). */
int gnnagg_plan_profile(gnnagg_plan *plan, int enable);
int gnnagg_plan_profile_read(gnnagg_plan *plan, double *ms);

/* ---------------------------------------------------------------------------------
 * Transposed CSR arrays (colptr, row_T, value_T) of a CSR matrix: entries grouped by
 * column, rows ascending inside a column.  Replaces the torch_sparse storage accessors
 * the backward wrapper reads (model/ops/spmm_kernel.py:76-78: storage.colptr(),
 * storage.row_T(), storage.value_T()), so that `A^T @ G` runs through the same SpMM.
 * Outputs: colptr int64 [cols+1], row_t int64 [nnz], value_t fp32 [nnz].
 * `value`/`value_t` may both be NULL (structure only).  Allocates temporaries and
 * SYNCHRONISES the stream.  rows, cols < 2^31.
 * ------------------------------------------------------------------------------- */
int gnnagg_csr_transpose(const int64_t *rowptr, const int64_t *col, const float *value, int64_t rows,
                         int64_t cols, int64_t nnz, int64_t *colptr, int64_t *row_t, float *value_t,
                         void *stream);

/* ---------------------------------------------------------------------------------
 * COO -> CSR: entries ordered by (row, col), repeated (row, col) pairs KEPT, rowptr by
 * counting.  Replaces `SparseTensor(row=, col=, value=, sparse_sizes=)` at the call
 * sites data_manager/DataProcessor.py:104-116, :458-502 (torch_sparse, third party).
 * Outputs: rowptr int64 [rows+1], col_out int64 [nnz], value_out fp32 [nnz] (value and
 * value_out may both be NULL).  Validates 0 <= row < rows, 0 <= col < cols.  Allocates
 * temporaries and SYNCHRONISES the stream.  rows, cols < 2^31.
 * ------------------------------------------------------------------------------- */
int gnnagg_coo_to_csr(const int64_t *row, const int64_t *col, const float *value, int64_t nnz, int64_t rows,
                      int64_t cols, int64_t *rowptr, int64_t *col_out, float *value_out, void *stream);

/* ---------------------------------------------------------------------------------
 * Sorting and run detection for the index-map builders (set-up time).  `workspace`: device memory of at least
 * gnnagg_*_workspace_bytes(n) bytes, 16-byte aligned, for the call's temporaries; NULL: the call allocates them itself
 * and waits for its kernels before it returns.  gnnagg_argsort_i64 waits for the stream once either way (the
 * largest key decides the number of passes), gnnagg_runs_i64 too (the number of runs).  The reference walks sorted edge lists with per-edge Python loops
 * (data_manager/DataProcessor.py:39-53 halo renumbering, :238-246 pre/post decision, :434-444 buffer-row
 * renumbering) after `torch.argsort` (:21, :259, :306) and `torch.unique` (:127); on the device the same maps are
 * a stable sort plus the run structure of the sorted list.
 *
 * gnnagg_argsort_i64: perm int64 [n] such that x[perm] is ascending, equal keys in their input order (a stable
 * radix sort, 8 bits a pass over the bits the largest key needs); sorted (may be NULL) receives x[perm].  Keys must
 * be non-negative (GNNAGG_ERR_INVALID otherwise); n < 2^32.
 *
 * gnnagg_runs_i64: the runs of equal neighbours of x (a sorted list, or any list: torch.unique_consecutive).  A
 * run also starts at every position listed in forced_starts (int64 [forced_count], positions outside [0, n) are
 * ignored; NULL with 0): the per-rank segments of data_manager/DataProcessor.py:432-445, across which equality is
 * not carried.  Outputs, each may be NULL: uniq int64 [runs] the value of each run, inverse int64 [n] the run of
 * each position, counts int64 [runs] the length of each run (all three arrays sized n by the caller); *runs_out
 * (host) the number of runs.
 * ------------------------------------------------------------------------------- */
int64_t gnnagg_argsort_workspace_bytes(int64_t n);
int gnnagg_argsort_i64(const int64_t *x, int64_t n, int64_t *perm, int64_t *sorted, void *workspace,
                       int64_t workspace_bytes, void *stream);
int64_t gnnagg_runs_workspace_bytes(int64_t n);
int gnnagg_runs_i64(const int64_t *x, int64_t n, const int64_t *forced_starts, int64_t forced_count, int64_t *uniq,
                    int64_t *inverse, int64_t *counts, int64_t *runs_out, void *workspace, int64_t workspace_bytes,
                    void *stream);

/* ---------------------------------------------------------------------------------
 * Boundary-row gather, out[i,:] = src[index[i],:].  Replaces
 * `torch.index_select(local_nodes_feat, 0, idx_nodes_send_to_others, out=send_buf)`
 * (model/layers/aggregator.py:51).  src fp32 [src_rows, feat], index int64 [n_index].  An index outside
 * [0, src_rows) is never dereferenced: its output row is filled with NaN (torch.index_select raises for it;
 * raising needs the index values on the host -- gnnagg_check_index below does that once per index list).
 * ------------------------------------------------------------------------------- */
int gnnagg_gather_rows_f32(const float *src, int64_t src_rows, const int64_t *index, float *out, int64_t n_index,
                           int64_t feat, void *stream);

/* The same gather with the result rows stored as bf16 (round to nearest even, NaN -> 0x7FC0): the gather and the
 * `send_buf_fp16.copy_(send_buf)` of a 16-bit exchange (model/layers/aggregator.py:51 followed by
 * communicator/communicator.py:128) in one pass, the same bits as the two apart.  out: bf16 [n_index, feat];
 * feat a multiple of 4, src 16-byte and out 8-byte aligned (GNNAGG_ERR_UNSUPPORTED otherwise). */
int gnnagg_gather_rows_f32_bf16(const float *src, int64_t src_rows, const int64_t *index, void *out, int64_t n_index,
                                int64_t feat, void *stream);

/* Range check of an index list held on the device: GNNAGG_OK when every (index[i] >> shift) lies in [0, bound),
 * GNNAGG_ERR_INVALID (naming the first offending position found) otherwise.  index: `count` integers of
 * elem_bytes 4 (int32) or 8 (int64).  SYNCHRONISES the stream: meant to run once per index list (the boundary
 * row list of a graph, the column array handed to gnnagg_spmm_csr_f32, the row codes of a packed buffer), not per
 * call.  Replaces the bounds checks torch's indexing ops make on the host in the reference
 * (torch.index_select / index_add_, model/layers/aggregator.py:51, :197-199). */
int gnnagg_check_index(const void *index, int elem_bytes, int64_t count, int shift, int64_t bound, void *stream);

/* ---------------------------------------------------------------------------------
 * Fused layer epilogue around the aggregation path (the full train-step workload):
 *   y[i,f]  = relu(z[i,f] / row_div[i] + bias[f]) * (keep[i,f] ? scale : 0)     forward
 *   grad_z  = (y > 0 ? grad_y * scale : 0) / row_div[i]                          backward
 *   bias_partial[b, f] = sum over the rows of block b of (y > 0 ? grad_y * scale : 0)
 * z, y, grad_* fp32 [rows, feat] (y may alias z, grad_z may alias grad_y), bias fp32
 * [feat], keep uint8 [rows, feat] or NULL (no dropout; pass scale = 1), row_div fp32 [rows]
 * or NULL (no division).  bias_partial is NULL, or fp32 [blocks, feat] with blocks =
 * gnnagg_relu_dropout_backward_blocks(rows, feat) (0 = this width cannot use it: needs
 * feat % 4 == 0 and 256 % (feat / 4) == 0); summing it over its first axis gives the bias
 * gradient without another pass over the activations (fixed order: deterministic).
 * row_div carries the reference layer's `out /= graph.in_degrees`
 * (model/layers/sageconv.py:84) moved behind the dense product, where it costs no pass of
 * its own.  The reference runs its epilogue (dropout, LayerNorm, ReLU) as separate torch
 * ops (model/DistSAGE.py:55-66); this fused form belongs to this build's GCN layer stack.
 * ------------------------------------------------------------------------------- */
int gnnagg_bias_relu_dropout_f32(const float *z, const float *bias, const uint8_t *keep, const float *row_div,
                                 float scale, float *y, int64_t rows, int64_t feat, void *stream);
int gnnagg_relu_dropout_backward_blocks(int64_t rows, int64_t feat);
int gnnagg_relu_dropout_backward_f32(const float *grad_y, const float *y, const float *row_div, float scale,
                                     float *grad_z, float *bias_partial, int64_t rows, int64_t feat, void *stream);

/* ---------------------------------------------------------------------------------
 * Weight gradient of a dense layer, w_grad[fi, fo] = x^T @ g, with x fp32 [rows, fi] and
 * g fp32 [rows, fo] row-major, rows in the millions, fi, fo <= 256 (GNNAGG_ERR_UNSUPPORTED
 * otherwise).  Hand-written fp32 MFMA kernel plus a fixed-order reduction of per-slice
 * partial results: deterministic.  `workspace` is caller-provided device memory of
 * gnnagg_wgrad_workspace_bytes(rows, fi, fo) bytes (0 = unsupported shape); nothing is
 * allocated here.  `workspace_bytes` is the size of what the caller passes: less than that
 * figure returns GNNAGG_ERR_INVALID before anything is launched.  Part of this build's GCN layer stack (the reference leaves this product
 * to torch's Linear backward, model/layers/sageconv.py:87-88).
 * ------------------------------------------------------------------------------- */
int64_t gnnagg_wgrad_workspace_bytes(int64_t rows, int64_t fi, int64_t fo);
int gnnagg_wgrad_f32(const float *x, const float *g, float *w_grad, void *workspace, int64_t workspace_bytes,
                     int64_t rows, int64_t fi, int64_t fo, void *stream);
/* The same with x and / or g being column blocks of wider row-major arrays (row strides in
 * floats): the two halves of a SAGE layer's [A x | x] operand are read where they lie. */
int gnnagg_wgrad_strided_f32(const float *x, int64_t x_stride, const float *g, int64_t g_stride, float *w_grad,
                             void *workspace, int64_t workspace_bytes, int64_t rows, int64_t fi, int64_t fo, void *stream);

/* gnnagg_wgrad_f32 for callers that cannot allocate device memory (code recorded into a HIP graph, tight serving
 * loops, harnesses that forbid hipMalloc): no workspace argument, the per-slice partial results go to a 64 MiB
 * device array built into the library (one per GPU the library runs on, held until the process ends), which fits
 * every shape gnnagg_wgrad_f32 takes; fi or fo above 256 return GNNAGG_ERR_UNSUPPORTED.  Same kernels, same result
 * bit for bit.  Calls no hipMalloc / hipFree; its first call on a device looks the array's address up (make that call
 * outside any capture).  All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two
 * host threads) race -- order them.  No counterpart in the reference. */
int gnnagg_wgrad_noalloc_f32(const float *x, const float *g, float *w_grad, int64_t rows, int64_t fi, int64_t fo,
                             void *stream);

/* ---------------------------------------------------------------------------------
 * Dense layer product with the elementwise work behind it fused in (fp32 MFMA, hand-written):
 *   y = relu((x @ w) / row_div + bias) * (keep ? scale : 0)
 * x fp32 [rows, k] (row stride x_stride floats), w fp32 [k, n] row-major (row stride
 * w_stride), y fp32 [rows, n] (row stride y_stride); bias fp32 [n] or NULL; row_div fp32
 * [rows] or NULL; relu 0/1; keep_bits NULL (nothing dropped; pass scale = 1) or uint32
 * [rows, ceil(n / 32)] as written by gnnagg_pack_keep_bits from a uint8 [rows, n] mask: bit q
 * of word (r, v) is keep[r, 32 * v + q].  Shapes: k % 16 == 0, n % 4 == 0, n <= 256, 16-byte
 * aligned operands and row strides (GNNAGG_ERR_UNSUPPORTED otherwise;
 * gnnagg_linear_shape_supported tells beforehand).  The contraction is summed in a fixed
 * order: deterministic.
 *
 * Its counterpart in the gradient direction rides on the weight-gradient kernel below: with
 * g the gradient with respect to y,
 *   pre       = (y > 0 ? g * scale : 0)          bias_grad[f] = sum over rows of pre[:, f]
 *   grad_z    = pre / row_div                     (written out, [rows, fo] contiguous: the
 *                                                  operand of the input-gradient product)
 *   w_grad    = x^T @ grad_z
 * in one pass over x, g and y.  y = NULL: no ReLU / dropout behind the product (pre = g *
 * scale); grad_z = NULL: not written (a caller that only wants w_grad and bias_grad, e.g.
 * the SAGE layer's `+ bias`, model/layers/sageconv.py:91).  Needs fi, fo <= 256 and multiples of 4, 16-byte aligned
 * operands and row strides; workspace of gnnagg_wgrad_relu_dropout_backward_workspace_bytes
 * (0 = unsupported shape) bytes, its size passed as workspace_bytes (too small: GNNAGG_ERR_INVALID);
 * nothing is allocated.  Deterministic.
 * The reference leaves these products to torch's Linear and runs dropout / ReLU as separate
 * ops (model/layers/sageconv.py:87-91, model/DistSAGE.py:49-53); the fused forms belong to
 * this build's GCN layer stack.
 * ------------------------------------------------------------------------------- */
int gnnagg_linear_shape_supported(int64_t k, int64_t n);
int gnnagg_pack_keep_bits(const void *keep, uint32_t *bits, int64_t rows, int64_t feat, void *stream);
int gnnagg_linear_bias_relu_dropout_f32(const float *x, int64_t x_stride, const float *w, int64_t w_stride,
                                        const float *bias, const uint32_t *keep_bits, const float *row_div,
                                        float scale, int relu, float *y, int64_t y_stride, int64_t rows, int64_t k,
                                        int64_t n, void *stream);
/* The same with both operands of the product rounded to bf16 (round to nearest even) on their way
 * into the matrix units and fp32 accumulation: config 5's bf16-input variant.  HBM-bound. */
int gnnagg_linear_bias_relu_dropout_bf16_f32(const float *x, int64_t x_stride, const float *w, int64_t w_stride,
                                             const float *bias, const uint32_t *keep_bits, const float *row_div,
                                             float scale, int relu, float *y, int64_t y_stride, int64_t rows,
                                             int64_t k, int64_t n, void *stream);
/* The same in fp32 accuracy on the bf16 matrix units: every fp32 operand value is cut into three bf16 pieces
 * (hi = bf16(v), mid = bf16(v - hi), lo = bf16(v - hi - mid): both differences are exact) on its way into LDS, and
 * a product is the sum of six bf16 MFMAs (hi*hi, hi*mid, mid*hi, mid*mid, hi*lo, lo*hi) accumulated in fp32; what
 * is left out is below 2^-24 |x||w| per term, an fp32 rounding.  192 MFMA cycles per 32 x 32 x 16 block of
 * products instead of the fp32 MFMA's 512. */
int gnnagg_linear_bias_relu_dropout_bf16x3_f32(const float *x, int64_t x_stride, const float *w, int64_t w_stride,
                                               const float *bias, const uint32_t *keep_bits, const float *row_div,
                                               float scale, int relu, float *y, int64_t y_stride, int64_t rows,
                                               int64_t k, int64_t n, void *stream);
/* The same layer writing its result packed (the format of gnnagg_bias_relu_dropout_pack_f32 below: every row's
 * non-zero values at its front, plus the header of (bitmap, non-zeros in front) pairs): n in {32, 64, 128, 256},
 * ReLU always on, y_packed [rows, n] contiguous with 4 floats of slack behind it, header uint32 [rows, 2 * (n / 32)];
 * bf16_inputs picks the product's form: 0 fp32 MFMA, 1 operands rounded to bf16, 2 three bf16 pieces per operand. */
int gnnagg_linear_bias_relu_dropout_pack_f32(const float *x, int64_t x_stride, const float *w, int64_t w_stride,
                                             const float *bias, const uint32_t *keep_bits, const float *row_div,
                                             float scale, float *y_packed, uint32_t *header, int64_t rows, int64_t k,
                                             int64_t n, int bf16_inputs, void *stream);
int64_t gnnagg_wgrad_relu_dropout_backward_workspace_bytes(int64_t rows, int64_t fi, int64_t fo);
/* (the _bf16_ form below takes the same arguments and workspace; it rounds x and grad_z to bf16 for the
 * product x^T @ grad_z -- fp32 accumulation -- while grad_z and bias_grad are computed and written in fp32) */
int gnnagg_wgrad_relu_dropout_backward_f32(const float *x, int64_t x_stride, const float *grad_y, int64_t grad_stride,
                                           const float *y, int64_t y_stride, const float *row_div, float scale,
                                           float *grad_z, float *w_grad, float *bias_grad, void *workspace,
                                           int64_t workspace_bytes, int64_t rows, int64_t fi, int64_t fo, void *stream);
/* The same when the layer's output was written packed: which units were active is read from the bitmaps of its
 * header (fo in {32, 64, 128, 256}) instead of from y; bf16_inputs picks the product's form (0 fp32 MFMA, 1 operands
 * rounded to bf16, 2 three bf16 pieces per operand). */
int gnnagg_wgrad_relu_dropout_backward_from_header_f32(const float *x, int64_t x_stride, const float *grad_y,
                                                       int64_t grad_stride, const uint32_t *header, const float *row_div,
                                                       float scale, float *grad_z, float *w_grad, float *bias_grad,
                                                       void *workspace, int64_t workspace_bytes, int64_t rows, int64_t fi,
                                                       int64_t fo, int bf16_inputs, void *stream);
int gnnagg_wgrad_relu_dropout_backward_bf16_f32(const float *x, int64_t x_stride, const float *grad_y,
                                                int64_t grad_stride, const float *y, int64_t y_stride,
                                                const float *row_div, float scale, float *grad_z, float *w_grad,
                                                float *bias_grad, void *workspace, int64_t workspace_bytes, int64_t rows,
                                                int64_t fi, int64_t fo, void *stream);
/* (the _bf16x3_ form: the product x^T @ grad_z in fp32 accuracy on the bf16 matrix units, every value of x and
 * grad_z cut into three bf16 pieces, six bf16 MFMAs a product -- see gnnagg_linear_bias_relu_dropout_bf16x3_f32) */
int gnnagg_wgrad_relu_dropout_backward_bf16x3_f32(const float *x, int64_t x_stride, const float *grad_y,
                                                  int64_t grad_stride, const float *y, int64_t y_stride,
                                                  const float *row_div, float scale, float *grad_z, float *w_grad,
                                                  float *bias_grad, void *workspace, int64_t workspace_bytes, int64_t rows,
                                                  int64_t fi, int64_t fo, void *stream);

/* ---------------------------------------------------------------------------------
 * The elementwise chain between two SAGE layers (model/DistSAGE.py:49-53: F.dropout, LayerNorm
 * over the features, F.relu) as one pass each way:
 *   y = relu(layer_norm(z * keep * scale; gamma, beta, eps))
 * z fp32 [rows, feat] contiguous (the layer output), keep uint8 [rows, feat] (NULL: nothing
 * dropped), gamma / beta fp32 [feat].  y is written with row stride y_stride floats: the next
 * layer keeps its input in the right half of a [rows, 2 * feat] array whose left half receives
 * the aggregation (gnnagg_plan_spmm_strided_f32).  The backward takes the gradient with its own
 * row stride, the SAME z / keep / scale / gamma / beta / eps (the row moments are taken again,
 * nothing else is kept from the forward), writes grad_z fp32 [rows, feat] and, when `partial`
 * is given, per-block sums for the LayerNorm parameters: partial fp32 [blocks, 2, feat]
 * (blocks = gnnagg_dropout_layernorm_relu_blocks(rows, feat)); summing partial[:, 0, :] over the
 * blocks gives d/d gamma, partial[:, 1, :] d/d beta.  feat % 4 == 0, feat <= 1024
 * (GNNAGG_ERR_UNSUPPORTED otherwise; _blocks returns 0).  Allocates nothing, no host sync.
 * ------------------------------------------------------------------------------- */
int gnnagg_dropout_layernorm_relu_blocks(int64_t rows, int64_t feat);
int gnnagg_dropout_layernorm_relu_f32(const float *z, const uint8_t *keep, float scale, const float *gamma,
                                      const float *beta, float eps, float *y, int64_t y_stride, int64_t rows,
                                      int64_t feat, void *stream);
int gnnagg_dropout_layernorm_relu_backward_f32(const float *grad_y, int64_t grad_stride, const float *z,
                                               const uint8_t *keep, float scale, const float *gamma,
                                               const float *beta, float eps, float *grad_z, float *partial,
                                               int64_t rows, int64_t feat, void *stream);

/* ---------------------------------------------------------------------------------
 * Packed activations: the output of a ReLU + dropout layer with every row's non-zero values
 * moved to the front of the row (order kept, row stride still feat, the tail unspecified)
 * plus a header per row: for every 32 features a pair of 32-bit words, the bitmap of those
 * features (bit set = non-zero) and the number of non-zeros in front of them;
 * gnnagg_packed_header_words = 2 * feat / 32 words in all (0 = width not supported;
 * supported: 32, 64, 128, 256).  A gather of
 * such a row touches the header and the non-zero values only -- about a quarter of the row
 * in training.  Skipping the zeros leaves every row's FMA chain as it is (fma(v, 0, acc) ==
 * acc), so results equal the dense ones up to the sign of a zero.
 *   gnnagg_bias_relu_dropout_pack_f32: gnnagg_bias_relu_dropout_f32 writing the packed form
 *     (y_packed fp32 [rows, feat] -- allocate 4 floats more than rows * feat: the consumer's
 *     16-byte loads may run up to 3 floats past a row -- and header uint32 [rows, words]).
 *   gnnagg_relu_dropout_backward_packed_f32: gnnagg_relu_dropout_backward_f32 with the
 *     header's bitmap in place of the forward output; bias_partial is required.
 *   gnnagg_plan_spmm_packed_f32: gnnagg_plan_spmm_f32 whose dense operand is given packed.
 * Part of this build's GCN layer stack (no counterpart in the reference, which keeps
 * activations dense).  No allocation, no host synchronisation.
 * ------------------------------------------------------------------------------- */
int gnnagg_packed_header_words(int64_t feat);
int gnnagg_bias_relu_dropout_pack_f32(const float *z, const float *bias, const uint8_t *keep, const float *row_div,
                                      float scale, float *y_packed, uint32_t *header, int64_t rows, int64_t feat,
                                      void *stream);
int gnnagg_relu_dropout_backward_packed_f32(const float *grad_y, const uint32_t *header, const float *row_div,
                                            float scale, float *grad_z, float *bias_partial, int64_t rows, int64_t feat,
                                            void *stream);
int gnnagg_plan_spmm_packed_f32(gnnagg_plan *plan, const float *value, const float *y_packed, const uint32_t *header,
                                float *out, int64_t feat, int accumulate, void *stream);

/* ---------------------------------------------------------------------------------
 * Codec of the boundary buffers: fp32 rows <-> int2 / int4 / int8 (bits = 2, 4, 8).
 *
 * Row-packed layout, one segment per destination rank.  Replaces
 * `quantize_tensor_for_all_procs` / `dequantize_tensor_for_all_procs`
 * (model/ops/src/quantization_arm.cpp:364-479, called from quantizer.py:80-90) and, with a
 * single segment, `quantize_tensor` / `dequantize_tensor` (quantization_arm.cpp:302-362,
 * quantization_x86.cpp:17-162).  x / out fp32 [rows, feat]; params fp32 [rows, 2] =
 * (zero_point, scale) per row -- written by quantize (zero_point = row minimum, scale =
 * (max - min) / (2^bits - 1), 1 when that is 0), read by dequantize; packed uint8
 * [packed_rows, feat]: 8/bits consecutive rows of a segment share one byte per column, row
 * k of a group at bit (8/bits - k - 1) * bits, and every segment starts a new group.
 * row_range / packed_range: int32 [segments + 1] in DEVICE memory, prefix sums of the rows
 * and of the packed rows (ceil(rows_p * bits / 8)) per segment -- the reference's
 * `quantized_work_range_per_proc` (data_manager/CommBuffer.py:37-43) and what its
 * divide_work_v1 derives from it (quantization_arm.cpp:21-31).  q = rint((x - zero_point)
 * / scale) to nearest even; x' = fma(q, scale, zero_point).  The reference hard-codes 2
 * bits in the per-rank variant; 4 and 8 follow the same rule as its x86 kernels.
 * No allocation, no host synchronisation.
 *
 * Feature-packed layout with a width per row ("mixed bits").  Replaces
 * `quantize_tensor_v1` / `dequantize_tensor_v1` (quantization_x86.cpp:164-305, called from
 * quantizer.py:52-66).  params fp32 [rows, 3] = (bits, zero_point, scale): column 0 is read
 * (2, 4 or 8 per row), columns 1-2 written by quantize; feat_range int64 [rows + 1] in
 * device memory = byte offset of every row in `data`
 * (quantizer.py:69-77); 8/bits consecutive features share a byte, same shift rule.  A row
 * whose width is not 2, 4 or 8 is left alone and sets *bad_width (device int32, zeroed by
 * the caller) to 1 -- the reference prints an error for it (quantization_x86.cpp:241).
 * ------------------------------------------------------------------------------- */
int gnnagg_quantize_segments_f32(const float *x, uint8_t *packed, float *params, const int32_t *row_range,
                                 const int32_t *packed_range, int64_t segments, int64_t rows, int64_t packed_rows,
                                 int64_t feat, int bits, void *stream);
int gnnagg_dequantize_segments_f32(const uint8_t *packed, const float *params, float *out, const int32_t *row_range,
                                   const int32_t *packed_range, int64_t segments, int64_t rows, int64_t packed_rows,
                                   int64_t feat, int bits, void *stream);
/* Raw boundary rows straight into the packed bytes: gnnagg_quantize_segments_f32 whose fp32 row r is row index[r] of
 * src -- `torch.index_select(local_nodes_feat, 0, idx_nodes_send_to_others, out=send_buf)` followed by
 * `quantize_tensor_for_all_procs(send_buf, ...)` (model/layers/aggregator.py:51, communicator/communicator.py:281-311) as
 * one pass; same bytes and parameters, the gathered fp32 rows never written.  src fp32 [src_rows, feat] contiguous,
 * index int64 [rows]; an index outside [0, src_rows) is never dereferenced (row 0 is read in its place and the row's
 * two parameters are stored as NaN, so the row dequantises to NaN -- what gnnagg_gather_rows_f32 stores for such an
 * index; raising for it is gnnagg_check_index's part).  No allocation, no host synchronisation. */
int gnnagg_gather_quantize_segments_f32(const float *src, int64_t src_rows, const int64_t *index, uint8_t *packed,
                                        float *params, const int32_t *row_range, const int32_t *packed_range,
                                        int64_t segments, int64_t rows, int64_t packed_rows, int64_t feat, int bits,
                                        void *stream);
/* Pre-aggregation straight into the packed bytes: packed / params = quantize(A @ mat), every segment on its own --
 * `send_buf += A_to @ X` followed by `quantize_tensor_for_all_procs(send_buf, ...)` (model/layers/aggregator.py:44-49,
 * communicator/communicator.py:281-311; backward: :144-149 with the buffers' roles swapped) as one pass.  A is given as
 * CSR arrays (rowptr int64 [rows + 1], col int64, value fp32; the transposed arrays for the gradient direction), mat
 * fp32 with row stride mat_stride; the other arguments are gnnagg_quantize_segments_f32's.  Every result row is the
 * single FMA chain over its stored elements, in their order, that gnnagg_plan_spmm_f32 runs, and is quantised by the
 * same arithmetic, so parameters and bytes equal those of the two calls bit for bit while the fp32 rows are never
 * written or read.  feat a multiple of 4 up to 512, mat rows on 16-byte boundaries (GNNAGG_ERR_UNSUPPORTED otherwise:
 * use the two calls).  Column indices are not range-checked here (gnnagg_check_index).  No allocation, no host
 * synchronisation. */
int gnnagg_spmm_csr_quantize_segments_f32(const int64_t *rowptr, const int64_t *col, const float *value,
                                          const float *mat, int64_t mat_stride, uint8_t *packed, float *params,
                                          const int32_t *row_range, const int32_t *packed_range, int64_t segments,
                                          int64_t rows, int64_t packed_rows, int64_t feat, int bits, void *stream);
/* Post-aggregation straight from the packed bytes: gnnagg_plan_spmm_f32 whose dense operand
 * row c is given quantised -- packed / params as written by gnnagg_quantize_segments_f32 (or
 * received from a peer), row_code int32 [rows of the operand] = packed_row * 8 + position of
 * the row inside its byte group.  Each gathered value is fma(q, scale, zero_point), exactly
 * what gnnagg_dequantize_segments_f32 would have stored, so the result equals dequantise
 * followed by gnnagg_plan_spmm_f32 bit for bit, without the fp32 buffer ever being written
 * or read (the reference dequantises into recv_buf and then aggregates,
 * model/layers/aggregator.py:83-104).  feat % 4 == 0; row r of out starts at out + r * out_stride
 * floats (out_stride % 4 == 0; feat for rows back to back). */
int gnnagg_plan_spmm_quantized_f32(gnnagg_plan *plan, const float *value, const uint8_t *packed, const float *params,
                                   const int32_t *row_code, float *out, int64_t out_stride, int64_t feat, int bits,
                                   int accumulate, void *stream);
/* The same product with the row codes translated once per matrix: elem_code int64 [nnz], entry e =
 * (row_code[col[e]] << 32) | col[e] in the order of the CSR arrays the plan was made from (the caller builds it once
 * per matrix and code table).  The kernel then asks for a row's bytes as soon as its index chunk has arrived -- two
 * dependent loads per gather instead of three; same result bit for bit. */
int gnnagg_plan_spmm_quantized_elements_f32(gnnagg_plan *plan, const float *value, const uint8_t *packed,
                                            const float *params, const int64_t *elem_code, float *out,
                                            int64_t out_stride, int64_t feat, int bits, int accumulate, void *stream);

/* The pre- and post-aggregation of a 16-bit exchange (communicator.py:111-137) without the two tensor copies around
 * it: gnnagg_plan_spmm_strided_f32 whose dense operand rows and / or result rows are bf16.
 *   mat_is_bf16: row c of the operand is mat + c * mat_stride 16-bit values, widened in the gather (exact), so the
 *                result equals recv_buf.copy_(recv_buf_fp16) followed by the fp32 product, bit for bit
 *                (model/layers/aggregator.py:98-104 behind communicator.py:137);
 *   out_is_bf16: row r of the result is out + r * out_stride 16-bit values, each the fp32 sum rounded to nearest even
 *                (NaN -> 0x7FC0), i.e. what send_buf_fp16.copy_(send_buf) stores behind the fp32 product
 *                (aggregator.py:47-49, communicator.py:128); accumulate must be 0.
 * An operand that is not bf16 is fp32 as everywhere else.  feat and both strides multiples of 4; bf16 rows 8-byte
 * aligned, fp32 rows 16-byte aligned.  Allocates nothing, no host synchronisation. */
int gnnagg_plan_spmm_bf16_f32(gnnagg_plan *plan, const float *value, const void *mat, int mat_is_bf16,
                              int64_t mat_stride, void *out, int out_is_bf16, int64_t out_stride, int64_t feat,
                              int accumulate, void *stream);
int gnnagg_quantize_mixed_f32(const float *x, uint8_t *data, const int64_t *feat_range, float *params, int64_t rows,
                              int64_t feat, int32_t *bad_width, void *stream);
int gnnagg_dequantize_mixed_f32(const uint8_t *data, const int64_t *feat_range, const float *params, float *out,
                                int64_t rows, int64_t feat, int32_t *bad_width, void *stream);

/* bf16 rows on the wire: what `send_buf_fp16.copy_(send_buf)` and `recv_buf.copy_(recv_buf_fp16)` do
 * around the 16-bit exchange (communicator.py:111-137).  fp32 -> bf16 rounds to nearest even (NaN ->
 * 0x7FC0), bf16 -> fp32 is exact.  x, y: `count` contiguous values.  6 bytes moved per value;
 * allocate nothing, no host sync. */
int gnnagg_f32_to_bf16(const float *x, uint16_t *y, int64_t count, void *stream);
int gnnagg_bf16_to_f32(const uint16_t *x, float *y, int64_t count, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GNN_AGG_H */
