/*
 * liteform_hip.h - C ABI of liblfhip.so, the MI355X (gfx950) implementation of
 * LiteForm's CELL/hyb SpMM path:
 *
 *     CSR -> bucket statistics -> bucket-width search -> hyb composition -> fused SpMM
 *
 * The reference (johnpzh/liteform_ae) is Python that reaches the GPU through TVM
 * (playground_pipline/format_algos.py:543-578, 595, 601); it has no FFI of its own.
 * Each entry point below names the reference function whose work it takes over.
 *
 * Conventions
 *   - Every function returns an int status: LF_OK (0) or a negative LF_ERR_* code.
 *     lf_last_error() returns a thread-local, human-readable message for the last
 *     failure on the calling thread.  The library never aborts or exits.
 *   - Pointers named d_* are device pointers (hipMalloc / torch-ROCm storage),
 *     pointers named h_* are host pointers.  The caller allocates and owns all of
 *     them; the library owns only what an lf_spmm_plan holds, released by
 *     lf_spmm_destroy.
 *   - lf_stream_t is a hipStream_t (NULL = the null stream).  Kernels are enqueued on
 *     it; a function synchronises that stream only where it must return host data
 *     (documented per function).
 *   - Index arrays are int32, row-major; values are float32.  A matrix must have
 *     fewer than 2^31 stored entries.
 *   - Handles and workspaces must not be used from two threads at once.
 */
#ifndef LITEFORM_HIP_H
#define LITEFORM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LF_VERSION 110 /* 0.1.1 */

#define LF_OK 0
#define LF_ERR_INVALID (-1)     /* bad argument (null pointer, size, non power-of-two width ...) */
#define LF_ERR_TOO_SMALL (-2)   /* a column partition holds a single nonzero: the reference raises
                                   ValueError("The partition is too small, only having 1 non-zero
                                   element.") at format_algos.py:920-921 */
#define LF_ERR_HIP (-3)         /* a HIP runtime call failed; message carries hipGetErrorString */
#define LF_ERR_CONFIG (-4)      /* width list does not fit the matrix (a partition with nonzeros
                                   has no widths: IndexError at format_algos.py:279) */
#define LF_ERR_UNSUPPORTED (-5) /* outside the implemented range (feature size, nnz >= 2^31 ...) */
#define LF_ERR_WORKSPACE (-6)   /* workspace smaller than lf_*_workspace_bytes() asked for */

#define LF_MAX_CLASSES 11       /* initial widths 1,2,...,1024 (format_algos.py:821 width_limit) */
#define LF_STATS_FIELDS 4       /* per class: cost-model rows, nnz, distinct rows, reserved */

#define LF_DTYPE_F32 0
#define LF_DTYPE_BF16 1

#define LF_COST_REFERENCE 0     /* format_algos.py:1035-1166 bit for bit */
#define LF_COST_GFX950 1        /* measured cost of ELL rows, staged slots and slab bytes on MI355X; same search */

typedef void* lf_stream_t;
typedef struct lf_spmm_plan lf_spmm_plan;

int lf_version(void);
const char* lf_last_error(void);
const char* lf_status_string(int status);

/* ------------------------------------------------------------------------------------
 * Bucket statistics.  Replaces get_init_buckets (format_algos.py:819-900): instead of
 * materialising per-bucket row lists and column sets on the host it returns, per column
 * partition p and initial width class k (width 2^k, capped at width_limit):
 *     h_stats[p][k] = { cost-model rows, nnz, distinct rows, 0 }
 * and a histogram over columns of "which classes touch this column":
 *     h_colhist[p][m] = number of columns of partition p whose class bitmask is m
 * from which the size of the column set of any union of classes follows.
 *
 * d_seg_deg (optional, [num_parts][num_rows] int32) carries per-(partition,row) degrees
 * counted from raw COO triplets as the reference does (format_algos.py:846-849); when
 * NULL the degrees are the CSR segment lengths (identical for duplicate-free input).
 * h_colhist may be NULL: the column sets are then not collected (LF_COST_GFX950 does not
 * read them), which leaves one pass over indptr.
 * Synchronises the stream before returning (host outputs).
 * ------------------------------------------------------------------------------------ */
size_t lf_stats_workspace_bytes(int64_t num_rows, int64_t num_cols, int32_t num_parts);

/* Where lf_bucket_stats left the per-partition row bounds in its workspace:
 * bounds[p][r] = first CSR position of row r whose column is >= p * ceil(num_cols / num_parts),
 * p = 0..num_parts, int32 [num_parts + 1][num_rows].  NULL when num_parts == 1 (the row
 * pointer is the bound).  Valid after lf_bucket_stats ran on that workspace with the same
 * matrix and num_parts; lf_hyb_plan takes it as d_seg_bounds and then skips its own pass of
 * binary searches over the column indices. */
const int32_t* lf_stats_seg_bounds(const void* d_stats_workspace, int64_t num_rows, int32_t num_parts);

int lf_bucket_stats(const int32_t* d_indptr, const int32_t* d_indices, const int32_t* d_seg_deg,
                    int64_t num_rows, int64_t num_cols, int32_t num_parts, int32_t width_limit,
                    void* d_workspace, size_t workspace_bytes,
                    int64_t* h_stats,   /* [num_parts][LF_MAX_CLASSES][LF_STATS_FIELDS] */
                    int64_t* h_colhist, /* [num_parts][1 << LF_MAX_CLASSES] */
                    lf_stream_t stream);

/* Per-(partition,row) degrees from COO triplets (format_algos.py:249-252, 846-849).
 * d_seg_deg [num_parts][num_rows] is cleared and filled on the stream. */
int lf_coo_degrees(const int32_t* d_coo_row, const int32_t* d_coo_col, int64_t nnz,
                   int64_t num_rows, int64_t num_cols, int32_t num_parts,
                   int32_t* d_seg_deg, lf_stream_t stream);

/* Row-length statistics of a CSR matrix, the integer part of MTX.matrix_features
 * (format_matrix_market.py:153-202): h_out = {min, max, sum, sum of squares} of the row
 * lengths indptr[r+1] - indptr[r] (exact integers; mean and standard deviation follow on
 * the host).  num_rows == 0 gives {0, 0, 0, 0}.  d_scratch: 32 bytes of device memory.
 * Synchronises the stream. */
int lf_row_features(const int32_t* d_indptr, int64_t num_rows, void* d_scratch,
                    int64_t* h_out /* [4] */, lf_stream_t stream);

/* The same statistics for callers that cannot allocate or bring device scratch memory along:
 * code recorded into a HIP graph, tight serving loops, harnesses that forbid hipMalloc.  It has
 * no counterpart in the reference.  The four accumulators live in a 32-byte array that is part
 * of the library's device image (every GPU the library runs on holds its own copy until the
 * process ends); the function allocates and frees nothing and does not synchronise: d_out
 * (device memory, int64 [4], 8-byte aligned) receives {min, max, sum, sum of squares} in stream
 * order.  num_rows above LF_ROW_FEATURES_STATIC_MAX_ROWS is refused with LF_ERR_UNSUPPORTED.
 * All calls on one GPU share that GPU's array: calls that overlap there (two streams, two
 * threads) race and must be serialised by the caller.  The first call on a device asks the
 * runtime for the array's address there (hipGetSymbolAddress): make one call outside any
 * stream capture before recording the function into a graph. */
#define LF_ROW_FEATURES_STATIC_MAX_ROWS 2147483646LL
int lf_row_features_static(const int32_t* d_indptr, int64_t num_rows, int64_t* d_out /* [4] */,
                           lf_stream_t stream);

/* ------------------------------------------------------------------------------------
 * Bucket-width search on the host (no GPU work).  Replaces modify_single_row_buckets,
 * get_bucket_config, modify_bucket_widths, move_largest_bucket, move_width_one_bucket and
 * get_memory_cost (format_algos.py:623-648, 709-816, 903-954, 1035-1166), including dict
 * insertion order, the stale key snapshot and the strict-< rule, in IEEE double without
 * contraction.  cfg_feat_size / cfg_num_parts are CostModelSettings' two fields
 * (format_algos.py:45-49).
 *   h_widths  [num_parts][LF_MAX_CLASSES]  ascending widths per partition
 *   h_nwidths [num_parts]                  how many are valid (0 for an empty partition)
 *   h_trace_cost / h_trace_len (optional)  cost of every state the search visited, in
 *                                          visiting order ([num_parts][LF_MAX_CLASSES+1])
 * Returns LF_ERR_TOO_SMALL where the reference raises ValueError.
 * ------------------------------------------------------------------------------------ */
int lf_search_bucket_config(const int64_t* h_stats, const int64_t* h_colhist, int32_t num_parts,
                            int32_t width_limit, int32_t cfg_feat_size, int32_t cfg_num_parts,
                            int32_t cost_model, int32_t* h_widths, int32_t* h_nwidths,
                            double* h_trace_cost, int32_t* h_trace_len);

/* Launch shape without running the kernel: the predicted time in milliseconds of one product
 * with num_parts column partitions (h_stats: their bucket statistics from lf_bucket_stats,
 * [num_parts][LF_MAX_CLASSES][LF_STATS_FIELDS]) and n_windows feature windows
 * (lf_spmm_set_windows), for a matrix whose rows do not share columns (scattered gathers).
 * Stands where the reference predicts num_parts from matrix features with a trained model
 * (proc05.spmm.end-to-end.py:82-97, 142): the caller evaluates the candidates and takes the
 * cheapest.  The model prices the gathers, the read-modify-write of C by later partitions and
 * the slabs against the fabric rate and the scattered-row HBM rate of MI355X, with the share of
 * B that the 256 MB memory-side cache holds.  Host only. */
int lf_model_spmm_ms(const int64_t* h_stats, int32_t num_parts, int32_t n_windows, int64_t num_rows,
                     int64_t num_cols, int32_t feat_size, int32_t b_dtype, double* h_ms);

/* Share of the entries of every sample_stride-th row whose column also occurs in the row
 * before it (the first 64 entries of either row): h_out = {entries in both rows, entries
 * looked at}.  Near 0 for matrices with
 * scattered columns, 0.67 for a 27-point stencil; rows that share columns read B through the
 * L2 and gain nothing from column partitions or feature windows.  d_scratch: 16 bytes of
 * device memory.  Synchronises the stream.  (One of the inputs of the launch-shape choice, as
 * MTX.matrix_features, format_matrix_market.py:153-202, is of the reference's predictor.) */
int lf_row_overlap(const int32_t* d_indptr, const int32_t* d_indices, int64_t num_rows, int64_t sample_stride,
                   void* d_scratch, int64_t* h_out /* [2] */, lf_stream_t stream);

/* ------------------------------------------------------------------------------------
 * hyb composition.  Replaces build_hyb_format (format_algos.py:226-385).
 * Bucket k = (partition p, width index b) in row-major (p, b) order; widths of partition
 * p are h_widths_flat[h_widths_off[p] .. h_widths_off[p+1]), ascending powers of two.
 *
 * lf_hyb_plan counts the ELL rows of every bucket (h_ell_rows[k]) and leaves per-block
 * offsets in the workspace; it synchronises the stream.  lf_hyb_layout (host only) turns
 * those counts into the flat layout: bucket k owns ELL rows [h_row_off[k], +R_k) of
 * d_rows / d_meta and slots [h_slot_off[k], +R_k*W_k) of d_cols / d_vals / d_mask; offsets
 * are padded so that every slab is 256-byte aligned, and h_total_rows / h_total_slots are
 * the element counts to allocate.  The caller then calls lf_hyb_build with the same
 * arguments and workspace.  Bucket contents are exactly the reference's: rows[e] = source
 * row, cols / mask row-major (R, W) padded with (0, 0); vals carries A's values (d_values
 * NULL = all ones, which makes vals == mask).  Padding between slabs is left unwritten.
 *
 * d_meta[e] describes ELL row e for the SpMM kernels: bits 0..10 = valid slots (1..W);
 * bits 11..30 = number of consecutive ELL rows holding the same source row when e is the
 * first of them, or e's index among them on a continuation row; bit 31 set on a
 * continuation row.  It is an acceleration structure, not part of the reference format.
 * ------------------------------------------------------------------------------------ */
size_t lf_hyb_workspace_bytes(int64_t num_rows, int32_t num_parts, int32_t total_buckets);

int lf_hyb_plan(const int32_t* d_indptr, const int32_t* d_indices, const int32_t* d_seg_deg,
                const int32_t* d_seg_bounds,
                int64_t num_rows, int64_t num_cols, int32_t num_parts,
                const int32_t* h_widths_flat, const int32_t* h_widths_off,
                void* d_workspace, size_t workspace_bytes,
                int64_t* h_ell_rows, lf_stream_t stream);

int lf_hyb_layout(const int64_t* h_ell_rows, const int32_t* h_widths_flat, int32_t total_buckets,
                  int64_t* h_row_off, int64_t* h_slot_off, int64_t* h_total_rows, int64_t* h_total_slots);

int lf_hyb_build(const int32_t* d_indptr, const int32_t* d_indices, const float* d_values,
                 const int32_t* d_seg_deg,
                 int64_t num_rows, int64_t num_cols, int32_t num_parts,
                 const int32_t* h_widths_flat, const int32_t* h_widths_off,
                 const int64_t* h_ell_rows,
                 void* d_workspace, size_t workspace_bytes,
                 int32_t* d_rows, int32_t* d_meta, int32_t* d_cols, float* d_vals, float* d_mask,
                 lf_stream_t stream);

/* ------------------------------------------------------------------------------------
 * SpMM  C[num_rows][feat] = A_hyb . B[num_cols][feat].  Replaces the kernel that
 * bench_hyb_with_config builds and launches (format_algos.py:388-605): one launch per
 * column partition (and per feature window, lf_spmm_set_windows) walks every bucket of that
 * partition - "fused" here means the buckets of a partition, not the partitions; rows served
 * with shared gathers and the second stage of very long rows have small launches of their
 * own behind it.  Partitions run in ascending order on the stream, partition 0 stores and
 * later partitions add, so the result does not depend on scheduling and no atomics are used.
 * C needs no clearing.
 *
 * A bucket is described the way the reference passes it to the kernel
 * (format_algos.py:552-578: values float32, rows int32, cols int32 row-major), plus the
 * optional meta array of lf_hyb_build (NULL: derived from rows/vals at create time).
 * The slabs must stay alive and unchanged while the plan exists.
 * At creation every slab is checked on the GPU: a column outside [0, num_cols), a row outside
 * [0, num_rows) or a meta word that does not fit its bucket gives LF_ERR_INVALID, a source row
 * spanning more ELL rows than a meta word can count LF_ERR_UNSUPPORTED (the reference casts the
 * arrays it is given and launches, format_algos.py:568-577).
 * At creation, buckets of 8..64-slot rows whose neighbouring rows hold mostly the same columns
 * (stencils, banded and block-structured matrices) are rewritten inside the plan so that one
 * read of a B row serves several output rows: as groups of four consecutive rows with merged
 * column lists (about 21 bytes per merged entry), or - float32 B, 128 or 256 features per pass - as
 * cells of 16 rows that are neighbours in up to three directions of the underlying grid (the
 * directions are read off the column differences of sampled rows; 69 bytes per merged entry),
 * accumulated with the fp32 outer-product matrix instruction.  This costs plan time and memory
 * only where a sample of the bucket shows at least 30 % fewer reads.
 * Rows that hold at least 1/32 of their partition's columns (and 4096 entries), in a partition
 * whose part of B is larger than 128 MB, are reduced in chunks of 1024 slots that are walked in
 * column order, so that such rows share what the memory-side cache holds of B (LF_DENSE_ROWS=0
 * in the environment at plan creation: chunked like any other long row).
 * feat_size must be a multiple of 32 (float32 B) or 64 (bf16 B), at most 1024.
 * ------------------------------------------------------------------------------------ */
typedef struct lf_bucket_desc {
    int32_t width;          /* W, power of two, 1..1024 */
    int32_t part;           /* column partition this bucket belongs to */
    int64_t num_ell_rows;   /* R */
    const int32_t* d_rows;  /* [R]     */
    const int32_t* d_cols;  /* [R][W]  */
    const float* d_vals;    /* [R][W]  */
    const int32_t* d_meta;  /* [R] or NULL */
} lf_bucket_desc;

int lf_spmm_create(lf_spmm_plan** out_plan, const lf_bucket_desc* h_buckets, int32_t num_buckets,
                   int32_t num_parts, int64_t num_rows, int64_t num_cols, int32_t feat_size,
                   int32_t b_dtype, lf_stream_t stream);
int lf_spmm_run(lf_spmm_plan* plan, const void* d_B, float* d_C, lf_stream_t stream);
int lf_spmm_destroy(lf_spmm_plan* plan);

/* Feature windows.  A plan created for feat_size features can cover operands n_windows times
 * as wide: B [num_cols][n_windows * feat_size], C [num_rows][n_windows * feat_size]; a run then
 * makes one pass per window of feat_size features (all partitions inside), reading and
 * writing only that window's columns.  Features are independent, so the result is that of a
 * plan created for the full width, except that rows split over several ELL rows or reduced
 * cooperatively are summed in pieces whose size follows the lane count (same tolerance, not
 * the same bits).  Narrow
 * windows pay off when B is much larger than the memory-side cache: the part of B that one
 * pass touches is a fraction of the whole, and C is still written once (cfg3, 2.45M rows,
 * N = 128: 6.27 ms in two windows of 64 against 6.94 ms in one pass).  Applies to lf_spmm_run and lf_spmm_time_ms; the default is one window.  No
 * counterpart in the reference (its feature tiling lives inside one launch,
 * format_algos.py:491-520). */
int lf_spmm_set_windows(lf_spmm_plan* plan, int32_t n_windows);

/* h_info[0..LF_SPMM_INFO_FIELDS-1] = tiles, workgroups per launch, launches per run, LDS bytes
 * per workgroup, heavy (split) segments, partial rows, rows cleared by partition 0, buckets
 * served with shared gathers (rows close together holding mostly the same columns), and how
 * many of those are served as 16-row cells on the matrix cores rather than four consecutive
 * rows at a time.  The environment variable LF_ROW_GROUPS at plan creation: 0 turns both
 * paths off, 4 keeps the four-row groups only. */
#define LF_SPMM_INFO_FIELDS 9
int lf_spmm_info(const lf_spmm_plan* plan, int64_t* h_info);

/* Timing helper, the counterpart of the reference's profile_tvm_ms / run_100_times
 * (format_algos.py:164-202, 601): `warmup` untimed runs, then `repeat` runs each bracketed
 * by HIP events on `stream`; before every timed run d_flush (if not NULL) is overwritten
 * to evict the caches, as the reference zeroes a 256 MB buffer.  h_ms receives `repeat`
 * kernel durations in milliseconds (all launches of one run together). Synchronises. */
int lf_spmm_time_ms(lf_spmm_plan* plan, const void* d_B, float* d_C, int32_t warmup,
                    int32_t repeat, void* d_flush, size_t flush_bytes, float* h_ms,
                    lf_stream_t stream);

/* Structural check of CSR arrays that come from outside the library, on the GPU, before
 * anything gathers through them (the reference hands its arrays to the generated kernel
 * unchecked, format_algos.py:1729-1749).  LF_ERR_INVALID when the row pointer does not start at
 * 0, decreases anywhere or does not end at nnz, or when a column index lies outside
 * [0, num_cols).  *h_flags (optional) receives LF_CSR_CANONICAL when in addition the columns of
 * every row ascend strictly (sorted, no duplicates) - the form scipy's coo.tocsr() produces
 * (format_matrix_market.py:74-76) and lf_bucket_stats / lf_hyb_build expect, so that such
 * arrays can be used as they are instead of going through lf_coo_to_csr - and
 * LF_CSR_UNIT_VALUES when d_values (optional) holds nothing but 1.0, like every matrix of the
 * reference (format_matrix_market.py:54, 63-64).  The block structure of a BSR matrix is
 * checked the same way (rows and columns counted in blocks).  d_scratch: 16 bytes of device
 * memory.  Synchronises the stream. */
#define LF_CSR_CANONICAL 1
#define LF_CSR_UNIT_VALUES 2
int lf_csr_check(const int32_t* d_indptr, const int32_t* d_indices, const float* d_values,
                 int64_t num_rows, int64_t num_cols, int64_t nnz, void* d_scratch, int32_t* h_flags,
                 lf_stream_t stream);

/* Row-parallel CSR SpMM, the counterpart of bench_naive's kernel
 * (format_algos.py:1689-1755): C = A_csr . B with float32 values (NULL = ones).
 * lf_csr_spmm runs lf_csr_check on the arrays first (d_scratch: its 16 bytes; the stream is
 * synchronised for the verdict) and returns LF_ERR_INVALID without launching the product when
 * they fail.  lf_csr_spmm_trusted is the same product without the check, for arrays that
 * lf_csr_check has accepted or that lf_coo_to_csr produced: it only enqueues the kernel. */
int lf_csr_spmm(const int32_t* d_indptr, const int32_t* d_indices, const float* d_values,
                int64_t num_rows, int64_t num_cols, int64_t nnz, int32_t feat_size, int32_t b_dtype,
                const void* d_B, float* d_C, void* d_scratch, lf_stream_t stream);
int lf_csr_spmm_trusted(const int32_t* d_indptr, const int32_t* d_indices, const float* d_values,
                        int64_t num_rows, int64_t num_cols, int32_t feat_size, int32_t b_dtype,
                        const void* d_B, float* d_C, lf_stream_t stream);

/* COO -> canonical CSR on the GPU: entries sorted by (row, column), duplicates added up,
 * row pointer built - what the reference's container does with scipy's coo.tocsr() on every
 * CSR request (format_matrix_market.py:74-76).  d_coo_val NULL = all ones (the reference's
 * matrices, format_matrix_market.py:54, 63-64).  Outputs: d_indptr [num_rows + 1], d_indices
 * and d_values with room for nnz entries; *h_nnz_out = entries left after merging duplicates.
 * Synchronises the stream. */
size_t lf_coo_to_csr_workspace_bytes(int64_t nnz, int64_t num_rows, int64_t num_cols);
int lf_coo_to_csr(const int32_t* d_coo_row, const int32_t* d_coo_col, const float* d_coo_val, int64_t nnz,
                  int64_t num_rows, int64_t num_cols, void* d_workspace, size_t workspace_bytes,
                  int32_t* d_indptr, int32_t* d_indices, float* d_values, int64_t* h_nnz_out,
                  lf_stream_t stream);

/* Block-sparse SpMM on the matrix cores, the counterpart of bench_bsrmm's kernel
 * (format_algos.py:1182-1643): Y = A_bsr . X with square fp16 blocks of block_size = 16, 32 or
 * 64 rows (scipy BSR layout: indptr [num_block_rows + 1], indices [nnz blocks], data
 * [nnz blocks][block_size][block_size] row-major), X [num_block_cols * block_size][feat] fp16,
 * Y [num_block_rows * block_size][feat] fp16, fp32 accumulation (the reference accumulates in
 * fp16).  The reference's schedule takes any multiple of 16 (format_algos.py:1581-1582) and its
 * driver passes 32 (proc05.spmm.end-to-end.py:205); here the sizes are those whose block rows
 * fill whole 16- or 32-row matrix-instruction tiles with one tile shape (48, 80, ... would mix
 * the two): others return LF_ERR_UNSUPPORTED.  feat_size must be a multiple of 8; X, Y and the
 * block data 16-byte aligned.
 * lf_bsr_spmm checks the block index arrays like lf_csr_check (d_scratch: 16 bytes of device
 * memory; synchronises for the verdict) and returns LF_ERR_INVALID without launching the
 * product when they fail; lf_bsr_spmm_trusted only enqueues the kernel, for arrays that have
 * passed the check before. */
int lf_bsr_spmm(const int32_t* d_indptr, const int32_t* d_indices, const void* d_data,
                int64_t num_block_rows, int64_t num_block_cols, int64_t nnz_blocks, int32_t block_size,
                int32_t feat_size, const void* d_X, void* d_Y, void* d_scratch, lf_stream_t stream);
int lf_bsr_spmm_trusted(const int32_t* d_indptr, const int32_t* d_indices, const void* d_data,
                        int64_t num_block_rows, int64_t num_block_cols, int32_t block_size,
                        int32_t feat_size, const void* d_X, void* d_Y, lf_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LITEFORM_HIP_H */
