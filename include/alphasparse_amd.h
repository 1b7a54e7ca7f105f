/*
 * C-ABI of the MI355X (gfx950) CSR SpMV / SpMM path.
 *
 * Plain pointers and sizes only.  Every `d_*` pointer is device memory owned by the
 * caller; `stream` is a hipStream_t passed as void* (NULL = the default stream).  All
 * entry points return an alphasparseStatus_t value (0 = success) and launch
 * asynchronously on `stream` unless stated otherwise.  Indices are int32, zero based.
 *
 * The C++ entry points of the generic API (alphasparseSpMV, alphasparseSpMM and
 * friends, declared in alphasparse.h next to this file) are thin host wrappers over
 * the functions below and live in the same shared library.
 *
 * Each declaration cites the reference interface it stands in for
 * (paths relative to the AlphaSparse source tree).
 */
#ifndef ALPHASPARSE_AMD_H
#define ALPHASPARSE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes: include/alphasparse/spdef.h:10-22 */
enum {
    ASX_STATUS_SUCCESS = 0,
    ASX_STATUS_NOT_INITIALIZED = 1,
    ASX_STATUS_ALLOC_FAILED = 2,
    ASX_STATUS_INVALID_VALUE = 3,
    ASX_STATUS_EXECUTION_FAILED = 4,
    ASX_STATUS_INTERNAL_ERROR = 5,
    ASX_STATUS_NOT_SUPPORTED = 6,
    ASX_STATUS_INVALID_POINTER = 7,
    ASX_STATUS_INVALID_HANDLE = 8,
    ASX_STATUS_INVALID_KERNEL_PARAM = 9,
    ASX_STATUS_INVALID_SIZE = 10
};

/* value types: include/alphasparse/spdef.h:144-155 (ALPHA_R_32F = 0, ALPHA_R_64F = 1) */
enum { ASX_R_32F = 0, ASX_R_64F = 1 };

/* SpMV kernels.  Numeric values of the first group are alphasparseSpMVAlg_t values
 * (include/alphasparse/spdef.h:345-365); how each reference algorithm id maps onto these
 * kernels is decided by asx_spmv_resolve_alg. */
enum {
    ASX_SPMV_DEFAULT = 0, /* pick from the row-length histogram (plan) or from m, nnz */
    ASX_SPMV_VECTOR = 6,  /* wave64 sub-groups, one group per row */
    ASX_SPMV_STREAM = 3,  /* LDS-staged row blocks, segmented reduction */
    ASX_SPMV_MERGE = 9,   /* merge-path tiles + ordered carry fix-up */
    ASX_SPMV_FLAT = 15,   /* tiles of 1024 stored elements, register walk + ordered carry fix-up */
    ASX_SPMV_SLICED = 101, /* not a reference id: stored elements regrouped by column slice, each slice of x
                             held in LDS; one partial sum per (row, slice), added per row by a second pass
                             (needs a plan from asx_spmv_plan_create; NOT_SUPPORTED beyond 1024 slices of
                             128 KiB of x: 16.7 M columns in fp64, 33.5 M in fp32) */
    ASX_SPMV_WINDOW = 102 /* not a reference id: chains of blocks of consecutive rows with a sliding window of x
                             in LDS and 16-bit columns, for matrices whose rows reach only nearby columns
                             (needs a plan from asx_spmv_plan_create; NOT_SUPPORTED when some 256 rows reach
                             over 16376 columns or more) */
};

/* SpMM kernels (alphasparseSpMMAlg_t values, include/alphasparse/spdef.h:390-402) */
enum {
    ASX_SPMM_DEFAULT = 0,
    ASX_SPMM_ROW = 5,    /* CSR_ALG1: one wave per (row, 64-column tile) */
    ASX_SPMM_MERGE = 7,  /* CSR_ALG3: merge-path segments per wave + ordered carry fix-up */
    ASX_SPMM_BLOCKED = 10 /* CSR_ALG6: 16x4-blocked MFMA variant (needs asx_spmm_plan_create) */
};

/* ------------------------------------------------------------------------------------
 * Library / device
 * ---------------------------------------------------------------------------------- */

/* Version string "major.minor". */
const char *asx_version(void);
/* Number of compute units and wavefront size of the current device (host query).
 * Stands in for the device query in alphasparseGetHandle, hip/util/handle.hip:67-83. */
int asx_device_info(int *compute_units, int *wavefront_size);

/* ------------------------------------------------------------------------------------
 * CSR analysis: integer outputs, bit-identical to the reference functions cited.
 * ---------------------------------------------------------------------------------- */

/* Row-length histogram.  d_hist[b], b in [0,32]: b = 0 counts empty rows, b >= 1 counts rows
 * with 2^(b-1) <= len < 2^b.  d_stats[0] = max row length, [1] = rows with len < 2,
 * [2] = rows with 2 <= len < 1024, [3] = rows with len >= 1024 (the three bins of find_rows,
 * hip/kernel/level2/alphasparse_spmv_csr_adaptive2.h:5-47).  d_hist: 33 x int64,
 * d_stats: 4 x int64; both are overwritten. */
int asx_row_length_histogram(const int32_t *d_row_ptr, int32_t m, int64_t *d_hist, int64_t *d_stats,
                             void *stream);

/* balanced_partition_row_by_nnz, hygon/util/partition.cpp:83-96 (device twins:
 * dcu/kernel/level2/csrmv/dcu_gemv_row_partition.h:10-40).  d_partition: nparts+1 int32. */
int asx_partition_rows_by_nnz(const int32_t *d_row_ptr, int32_t m, int32_t nparts, int32_t *d_partition,
                              void *stream);

/* Row holding stored element t*items, t in [0, ceil(nnz/items)); out[ceil(nnz/items)] = m.
 * elebalance_partition_kernel, hip/kernel/level3/alphasparse_spmm_csr_nnz_split.h:7-47;
 * adaptive_partition_kernel, hip/kernel/level3/alphasparse_spmm_csr_adaptive.h:7-43;
 * flat_partition_kernel, hip/kernel/level3/alphasparse_spmm_csr_flat.h:6-25;
 * balanced_partition_row_by_nnz_flat (items = 1024),
 * hip/kernel/level2/alphasparse_spmv_csr_flat.h:7-38. */
int asx_nnz_split_rows(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t items, int32_t *d_out,
                       void *stream);

/* Merge-path split points on diagonals g*items, g in [0, ceil((m+nnz)/items)]:
 * d_xs[g] rows consumed, d_ys[g] stored elements consumed.
 * abstract_merge_path_search, hip/kernel/level2/alphasparse_spmv_csr_merge_ginkgo.h:10-33,132-157
 * (items = 4096); merge_path_search_kernel,
 * hip/kernel/level3/alphasparse_spmm_csr_merge.h:6-30,32-75. */
int asx_merge_path_search(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t items, int32_t *d_xs,
                          int32_t *d_ys, void *stream);

/* clac_size, hip/kernel/level2/alphasparse_spmv_csr_row_partition_ginkgo.h:93-122 (host). */
int64_t asx_loadbalance_nwarps(int64_t nnz, int64_t warp_size, int64_t nwarps_base);
/* balanced_partition_row_by_nnz<T,warp_size>,
 * hip/kernel/level2/alphasparse_spmv_csr_row_partition_ginkgo.h:15-42 as launched at :419-424.
 * d_out: nwarps int32. */
int asx_loadbalance_partition(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t warp_size,
                              int32_t nwarps, int32_t *d_out, void *stream);

/* ComputeRowBlocks, hip/kernel/level2/alphasparse_spmv_csr_adaptive.h:354-568.  HOST routine on a
 * HOST row_ptr, as in the reference.  Writes up to cap packed entries, returns through *count the
 * number of entries the full result has (call with cap = 0 to size the array). */
int asx_csr_adaptive_row_blocks(const int32_t *h_row_ptr, int32_t m, uint64_t *h_out, size_t cap,
                                size_t *count);

/* COO -> CSR row offsets from row indices sorted ascending: d_row_ptr[r] = first i with
 * d_row_ind[i] >= r, r in [0, m].  alphasparseXcoo2csr, hip/format/coo2csr.h:7-16 (which
 * forwards to hipsparseXcoo2csr). */
int asx_coo2csr(const int32_t *d_row_ind, int32_t nnz, int32_t m, int32_t *d_row_ptr, void *stream);
/* Sorts device COO triplets by (row, column) in place (stable for equal keys).  Device twin of
 * the host qsort in coo_order, hip/format/coo_order.h:24-43.  Allocates temporaries and
 * synchronises `stream`. */
int asx_coo_sort(int value_type, int32_t *d_row_ind, int32_t *d_col_ind, void *d_val, int32_t nnz,
                 void *stream);

/* A (m x n, CSR, idx_base 0 or 1) -> A^T (n x m) as zero-based CSR; the stored elements of each
 * row of A^T come in ascending row of A, duplicates in their stored order.  What
 * opA = TRANSPOSE runs on; device twin of transpose_csr, hip/format/transpose_csr.h:9-71 (host
 * counting sort between two copies across PCIe, result written over the caller's arrays).
 * d_row_ptr_t has n+1 entries, d_col_t and d_val_t nnz.  Allocates temporaries and synchronises
 * `stream`. */
int asx_csr_transpose(int value_type, int32_t m, int32_t n, int32_t nnz, int32_t idx_base,
                      const int32_t *d_row_ptr, const int32_t *d_col, const void *d_val,
                      int32_t *d_row_ptr_t, int32_t *d_col_t, void *d_val_t, void *stream);
/* Zero-based copies of one-based (idx_base = 1) row offsets and column indices.  The reference
 * stores idx_base in the descriptor (hip/format/alphasparse_create_csr.h:44-47) and its CSR
 * kernels index with the stored values unchanged. */
int asx_csr_rebase(int32_t m, int32_t nnz, int32_t idx_base, const int32_t *d_row_ptr, const int32_t *d_col,
                   int32_t *d_row_ptr_out, int32_t *d_col_out, void *stream);
/* d_out[c*ld_out + r] = d_in[r*ld_in + c] for r < rows, c < cols: row-major <-> column-major
 * copies of the dense operands of SpMM.  transpose_dn_mat, hip/format/transpose_dn_mat.h:4-35. */
int asx_dense_transpose(int value_type, int64_t rows, int64_t cols, const void *d_in, int64_t ld_in,
                        void *d_out, int64_t ld_out, void *stream);

/* Reads a MatrixMarket coordinate file into HOST COO arrays (zero-based, file order; symmetric,
 * Hermitian and skew-symmetric files expanded by following every off-diagonal entry with its
 * mirror image carrying the same value; pattern entries are 1; the real part of complex entries).
 * alpha_read_coo, hip/test/io.hip:100-330.  The arrays are malloc'ed: release with
 * asx_host_free.  value_type selects float or double values. */
int asx_mtx_read(const char *path, int value_type, int32_t *m, int32_t *n, int32_t *nnz, int32_t **h_row,
                 int32_t **h_col, void **h_val);
void asx_host_free(void *p);

/* ------------------------------------------------------------------------------------
 * Plans: analysis results kept across calls (the reference recomputes them inside every
 * SpMV/SpMM call; its alphasparseSpMV_analysis is a stub, hip/kernel/level2/alphasparse_spmv.hip:
 * 229-247, and _alphasparse_csrmv_info, include/alphasparse/handle.h:147-198, is never filled).
 * A plan owns device memory (allocated at creation, freed at destruction) and is bound to the
 * sparsity pattern it was built from.
 * ---------------------------------------------------------------------------------- */
typedef struct asx_plan asx_plan;

/* Builds a plan for SpMV (ncols_dense = 1) or SpMM (ncols_dense = N > 1).  `alg` is one of
 * the ASX_SPMV_* / ASX_SPMM_* values; DEFAULT reads the row-length histogram back (one small
 * synchronous copy) and picks a kernel.  Synchronises `stream` before returning. */
int asx_plan_create(asx_plan **plan, int is_spmm, int alg, int value_type, int32_t m, int32_t n,
                    int32_t nnz, const int32_t *d_row_ptr, int32_t ncols_dense, void *stream);
/* SpMM plan that may look at A's columns and values.  alg = ASX_SPMM_BLOCKED re-tiles A into
 * zero-filled 16x4 blocks for the MFMA kernel (tc_preprocess,
 * hip/kernel/level3/alphasparse_spmm_tc4csr.h:38-153; the plan then holds a COPY of the values:
 * asx_plan_update_values after changing them; repeated (row, column) entries are summed; B must
 * be finite, see below).  alg = ASX_SPMM_DEFAULT measures the block fill nnz / (64 * blocks) and
 * picks the blocked kernel when it is at least 1/8, else the merge kernel.  Other algorithms
 * behave as asx_plan_create.  Synchronises `stream`. */
int asx_spmm_plan_create(asx_plan **plan, int alg, int value_type, int32_t m, int32_t k, int32_t nnz,
                         const int32_t *d_row_ptr, const int32_t *d_col, const void *d_val, int32_t ncols,
                         void *stream);
/* SpMV plan that may look at A's columns and values.  alg = ASX_SPMV_SLICED regroups the stored
 * elements by column slice (128 KiB of x per slice) for the kernel that holds its slice of x in
 * LDS.  The plan then holds a COPY of the columns and values (asx_plan_update_values after
 * changing the values) and the buffer for the partial sums of a call: calls through one plan
 * must not overlap.  alg = ASX_SPMV_DEFAULT picks that kernel when nnz >= 2^21, the columns are
 * scattered (a sample of 64 tiles of 1024 stored elements touches on average more than 512
 * distinct 128-byte lines of x per tile) and a cost model over the row-length histogram and the
 * sizes puts it at least 10 % ahead of the row-ordered kernels; the choice depends on the matrix
 * alone, not on timings.  Otherwise as asx_plan_create.  No counterpart in the reference (its
 * alphasparseSpMV_analysis is a stub).  alg = ASX_SPMV_WINDOW builds the row-block copy for the
 * kernel that keeps sliding windows of x in LDS (again a COPY of columns and values, and the
 * carry slots of a call; a matrix without rows of fewer than two stored elements needs no copy of
 * the values: an fp32 plan, or a plan made by asx_spmv_plan_create_checked, then reads A's values
 * in every call, ASX_PLAN_INFO_BY_REFERENCE = 1, and holds 2 bytes per stored element instead of
 * 14 or 10); DEFAULT picks it, when the sliced kernel is not chosen, for nnz >= 2^21
 * whenever the matrix qualifies: every 256 consecutive rows reach
 * over fewer than 16376 columns, or the stored elements lie on at most 4 bands of diagonals whose
 * windows fit the LDS together (stencils on three-dimensional grids); otherwise
 * ASX_STATUS_NOT_SUPPORTED for the explicit id, the row-ordered plan for DEFAULT.  Synchronises
 * `stream`. */
int asx_spmv_plan_create(asx_plan **plan, int alg, int value_type, int32_t m, int32_t n, int32_t nnz,
                         const int32_t *d_row_ptr, const int32_t *d_col, const void *d_val, void *stream);
/* Brings a plan that holds a copy of A's values (ASX_SPMV_SLICED, ASX_SPMV_WINDOW, ASX_SPMM_BLOCKED) up to date
 * with d_val (same sparsity pattern as when the plan was built); asynchronous on `stream`; one
 * pass over the values (sliced: 156 us for 34 M fp64 values, 38 us for 16.8 M fp32 ones).  For
 * the other kernels, which read the caller's values in every call, it does nothing.
 * asx_plan_holds_values tells the two kinds apart.  No counterpart in the reference. */
int asx_plan_update_values(asx_plan *plan, const void *d_val, void *stream);
int asx_plan_holds_values(const asx_plan *plan);
/* For callers who may change A's values in place without saying so (the reference's own callers:
 * its alphasparseSpMV reads A's arrays in every call, hip/kernel/level2/alphasparse_spmv.hip:16-199,
 * and its analysis keeps nothing).  asx_spmv_plan_create_checked is asx_spmv_plan_create, except
 * that a plan which ends up holding a copy of the values also keeps two 64-bit checksums of
 * them (position-dependent sums over their 32-bit words; a single changed word always changes
 * them, several changes escape with probability 2^-128) and that DEFAULT's choice counts what
 * checking costs.  d_val must lie on a 16-byte boundary for such a plan (otherwise DEFAULT makes
 * the plan row-ordered, and ASX_SPMV_SLICED / ASX_SPMV_WINDOW return ASX_STATUS_INVALID_VALUE).  A
 * window plan over a matrix without rows of fewer than two stored elements keeps no copy of the
 * values at all and so needs neither checksums nor refreshes (fp64: 5-point stencil on 4096^2,
 * 210 us a multiply in place, 201 from a copy that the caller keeps up to date, 285 from a checked
 * copy).  asx_plan_refresh_if_changed, called before every SpMV through the plan with the
 * values as they are now, takes their checksums (one read of the values: 42 us for 34 M fp64
 * values) and brings the copy up to date where they differ from the kept ones; all on the device,
 * asynchronous on `stream`, nothing is read back.  It does nothing for a plan that was made
 * unchecked or that reads the caller's values anyway (asx_plan_is_checked = 0).  The sparsity
 * pattern is taken to stay as it was.  Calls through one checked plan on several streams at once
 * may refresh the copy more often than needed (they share the checksum words); results stay
 * right.  No counterpart in the reference. */
int asx_spmv_plan_create_checked(asx_plan **plan, int alg, int value_type, int32_t m, int32_t n, int32_t nnz,
                                 const int32_t *d_row_ptr, const int32_t *d_col, const void *d_val, void *stream);
int asx_plan_refresh_if_changed(asx_plan *plan, const void *d_val, void *stream);
int asx_plan_is_checked(const asx_plan *plan);
/* Number of 16x4 blocks and their fill of a blocked plan. */
int asx_plan_block_stats(const asx_plan *plan, int64_t *nblocks, double *fill);
int asx_plan_destroy(asx_plan *plan);
/* Short name of a kernel id (ASX_SPMV_* / ASX_SPMM_* value): "vector", "stream", "merge", "flat",
 * "sliced", "window"; "row", "merge", "blocked"; "?" for anything else. */
const char *asx_kernel_name(int is_spmm, int kernel);
/* Kernel the plan resolved to, and bytes of per-call workspace its launches need (carries; for a
 * sliced plan the partial sums of a call, for a window plan with cut rows its carries).  A sliced
 * or window plan also keeps a buffer of that size of its own, used by calls whose workspace is
 * NULL or smaller: such calls share it and must not overlap, while calls that each bring a
 * workspace of this size may run at the same time on different streams (the plan itself is only
 * read). */
int asx_plan_alg(const asx_plan *plan);
size_t asx_plan_workspace_bytes(const asx_plan *plan);
/* What a plan that holds a regrouped copy of A looks like (for logs and tests; -1 where the
 * figure does not apply to the plan's kernel).  No counterpart in the reference. */
enum {
    ASX_PLAN_INFO_TILES = 0,          /* tiles of 256 slots (sliced, window) */
    ASX_PLAN_INFO_SLICES = 1,         /* column slices (sliced) */
    ASX_PLAN_INFO_PARTIAL_SUMS = 2,   /* partial sums per call (sliced) */
    ASX_PLAN_INFO_ROWS_PER_WAVE = 3,  /* rows of a row block of pass 2 (sliced) */
    ASX_PLAN_INFO_ROWS_PER_BLOCK = 4, /* rows of a block (window) */
    ASX_PLAN_INFO_BANDS = 5,          /* rings of x in LDS: 1 = one window, 2..4 = bands of diagonals (window) */
    ASX_PLAN_INFO_CHAINS = 6,         /* chains of blocks = workgroups (window) */
    ASX_PLAN_INFO_CARRY_PASS = 7,     /* 1 if a call runs the ordered carry pass (window) */
    ASX_PLAN_INFO_ROW_BLOCKS = 8,     /* row blocks of pass 2 (sliced), blocks of rows (window) */
    ASX_PLAN_INFO_STEPS = 9,          /* steps of pass 2, each up to 64 partial sums (sliced) */
    ASX_PLAN_INFO_WIDTH = 10,         /* columns per slice (sliced), columns the rings hold together (window) */
    ASX_PLAN_INFO_WORKGROUPS = 11,    /* workgroups of pass 1 (sliced), chains (window) */
    ASX_PLAN_INFO_PIECES = 12,        /* pieces of x fetched over all blocks (window) */
    ASX_PLAN_INFO_STACKED_ROWS = 13,  /* rows of a plane when the three bands share rotating regions of LDS and the
                                         blocks are stored plane above plane (window; 0 otherwise) */
    ASX_PLAN_INFO_BY_REFERENCE = 14   /* 1 when the plan keeps no copy of A's values (window: no row of A holds fewer than two
                                         stored elements, so the stored elements of a tile are consecutive in A's val, which
                                         every call reads in place; asx_plan_holds_values is 0 then) */
};
int64_t asx_plan_info(const asx_plan *plan, int what);
/* Frees the buffer a sliced or window plan keeps for the partial sums / carries of a call.  Calls
 * through the plan then need a workspace of asx_plan_workspace_bytes(plan) bytes (without one they
 * return ASX_STATUS_INVALID_POINTER); for callers who always bring their own buffer and want the
 * memory back.  The plan must not be in use by a call that is still running.  No counterpart in
 * the reference. */
int asx_plan_release_scratch(asx_plan *plan);
/* Bytes of the buffer the plan itself keeps for that purpose (0: none, or released). */
size_t asx_plan_own_scratch_bytes(const asx_plan *plan);
/* Copies one array of a plan that holds a regrouped copy of A to the host (for tests that check a
 * built plan on the host, and for debugging; synchronises `stream`).  `*bytes` receives the
 * array's size; with h_dst == NULL nothing is copied (sizing call), else `cap` must be at least
 * that.  ASX_STATUS_INVALID_VALUE when the plan's kernel has no such array.  No counterpart in the
 * reference. */
enum {
    ASX_PLAN_ARRAY_VAL = 0,          /* slots x value: the regrouped values, in the order the loads deliver them
                                      * (with PERM: absent, ASX_STATUS_INVALID_VALUE, in a plan that reads A's values in place) */
    ASX_PLAN_ARRAY_CF = 1,           /* slots x u16: local column | first-of-run << 15 */
    ASX_PLAN_ARRAY_PERM = 2,         /* slots x i32: position in A's values of each stored copy (-1: pad) */
    ASX_PLAN_ARRAY_TILE_WORDS = 3,   /* sliced: (tiles + 1) x i32 first partial sum of each tile; window: tiles x 4 i32
                                      * (first row | starts-inside-a-row << 31, rows, first stored element in A, stored elements) */
    ASX_PLAN_ARRAY_WORKGROUPS = 4,   /* sliced: pieces x 4 i32 (slice, first tile, end tile, 0): what the workgroups of pass 1
                                      * work off; window: chains x 2 i32 */
    ASX_PLAN_ARRAY_PARTIAL_ROWS = 5, /* sliced: partial sums x u16 row inside the row block | may-repeat << 15 */
    ASX_PLAN_ARRAY_RANGES = 6,       /* sliced: (row blocks + 1) x slices i32: first partial sum of block b in slice s */
    ASX_PLAN_ARRAY_STEP_PTR = 7,     /* sliced: (row blocks + 1) x i32: first step of each row block */
    ASX_PLAN_ARRAY_STEPS = 8,        /* sliced: steps x 4 i32 */
    ASX_PLAN_ARRAY_BLOCKS = 9,       /* window: blocks x 4 i32 (first tile, end tile, first piece, end piece) */
    ASX_PLAN_ARRAY_PIECES = 10,      /* window: pieces x 4 i32 (from column, to column, ring base, ring size) */
    ASX_PLAN_ARRAY_WG_PIECES = 11    /* sliced: workgroups x 8 i32 (first, end entry of ASX_PLAN_ARRAY_WORKGROUPS, 0, 0,
                                      * the first of those entries again) */
};
int asx_plan_export(const asx_plan *plan, int what, void *h_dst, size_t cap, size_t *bytes, void *stream);
/* Copies the plan's histogram (33 bins) and stats (4) to host arrays. */
int asx_plan_histogram(const asx_plan *plan, int64_t h_hist[33], int64_t h_stats[4]);

/* ------------------------------------------------------------------------------------
 * SpMV  y = alpha*A*x + beta*y      (alphasparseSpMV, include/alphasparse/spapi.h:6895-6905;
 *                                    CPU twin alphasparse_?_mv, spapi.h:1000-1020)
 * ---------------------------------------------------------------------------------- */

/* Kernel an alphasparseSpMVAlg_t value runs as when no plan is given. */
int asx_spmv_resolve_alg(int alg, int32_t m, int32_t nnz);
/* Workspace bytes for a plan-less call (analysis metadata + carries).
 * alphasparseSpMV_bufferSize, hip/kernel/level2/alphasparse_spmv.hip:258-338. */
size_t asx_spmv_workspace_bytes(int alg, int value_type, int32_t m, int32_t nnz);

/* With plan != NULL the kernel and its split points come from the plan and d_workspace only
 * holds carries (asx_plan_workspace_bytes).  With plan == NULL the split points are computed
 * into d_workspace by this call (asx_spmv_workspace_bytes), as the reference does on every
 * call.  beta == 0 never reads y. */
int asx_spmv_csr_f64(const asx_plan *plan, int alg, int32_t m, int32_t n, int32_t nnz, double alpha,
                     const int32_t *d_row_ptr, const int32_t *d_col, const double *d_val,
                     const double *d_x, double beta, double *d_y, void *d_workspace,
                     size_t workspace_bytes, void *stream);
int asx_spmv_csr_f32(const asx_plan *plan, int alg, int32_t m, int32_t n, int32_t nnz, float alpha,
                     const int32_t *d_row_ptr, const int32_t *d_col, const float *d_val,
                     const float *d_x, float beta, float *d_y, void *d_workspace,
                     size_t workspace_bytes, void *stream);

/* asx_spmv_csr_f64 without a plan and without a workspace argument, for callers that cannot
 * allocate device memory and have no buffer to pass (code under HIP graph capture, serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  The split points and
 * carries that asx_spmv_csr_f64 puts into the caller's workspace live in an array inside the
 * library, one copy per GPU, asx_spmv_noalloc_max_workspace() bytes (4 MiB) large: a call whose
 * asx_spmv_workspace_bytes(alg, ASX_R_64F, m, nnz) exceeds that returns ASX_STATUS_INVALID_SIZE
 * and launches nothing (sized for the kernel the call runs; the flat kernel, alg 0, needs 12 bytes
 * per 1024 stored elements: about 350 million stored elements fit).  The call allocates nothing and frees nothing.  Every call on
 * a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two threads)
 * race; calls on one stream are safe.  Same kernels, same results as asx_spmv_csr_f64 with the
 * same `alg`.  The array's device address is looked up once per device, by asx_device_info or by
 * the first call on that device (a host-side lookup that may load the library's code): before
 * capturing a call into a HIP graph, call asx_device_info or make one call eagerly. */
int asx_spmv_csr_f64_noalloc(int alg, int32_t m, int32_t n, int32_t nnz, double alpha,
                             const int32_t *d_row_ptr, const int32_t *d_col, const double *d_val,
                             const double *d_x, double beta, double *d_y, void *stream);
size_t asx_spmv_noalloc_max_workspace(void);

/* ------------------------------------------------------------------------------------
 * SpMM  C = alpha*A*B + beta*C, B (k x ncols) and C (m x ncols) row-major
 *       (alphasparseSpMM, include/alphasparse/spapi.h:6963-6974; CPU twin alphasparse_?_mm,
 *        spapi.h:1272-1306)
 * ---------------------------------------------------------------------------------- */
int asx_spmm_resolve_alg(int alg, int32_t m, int32_t nnz, int32_t ncols);
/* alphasparseSpMM_bufferSize, hip/kernel/level3/alphasparse_spmm.hip:699-850. */
size_t asx_spmm_workspace_bytes(int alg, int value_type, int32_t m, int32_t nnz, int32_t ncols);

int asx_spmm_csr_f32(const asx_plan *plan, int alg, int32_t m, int32_t k, int32_t nnz, int32_t ncols,
                     float alpha, const int32_t *d_row_ptr, const int32_t *d_col, const float *d_val,
                     const float *d_B, int64_t ldb, float beta, float *d_C, int64_t ldc,
                     void *d_workspace, size_t workspace_bytes, void *stream);
int asx_spmm_csr_f64(const asx_plan *plan, int alg, int32_t m, int32_t k, int32_t nnz, int32_t ncols,
                     double alpha, const int32_t *d_row_ptr, const int32_t *d_col, const double *d_val,
                     const double *d_B, int64_t ldb, double beta, double *d_C, int64_t ldc,
                     void *d_workspace, size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif
