/*
 * CPU oracle for the CSR SpMV / SpMM hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * Nothing in the shipped library links, loads or calls this file.  It restates,
 * in plain C, the arithmetic and the integer analysis outputs of the reference
 * (AlphaSparse) so that GPU results can be checked against them.  Every
 * function names the reference file:line it follows.
 *
 * Pinning status (what independently checks each function):
 *   orc_partition_rows_by_nnz   bit-exact vs the compiled reference (oracle/_ref) + brute force
 *   orc_spmv_csr_f64 / _f32     bit-exact vs the compiled reference x86 asm kernels (oracle/_ref),
 *                               golden fixtures, exact-integer inputs, closed forms
 *   orc_spmm_csr_row_f32/_f64   bit-exact vs the compiled reference (oracle/_ref), column-wise
 *                               equivalence with SpMV, golden fixtures
 *   orc_nnz_split_rows          brute force (row containing element t*I)
 *   orc_merge_path_search       brute force of the merge-path predicate + invariants
 *   orc_loadbalance_*           brute force of the predicate; clac thresholds by table
 *   orc_find_rows_counts        brute force
 *   orc_csr_adaptive_row_blocks bit-exact vs the reference's host routine compiled from its header
 *                               (oracle/_ref) + golden fixtures
 *   orc_coo2csr                 numpy searchsorted / bincount (the reference forwards to hipSPARSE)
 */
#ifndef ALPHASPARSE_ORACLE_H
#define ALPHASPARSE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* hygon/util/partition.cpp:83-96 (balanced_partition_row_by_nnz) with
 * hygon/util/partition.cpp:50-65 (lower_bound_int).  row_end = row_ptr + 1. */
void orc_partition_rows_by_nnz(const int32_t *row_end, int32_t rows, int32_t nthreads,
                               int32_t *partition /* nthreads+1 */);

/* hygon/kernel/level2/mv/gemv/gemv_csr.hpp:48-78 +
 * hygon/kernel/level2/mv/gemv/csrmv/gemv_csr_serial_fma_fp64_u4.S:70-151. */
void orc_spmv_csr_f64(int32_t m, const int32_t *row_ptr, const int32_t *col, const double *val,
                      const double *x, double alpha, double beta, double *y, int nthreads);

/* hygon/kernel/level2/mv/gemv/gemv_csr.hpp:14-46 +
 * hygon/kernel/level2/mv/gemv/csrmv/gemv_sload_shuffle_shuffle_reduce_128.S:61-169. */
void orc_spmv_csr_f32(int32_t m, const int32_t *row_ptr, const int32_t *col, const float *val,
                      const float *x, float alpha, float beta, float *y, int nthreads);

/* hygon/kernel/level3/mm/gemm/gemm_csr_row.hpp:15-73,124-165 (row-major B and C). */
void orc_spmm_csr_row_f32(int32_t m, const int32_t *row_ptr, const int32_t *col, const float *val,
                          const float *B, int32_t n, int32_t ldb, float alpha, float beta,
                          float *C, int32_t ldc, int nthreads);
/* hygon/kernel/level3/mm/gemm/gemm_csr_row.hpp:75-122 (generic-type twin). */
void orc_spmm_csr_row_f64(int32_t m, const int32_t *row_ptr, const int32_t *col, const double *val,
                          const double *B, int32_t n, int32_t ldb, double alpha, double beta,
                          double *C, int32_t ldc, int nthreads);

/* Row that holds stored element t*items for t in [0, nseg), nseg = ceil(nnz/items);
 * out[nseg] = m.  Same function as
 * hip/kernel/level3/alphasparse_spmm_csr_nnz_split.h:7-47 (elebalance_partition_kernel),
 * hip/kernel/level3/alphasparse_spmm_csr_adaptive.h:7-43,
 * hip/kernel/level3/alphasparse_spmm_csr_flat.h:6-25 and (items=1024)
 * hip/kernel/level2/alphasparse_spmv_csr_flat.h:7-38. */
void orc_nnz_split_rows(const int32_t *row_ptr, int32_t m, int32_t nnz, int32_t items,
                        int32_t *out /* ceil(nnz/items)+1 */);

/* hip/kernel/level2/alphasparse_spmv_csr_merge_ginkgo.h:10-33,132-157 (items=4096) and
 * hip/kernel/level3/alphasparse_spmm_csr_merge.h:6-30,32-75.  nblk = ceil((m+nnz)/items);
 * writes nblk+1 (x = rows consumed, y = nnz consumed) pairs. */
void orc_merge_path_search(const int32_t *row_ptr, int32_t m, int32_t nnz, int32_t items,
                           int32_t *xs, int32_t *ys);

/* hip/kernel/level2/alphasparse_spmv_csr_row_partition_ginkgo.h:93-122 (clac_size). */
int64_t orc_loadbalance_nwarps(int64_t nnz, int64_t warp_size, int64_t nwarps_base);
/* hip/kernel/level2/alphasparse_spmv_csr_row_partition_ginkgo.h:15-42,388-432. */
void orc_loadbalance_partition(const int32_t *row_ptr, int32_t m, int32_t nnz, int32_t warp_size,
                               int32_t nwarps, int32_t *out /* nwarps */);

/* hip/kernel/level2/alphasparse_spmv_csr_adaptive2.h:5-47 (find_rows): bin sizes and the nnz of the
 * middle bin.  The reference's row lists are filled through atomics, so only these are defined. */
void orc_find_rows_counts(const int32_t *row_ptr, int32_t m, int32_t thr1, int32_t thr2,
                          int32_t counts[3], int64_t *nnz_mid);

/* hip/kernel/level2/alphasparse_spmv_csr_adaptive.h:354-568 (ComputeRowBlocks) with
 * include/alphasparse/common.h:12-20,192-200.  Returns the number of entries written
 * (the reference reports twice that as its array size).  cap = capacity of out. */
size_t orc_csr_adaptive_row_blocks(const int32_t *row_ptr, int32_t m, uint64_t *out, size_t cap);

/* hip/format/coo2csr.h:7-16 forwards to hipsparseXcoo2csr (hipSPARSE, a system install the
 * reference does not pin and that is not part of its tree).  Its documented contract, restated:
 * for row indices sorted ascending, row_ptr[r] = number of entries with row index < r. */
void orc_coo2csr(const int32_t *row_ind, int32_t nnz, int32_t m, int32_t *row_ptr);

#ifdef __cplusplus
}
#endif
#endif
