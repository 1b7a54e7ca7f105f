// TEST INFRASTRUCTURE ONLY.  extern "C" doors onto the *real* reference CPU path, so that
// Python tests and the CPU-baseline leg of the benchmark can call it through ctypes.
// This file holds no arithmetic: it only forwards to the reference's public entry points
// (alphasparse_?_create_csr, alphasparse_?_mv, alphasparse_?_mm, alphasparse_destroy:
// include/alphasparse/spapi.h:226-245,428,1000-1020,1272-1306) and to
// balanced_partition_row_by_nnz (hygon/util/partition.cpp:83-96).  It is compiled together
// with the reference's own sources, where they lie, by oracle/Makefile into oracle/_ref/.
#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "alphasparse/spapi.h"
#include "alphasparse/util/partition.h"
#include "alphasparse/util/thread.h"

namespace {
void set_threads(int nthreads)
{
    // alpha_get_thread_num() reads OMP_NUM_THREADS on every call (hygon/util/thread.cpp:33-44)
    char buf[32];
    std::snprintf(buf, sizeof buf, "%d", nthreads < 1 ? 1 : nthreads);
    setenv("OMP_NUM_THREADS", buf, 1);
    alpha_set_thread_num(nthreads < 1 ? 1 : nthreads);
}
struct alpha_matrix_descr general_descr()
{
    struct alpha_matrix_descr d;
    d.type = ALPHA_SPARSE_MATRIX_TYPE_GENERAL;
    d.mode = ALPHA_SPARSE_FILL_MODE_LOWER;
    d.diag = ALPHA_SPARSE_DIAG_NON_UNIT;
    d.base = ALPHA_SPARSE_INDEX_BASE_ZERO;
    return d;
}
}  // namespace

extern "C" {

void ref_partition_rows_by_nnz(const int32_t *row_end, int32_t rows, int32_t nthreads,
                               int32_t *partition)
{
    balanced_partition_row_by_nnz(row_end, rows, nthreads, partition);
}

// Handles: the reference deep-copies the arrays (hygon/format/create_csr.hpp:17-88).
void *ref_create_csr_f64(int32_t m, int32_t n, int32_t *row_ptr, int32_t *col, double *val)
{
    alphasparse_matrix_t A = nullptr;
    if (alphasparse_d_create_csr(&A, ALPHA_SPARSE_INDEX_BASE_ZERO, m, n, row_ptr, row_ptr + 1, col,
                                 val) != ALPHA_SPARSE_STATUS_SUCCESS)
        return nullptr;
    return A;
}
void *ref_create_csr_f32(int32_t m, int32_t n, int32_t *row_ptr, int32_t *col, float *val)
{
    alphasparse_matrix_t A = nullptr;
    if (alphasparse_s_create_csr(&A, ALPHA_SPARSE_INDEX_BASE_ZERO, m, n, row_ptr, row_ptr + 1, col,
                                 val) != ALPHA_SPARSE_STATUS_SUCCESS)
        return nullptr;
    return A;
}
void ref_destroy(void *A) { alphasparse_destroy((alphasparse_matrix_t)A); }

int ref_mv_f64(void *A, const double *x, double alpha, double beta, double *y, int nthreads)
{
    set_threads(nthreads);
    return (int)alphasparse_d_mv(ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, alpha,
                                 (alphasparse_matrix_t)A, general_descr(), x, beta, y);
}
int ref_mv_f32(void *A, const float *x, float alpha, float beta, float *y, int nthreads)
{
    set_threads(nthreads);
    return (int)alphasparse_s_mv(ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, alpha,
                                 (alphasparse_matrix_t)A, general_descr(), x, beta, y);
}
int ref_mm_row_f32(void *A, const float *B, int32_t n, int32_t ldb, float alpha, float beta,
                   float *C, int32_t ldc, int nthreads)
{
    set_threads(nthreads);
    return (int)alphasparse_s_mm(ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, alpha,
                                 (alphasparse_matrix_t)A, general_descr(),
                                 ALPHA_SPARSE_LAYOUT_ROW_MAJOR, B, n, ldb, beta, C, ldc);
}
int ref_mm_row_f64(void *A, const double *B, int32_t n, int32_t ldb, double alpha, double beta,
                   double *C, int32_t ldc, int nthreads)
{
    set_threads(nthreads);
    return (int)alphasparse_d_mm(ALPHA_SPARSE_OPERATION_NON_TRANSPOSE, alpha,
                                 (alphasparse_matrix_t)A, general_descr(),
                                 ALPHA_SPARSE_LAYOUT_ROW_MAJOR, B, n, ldb, beta, C, ldc);
}

}  // extern "C"
