// Drop-in header for the generic CSR SpMV / SpMM path of AlphaSparse on AMD gfx950.
//
// Callers written against the reference's <alphasparse.h> compile against this file for that
// path: the same type names, enumerator values, descriptor field names and function
// signatures (C++ linkage, as in the reference: none of its headers use extern "C").
// Struct layouts follow include/alphasparse/handle.h:26-87 (handle), :395-435 (sparse matrix
// descriptor), :478-499 (dense vector / matrix descriptors); enumerators follow
// include/alphasparse/spdef.h.  Everything else the reference's umbrella header drags in
// (other formats, solvers, SpGEMM, CPU back ends) is not part of this library.
//
// The arithmetic lives behind the C-ABI declared in alphasparse_amd.h.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

#include "alphasparse_amd.h"

// ---- enumerations (values are ABI; include/alphasparse/spdef.h) -----------------------------
typedef enum {  // spdef.h:10-22
    ALPHA_SPARSE_STATUS_SUCCESS = 0,
    ALPHA_SPARSE_STATUS_NOT_INITIALIZED = 1,
    ALPHA_SPARSE_STATUS_ALLOC_FAILED = 2,
    ALPHA_SPARSE_STATUS_INVALID_VALUE = 3,
    ALPHA_SPARSE_STATUS_EXECUTION_FAILED = 4,
    ALPHA_SPARSE_STATUS_INTERNAL_ERROR = 5,
    ALPHA_SPARSE_STATUS_NOT_SUPPORTED = 6,
    ALPHA_SPARSE_STATUS_INVALID_POINTER = 7,
    ALPHA_SPARSE_STATUS_INVALID_HANDLE = 8,
    ALPHA_SPARSE_STATUS_INVALID_KERNEL_PARAM = 9,
    ALPHA_SPARSE_STATUS_INVALID_SIZE = 10
} alphasparseStatus_t;

typedef enum {  // spdef.h:25-29
    ALPHA_SPARSE_OPERATION_NON_TRANSPOSE = 0,
    ALPHA_SPARSE_OPERATION_TRANSPOSE = 1,
    ALPHA_SPARSE_OPERATION_CONJUGATE_TRANSPOSE = 2
} alphasparseOperation_t;

typedef enum {  // spdef.h:33-43
    ALPHA_SPARSE_MATRIX_TYPE_GENERAL = 0,
    ALPHA_SPARSE_MATRIX_TYPE_SYMMETRIC = 1,
    ALPHA_SPARSE_MATRIX_TYPE_HERMITIAN = 2,
    ALPHA_SPARSE_MATRIX_TYPE_TRIANGULAR = 3,
    ALPHA_SPARSE_MATRIX_TYPE_DIAGONAL = 4,
    ALPHA_SPARSE_MATRIX_TYPE_BLOCK_TRIANGULAR = 5,
    ALPHA_SPARSE_MATRIX_TYPE_BLOCK_DIAGONAL = 6
} alphasparse_matrix_type_t;

typedef enum { ALPHA_SPARSE_INDEX_BASE_ZERO = 0, ALPHA_SPARSE_INDEX_BASE_ONE = 1 } alphasparseIndexBase_t;  // :49-52
typedef enum { ALPHA_SPARSE_FILL_MODE_LOWER = 0, ALPHA_SPARSE_FILL_MODE_UPPER = 1 } alphasparse_fill_mode_t;
typedef enum { ALPHA_SPARSE_DIAG_NON_UNIT = 0, ALPHA_SPARSE_DIAG_UNIT = 1 } alphasparse_diag_type_t;
typedef enum { ALPHASPARSE_ORDER_ROW = 0, ALPHASPARSE_ORDER_COL = 1 } alphasparseOrder_t;  // :83-86

typedef enum {  // spdef.h:125-140
    ALPHA_SPARSE_FORMAT_COO = 0,
    ALPHA_SPARSE_FORMAT_CSR = 1,
    ALPHA_SPARSE_FORMAT_CSC = 2,
    ALPHA_SPARSE_FORMAT_BSR = 3,
    ALPHA_SPARSE_FORMAT_SKY = 4,
    ALPHA_SPARSE_FORMAT_DIA = 5,
    ALPHA_SPARSE_FORMAT_ELL = 6,
    ALPHA_SPARSE_FORMAT_GEBSR = 7,
    ALPHA_SPARSE_FORMAT_HYB = 8,
    ALPHA_SPARSE_FORMAT_COOAOS = 9,
    ALPHA_SPARSE_FORMAT_CSR5 = 10,
    ALPHA_SPARSE_FORMAT_SELL_C_SIGMA = 11,
    ALPHA_SPARSE_FORMAT_ELLR = 12,
    ALPHA_SPARSE_FORMAT_BLOCKED_ELL = 13
} alphasparseFormat_t;

typedef enum {  // spdef.h:144-155
    ALPHA_R_32F = 0,
    ALPHA_R_64F = 1,
    ALPHA_C_32F = 2,
    ALPHA_C_64F = 3,
    ALPHA_R_16F = 4,
    ALPHA_R_16BF = 5,
    ALPHA_C_16F = 6,
    ALPHA_C_16BF = 7,
    ALPHA_R_8I = 8,
    ALPHA_R_32I = 9
} alphasparseDataType;

typedef enum { ALPHA_SPARSE_POINTER_MODE_HOST = 0, ALPHA_SPARSE_POINTER_MODE_DVICE = 1 } alphasparse_pointer_mode_t;
typedef enum {
    ALPHA_SPARSE_LAYER_MODE_NONE = 0,
    ALPHA_SPARSE_LAYER_MODE_LOG_TRACE = 1,
    ALPHA_SPARSE_LAYER_MODE_LOG_BENCH = 2
} alphasparse_layer_mode_t;

typedef enum {  // spdef.h:310-314
    ALPHA_SPARSE_INDEXTYPE_U16 = 1,
    ALPHA_SPARSE_INDEXTYPE_I32 = 2,
    ALPHA_SPARSE_INDEXTYPE_I64 = 3
} alphasparseIndexType_t;

typedef enum {  // spdef.h:345-365
    ALPHA_SPARSE_SPMV_ALG_DEFAULT = 0,
    ALPHA_SPARSE_SPMV_ALG_COO = 1,
    ALPHA_SPARSE_SPMV_ALG_CSR_ADAPTIVE = 2,
    ALPHA_SPARSE_SPMV_ALG_CSR_STREAM = 3,
    ALPHA_SPARSE_SPMV_ALG_ELL = 4,
    ALPHA_SPARSE_SPMV_ALG_SCALAR = 5,
    ALPHA_SPARSE_SPMV_ALG_VECTOR = 6,
    ALPHA_SPARSE_SPMV_ROW_PARTITION = 7,
    ALPHA_SPARSE_SPMV_ADAPTIVE = 8,
    ALPHA_SPARSE_SPMV_ALG_MERGE = 9,
    ALPHA_SPARSE_SPMV_ALG_LINE = 10,
    ALPHA_SPARSE_SPMV_ALG_FLAT1 = 11,
    ALPHA_SPARSE_SPMV_ALG_FLAT4 = 12,
    ALPHA_SPARSE_SPMV_ALG_FLAT8 = 13,
    ALPHA_SPARSE_SPMV_ALG_ACC = 14,
    ALPHA_SPARSE_SPMV_ALG_FLAT = 15,
    ALPHA_SPARSE_SPMV_ALG_LINE_ENHANCE = 16,
    ALPHA_SPARSE_SPMV_ALG_LOAD_BALANCE = 17,
    ALPHA_SPARSE_SPMV_ALG_PFLAT = 18
} alphasparseSpMVAlg_t;

typedef enum {  // spdef.h:390-402
    ALPHASPARSE_SPMM_ALG_DEFAULT = 0,
    ALPHASPARSE_SPMM_COO_ALG1 = 1,
    ALPHASPARSE_SPMM_COO_ALG2 = 2,
    ALPHASPARSE_SPMM_COO_ALG3 = 3,
    ALPHASPARSE_SPMM_COO_ALG4 = 4,
    ALPHASPARSE_SPMM_CSR_ALG1 = 5,
    ALPHASPARSE_SPMM_CSR_ALG2 = 6,
    ALPHASPARSE_SPMM_CSR_ALG3 = 7,
    ALPHASPARSE_SPMM_CSR_ALG4 = 8,
    ALPHASPARSE_SPMM_CSR_ALG5 = 9,
    ALPHASPARSE_SPMM_CSR_ALG6 = 10
} alphasparseSpMMAlg_t;

typedef enum { ALPHASPARSE_DIRECTION_ROW = 0, ALPHASPARSE_DIRECTION_COLUMN = 1 } alphasparseDirection_t;

typedef enum {  // spdef.h:175-184
    ALPHA_SPARSE_DATATYPE_FLOAT = 0,
    ALPHA_SPARSE_DATATYPE_DOUBLE = 1,
    ALPHA_SPARSE_DATATYPE_FLOAT_COMPLEX = 2,
    ALPHA_SPARSE_DATATYPE_DOUBLE_COMPLEX = 3,
    ALPHA_SPARSE_DATATYPE_HALF_FLOAT = 4,
    ALPHA_SPARSE_DATATYPE_HALF_DOUBLE = 5,
    ALPHA_SPARSE_DATATYPE_HALF_FLOAT_COMPLEX = 6,
    ALPHA_SPARSE_DATATYPE_HALF_DOUBLE_COMPLEX = 7
} alphasparse_datatype_t;

typedef enum {  // spdef.h:560-566
    ALPHA_SPARSE_DCU_SPMV_ALG_DEFAULT = 0,
    ALPHA_SPARSE_DCU_SPMV_ALG_COO = 1,
    ALPHA_SPARSE_DCU_SPMV_ALG_CSR_ADAPTIVE = 2,
    ALPHA_SPARSE_DCU_SPMV_ALG_CSR_STREAM = 3,
    ALPHA_SPARSE_DCU_SPMV_ALG_ELL = 4
} alphasparse_dcu_spmv_alg_t;

// ---- handle (include/alphasparse/handle.h:26-87) ---------------------------------------------
typedef struct alphasparse_handle_s {
    int device;
    int wavefront_size;
    int asic_rev;
    hipDeviceProp_t properties;
    hipStream_t stream;      // kernels of this library run on this stream
    hipStream_t streams[6];
    alphasparse_pointer_mode_t pointer_mode;
    alphasparse_layer_mode_t layer_mode;
    size_t buffer_size;
    void *buffer;            // device scratch owned by the handle
    float *sone;
    double *done;
    bool check_flag;
    int *process;
    void *pflat_analysis_data;  // here: the matrices that hold analysis results made through this handle

    alphasparse_handle_s()
        : device(0), wavefront_size(0), asic_rev(0), properties(), stream(nullptr), streams(),
          pointer_mode(ALPHA_SPARSE_POINTER_MODE_HOST), layer_mode(ALPHA_SPARSE_LAYER_MODE_NONE),
          buffer_size(0), buffer(nullptr), sone(nullptr), done(nullptr), check_flag(false),
          process(nullptr), pflat_analysis_data(nullptr)
    {
    }
} alphasparse_handle;
typedef alphasparse_handle *alphasparseHandle_t;

// ---- analysis info (include/alphasparse/handle.h:147-198, 216-248) ----------------------------
// The reference's home for what an analysis call learns about a matrix.  Nothing on the
// reference's generic SpMV / SpMM path fills it; here alphasparseSpMV_analysis and
// alphasparseSpMM_preprocess hang their results on the matrix through it (matA->info->csrmv_info,
// whose verification fields m, n, nnz, trans, csr_row_ptr, csr_col_ind are filled as the struct
// intends; the kernels' own metadata lives in an extension behind the same allocation).
struct alpha_matrix_descr {  // include/alphasparse/spdef.h:288-296
    alphasparse_matrix_type_t type;
    alphasparse_fill_mode_t mode;
    alphasparse_diag_type_t diag;
    alphasparseIndexBase_t base;
};
enum csrgemv_algo {  // handle.h:147-156
    ALPHA_CSRMV_AUTO,
    ALPHA_CSRMV_SCALAR,
    ALPHA_CSRMV_VECTOR,
    ALPHA_CSRMV_ROW_PARTITION,
    ALPHA_CSRMV_ADAPTIVE,
    ALPHA_CSRMV_MERGE,
    ALPHA_CSRMV_XXX
};
struct _alphasparse_csrmv_info {  // handle.h:158-198
    bool algo_tuning;
    csrgemv_algo algo;
    int iter;
    size_t size;
    unsigned long long *row_blocks;
    bool csr_adaptive_has_tuned;
    int32_t stream_num;
    int32_t vector_num;
    int32_t vectorL_num;
    int *partition;
    bool csr_rowpartition_has_tuned;
    void *coordinate;
    void *reduc_val;
    void *reduc_row;
    int num_merge_tiles;
    bool csr_merge_has_tuned;
    int *r_csr_row_ptr;
    int *r_csr_col_ind;
    int *r_row_indx;
    void *r_csr_val;
    alphasparseOperation_t trans;
    int m;
    int n;
    int nnz;
    const struct alpha_matrix_descr *descr;
    const void *csr_row_ptr;
    const void *csr_col_ind;
};
struct _alphasparse_trm_info;      // triangular-solve analysis: not on this path
struct _alphasparse_csrgemm_info;  // SpGEMM analysis: not on this path
typedef struct _alphasparse_trm_info *alphasparse_trm_info_t;
typedef struct _alphasparse_csrmv_info *alphasparse_csrmv_info_t;
typedef struct _alphasparse_csrgemm_info *alphasparse_csrgemm_info_t;
struct _alphasparse_mat_info {  // handle.h:216-248
    alphasparse_trm_info_t bsrsv_upper_info;
    alphasparse_trm_info_t bsrsv_lower_info;
    alphasparse_trm_info_t bsrsvt_upper_info;
    alphasparse_trm_info_t bsrsvt_lower_info;
    alphasparse_trm_info_t bsric0_info;
    alphasparse_trm_info_t bsrilu0_info;
    alphasparse_csrmv_info_t csrmv_info;
    alphasparse_trm_info_t csric0_info;
    alphasparse_trm_info_t csrilu0_info;
    alphasparse_trm_info_t csrsv_upper_info;
    alphasparse_trm_info_t csrsv_lower_info;
    alphasparse_trm_info_t csrsvt_upper_info;
    alphasparse_trm_info_t csrsvt_lower_info;
    alphasparse_trm_info_t csrsm_upper_info;
    alphasparse_trm_info_t csrsm_lower_info;
    alphasparse_trm_info_t csrsmt_upper_info;
    alphasparse_trm_info_t csrsmt_lower_info;
    alphasparse_csrgemm_info_t csrgemm_info;
    int *zero_pivot;
    int boost_enable;
    int use_double_prec_tol;
    const void *boost_tol;
    const void *boost_val;
};
typedef struct _alphasparse_mat_info *alphasparse_mat_info_t;

// ---- descriptors -----------------------------------------------------------------------------
struct _alphasparse_mat_descr {  // handle.h:329-358
    alphasparse_matrix_type_t type = ALPHA_SPARSE_MATRIX_TYPE_GENERAL;
    alphasparse_fill_mode_t fill_mode = ALPHA_SPARSE_FILL_MODE_LOWER;
    alphasparse_diag_type_t diag_type = ALPHA_SPARSE_DIAG_NON_UNIT;
    alphasparseIndexBase_t base = ALPHA_SPARSE_INDEX_BASE_ZERO;
    int64_t max_nnz_per_row = 0;
    bool spgemm_reuse_flag = false;
    void *row_map = {};
    void *rcsr_row_ptr = {};
    void *rcsr_col_idx = {};
    void *rcsr_val = {};
    int64_t warp_num_len = 0;
    void *d_warp_num = {};
    void *d_level_ptr = {};
    void *h_chain_ptr = {};
    int64_t h_level_size = 0;
    int64_t h_chain_size = 0;
    void *in_degree = {};
    void *csr_row_idx = {};
    void *csr_rdiag = {};
    void *rcsr_rdiag = {};
};
typedef struct _alphasparse_mat_descr *alphasparse_mat_descr_t;
typedef struct _alphasparse_mat_descr *alphasparseMatDescr_t;

struct _alphasparseSpMatDescr {  // handle.h:395-435
    bool init{};
    mutable bool analysed{};
    int64_t rows{};
    int64_t cols{};
    int64_t nnz{};
    int64_t nwarps{};
    int *row_data{};  // borrowed device pointers
    int *col_data{};
    int *ind_data{};
    void *val_data{};
    const int *const_row_data{};
    const int *const_col_data{};
    const int *const_ind_data{};
    const void *const_val_data{};
    alphasparseIndexType_t row_type{};
    alphasparseIndexType_t col_type{};
    alphasparseDataType data_type{};
    alphasparseIndexBase_t idx_base{};
    alphasparseFormat_t format{};
    alphasparse_mat_descr_t descr{};
    alphasparse_mat_info_t info{};
    alphasparseDirection_t block_dir{};
    int64_t block_dim{};
    int64_t ell_cols{};
    int64_t ell_width{};
    int64_t batch_count{};
    int64_t batch_stride{};
    int64_t offsets_batch_stride{};
    int64_t columns_values_batch_stride{};
};

struct _alphasparse_dnvec_descr {  // handle.h:478-485
    bool init{};
    int64_t size{};
    void *values{};
    alphasparseDataType data_type{};
};

struct _alphasparse_dnmat_descr {  // handle.h:487-499
    bool init{};
    int64_t rows{};
    int64_t cols{};
    int64_t ld{};
    void *values{};
    alphasparseDataType data_type{};
    alphasparseOrder_t order{};
};

typedef struct _alphasparseSpMatDescr *alphasparseSpMatDescr_t;
typedef struct _alphasparse_dnvec_descr *alphasparseDnVecDescr_t;
typedef struct _alphasparse_dnmat_descr *alphasparseDnMatDescr_t;
typedef struct _alphasparse_dnmat_descr *alphasparse_dnmat_descr_t;

// ---- handle life cycle (hip/util/handle.hip:53-154) ---------------------------------------------
alphasparseStatus_t initHandle(alphasparseHandle_t *handle);
alphasparseStatus_t alphasparseGetHandle(alphasparseHandle_t *handle);
alphasparseStatus_t alphasparse_destory_handle(alphasparseHandle_t handle);  // [sic], as in the reference

// ---- descriptor creation (hip/util/handle.hip:648-744; hip/format/alphasparse_create_csr.h:6-63) --
alphasparseStatus_t alphasparseCreateDnVec(alphasparseDnVecDescr_t *descr, int64_t size, void *values,
                                           alphasparseDataType data_type);
alphasparseStatus_t alphasparseCreateDnMat(alphasparseDnMatDescr_t *dnMatDescr, int64_t rows, int64_t cols,
                                           int64_t ld, void *values, alphasparseDataType valueType,
                                           alphasparseOrder_t order);
// Non-template body the header template below forwards to.
alphasparseStatus_t alphasparseCreateCsrUntyped(alphasparseSpMatDescr_t *spMatDescr, int64_t rows,
                                                int64_t cols, int64_t nnz, int *csrRowOffsets,
                                                int *col_data, void *val_data,
                                                alphasparseIndexType_t csrRowOffsetsType,
                                                alphasparseIndexType_t csrColIndType,
                                                alphasparseIndexBase_t idxBase,
                                                alphasparseDataType valueType);
template <typename T>
alphasparseStatus_t alphasparseCreateCsr(alphasparseSpMatDescr_t *spMatDescr, const int rows,
                                         const int cols, const int nnz, int *csrRowOffsets,
                                         int *col_data, T *val_data,
                                         const alphasparseIndexType_t csrRowOffsetsType,
                                         const alphasparseIndexType_t csrColIndType,
                                         const alphasparseIndexBase_t idxBase,
                                         const alphasparseDataType valueType)
{
    return alphasparseCreateCsrUntyped(spMatDescr, rows, cols, nnz, csrRowOffsets, col_data,
                                       (void *)val_data, csrRowOffsetsType, csrColIndType, idxBase,
                                       valueType);
}
// COO row indices (sorted) -> CSR row offsets, device arrays (hip/format/coo2csr.h:7-16).
template <typename T>
alphasparseStatus_t alphasparseXcoo2csr(const int *row_data, int nnz, int m, T *csrRowPtr)
{
    static_assert(sizeof(T) == sizeof(int32_t), "32-bit row offsets only");
    return (alphasparseStatus_t)asx_coo2csr(row_data, nnz, m, (int32_t *)csrRowPtr, nullptr);
}
// Extensions: the reference has no way to release these descriptors (they leak there).
alphasparseStatus_t alphasparseDestroySpMat(alphasparseSpMatDescr_t descr);
alphasparseStatus_t alphasparseDestroyDnVec(alphasparseDnVecDescr_t descr);
alphasparseStatus_t alphasparseDestroyDnMat(alphasparseDnMatDescr_t descr);

// ---- generic SpMV (include/alphasparse/spapi.h:6895-6926) ---------------------------------------
alphasparseStatus_t alphasparseSpMV(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                    const void *alpha, alphasparseSpMatDescr_t matA,
                                    alphasparseDnVecDescr_t vecX, const void *beta,
                                    alphasparseDnVecDescr_t vecY, alphasparseDataType computeType,
                                    alphasparseSpMVAlg_t alg, void *externalBuffer);
alphasparseStatus_t alphasparseSpMV_bufferSize(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                               const void *alpha, alphasparseSpMatDescr_t matA,
                                               alphasparseDnVecDescr_t vecX, const void *beta,
                                               alphasparseDnVecDescr_t vecY,
                                               alphasparseDataType computeType,
                                               alphasparseSpMVAlg_t alg, size_t *bufferSize);
alphasparseStatus_t alphasparseSpMV_analysis(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                             alphasparseSpMatDescr_t matA, alphasparseSpMVAlg_t alg);
alphasparseStatus_t alphasparseSpMV_clear(alphasparseHandle_t handle, alphasparseSpMVAlg_t alg);

// The two-phase form declared (and never defined) in include/alphasparse/spapi_dcu.h:4440-4450:
// with temp_buffer == nullptr only *buffer_size is written; otherwise the product is computed
// with temp_buffer as workspace.
alphasparseStatus_t alphasparse_spmv(alphasparseHandle_t handle, alphasparseOperation_t trans,
                                     const void *alpha, const alphasparseSpMatDescr_t mat,
                                     const alphasparseDnVecDescr_t x, const void *beta,
                                     const alphasparseDnVecDescr_t y, alphasparse_datatype_t compute_type,
                                     alphasparse_dcu_spmv_alg_t alg, size_t *buffer_size,
                                     void *temp_buffer);

// Not in the reference: the kernel the analysis kept on matA for (opA, algorithm, and for SpMM the
// number of dense columns) runs as, e.g. "sliced", "window", "flat", "merge" - or "none" when no
// analysis is kept (the call then picks a row-ordered kernel and recomputes its split points).
const char *alphasparseAmdKeptKernel(alphasparseSpMatDescr_t matA, alphasparseOperation_t opA, int is_spmm, int alg,
                                     int ncols);

// ---- generic SpMM (include/alphasparse/spapi.h:6963-6974,7004-7028) ------------------------------
alphasparseStatus_t alphasparseSpMM(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                    alphasparseOperation_t opB, const void *alpha,
                                    alphasparseSpMatDescr_t matA, alphasparseDnMatDescr_t matB,
                                    const void *beta, alphasparseDnMatDescr_t matC,
                                    alphasparseDataType computeType, alphasparseSpMMAlg_t alg,
                                    void *externalBuffer);
alphasparseStatus_t alphasparseSpMM_preprocess(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                               alphasparseOperation_t opB, const void *alpha,
                                               alphasparseSpMatDescr_t matA,
                                               alphasparseDnMatDescr_t matB, const void *beta,
                                               alphasparseDnMatDescr_t matC,
                                               alphasparseDataType computeType,
                                               alphasparseSpMMAlg_t alg, size_t *bufferSize);
alphasparseStatus_t alphasparseSpMM_bufferSize(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                               alphasparseOperation_t opB, const void *alpha,
                                               alphasparseSpMatDescr_t matA,
                                               alphasparseDnMatDescr_t matB, const void *beta,
                                               alphasparseDnMatDescr_t matC,
                                               alphasparseDataType computeType,
                                               alphasparseSpMMAlg_t alg, size_t *bufferSize);
