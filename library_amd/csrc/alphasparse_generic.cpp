// Host side of the generic API: alphasparseSpMV / alphasparseSpMM and their helpers, with the
// reference's signatures and C++ linkage, on top of the C-ABI in alphasparse_amd.h.
//
// Behaviour kept from the reference: descriptors borrow the caller's device pointers
// (hip/format/alphasparse_create_csr.h:32-38); alpha and beta are host pointers read at call
// time (hip/kernel/level2/alphasparse_spmv.hip:44,49); errors are status codes, nothing throws
// across the boundary; null descriptor out-pointers give INVALID_POINTER and negative sizes
// INVALID_SIZE (hip/util/handle.hip:655-682).
// Deliberate differences: ALPHA_SPARSE_SPMV_ALG_DEFAULT runs a kernel (the reference's switch
// has no case for it and returns SUCCESS without computing, alphasparse_spmv.hip:36-179);
// unsupported type / format / operation / order combinations return NOT_SUPPORTED (the
// reference returns SUCCESS, alphasparse_spmv.hip:213-226); alphasparseSpMV_analysis and
// alphasparseSpMV_clear do something (stubs in the reference, alphasparse_spmv.hip:229-256);
// kernels run on handle->stream.
#include <cstddef>
#include <cstdlib>
#include <new>
#include <vector>

#include "../../include/alphasparse.h"

// Layout checks against the reference headers compiled with the same ROCm headers.
static_assert(offsetof(_alphasparseSpMatDescr, rows) == 8, "SpMat layout");
static_assert(offsetof(_alphasparseSpMatDescr, row_data) == 40, "SpMat layout");
static_assert(offsetof(_alphasparseSpMatDescr, col_data) == 48, "SpMat layout");
static_assert(offsetof(_alphasparseSpMatDescr, val_data) == 64, "SpMat layout");
static_assert(offsetof(_alphasparseSpMatDescr, row_type) == 104, "SpMat layout");
static_assert(offsetof(_alphasparseSpMatDescr, data_type) == 112, "SpMat layout");
static_assert(offsetof(_alphasparseSpMatDescr, idx_base) == 116, "SpMat layout");
static_assert(offsetof(_alphasparseSpMatDescr, format) == 120, "SpMat layout");
static_assert(offsetof(_alphasparseSpMatDescr, descr) == 128, "SpMat layout");
static_assert(sizeof(_alphasparseSpMatDescr) == 208, "SpMat layout");
static_assert(sizeof(_alphasparse_dnvec_descr) == 32, "DnVec layout");
static_assert(sizeof(_alphasparse_dnmat_descr) == 48, "DnMat layout");

namespace {

alphasparseStatus_t st(int s) { return (alphasparseStatus_t)s; }

alphasparseStatus_t from_hip(hipError_t e)  // hip/util/handle.hip:19-51
{
    switch (e) {
    case hipSuccess: return ALPHA_SPARSE_STATUS_SUCCESS;
    case hipErrorOutOfMemory: return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
    case hipErrorInvalidDevicePointer: return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    case hipErrorInvalidDevice:
    case hipErrorInvalidResourceHandle: return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
    case hipErrorInvalidValue: return ALPHA_SPARSE_STATUS_INVALID_VALUE;
    default: return ALPHA_SPARSE_STATUS_INTERNAL_ERROR;
    }
}

// Analysis results kept on the handle (its pflat_analysis_data slot).
struct KeptPlan {
    bool spmm;
    int requested_alg;
    const int *row_data;
    int64_t rows, nnz;
    int value_type;
    int ncols;
    asx_plan *plan;
};
struct HandlePlans {
    std::vector<KeptPlan> plans;
};
HandlePlans *plans_of(alphasparseHandle_t h, bool create)
{
    if (!h->pflat_analysis_data && create) h->pflat_analysis_data = new (std::nothrow) HandlePlans();
    return (HandlePlans *)h->pflat_analysis_data;
}
const asx_plan *find_plan(alphasparseHandle_t h, bool spmm, int alg, const _alphasparseSpMatDescr *A,
                          int ncols)
{
    HandlePlans *hp = plans_of(h, false);
    if (!hp) return nullptr;
    for (const KeptPlan &k : hp->plans)
        if (k.spmm == spmm && k.requested_alg == alg && k.row_data == A->row_data &&
            k.rows == A->rows && k.nnz == A->nnz && k.value_type == (int)A->data_type &&
            k.ncols == ncols)
            return k.plan;
    return nullptr;
}
void drop_plans(alphasparseHandle_t h, bool spmm, int alg, bool all)
{
    HandlePlans *hp = plans_of(h, false);
    if (!hp) return;
    std::vector<KeptPlan> keep;
    for (KeptPlan &k : hp->plans) {
        if (all || (k.spmm == spmm && k.requested_alg == alg))
            asx_plan_destroy(k.plan);
        else
            keep.push_back(k);
    }
    hp->plans.swap(keep);
}

// Checks shared by SpMV and SpMM on the sparse operand.
alphasparseStatus_t check_csr(const _alphasparseSpMatDescr *A, alphasparseOperation_t opA)
{
    if (!A->init) return ALPHA_SPARSE_STATUS_NOT_INITIALIZED;
    if (A->format != ALPHA_SPARSE_FORMAT_CSR) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    if (opA != ALPHA_SPARSE_OPERATION_NON_TRANSPOSE) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    if (A->idx_base != ALPHA_SPARSE_INDEX_BASE_ZERO) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    if (A->row_type != ALPHA_SPARSE_INDEXTYPE_I32 || A->col_type != ALPHA_SPARSE_INDEXTYPE_I32)
        return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    if (A->data_type != ALPHA_R_32F && A->data_type != ALPHA_R_64F)
        return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    if (A->rows < 0 || A->cols < 0 || A->nnz < 0) return ALPHA_SPARSE_STATUS_INVALID_SIZE;
    if (A->rows > INT32_MAX || A->cols > INT32_MAX || A->nnz > INT32_MAX)
        return ALPHA_SPARSE_STATUS_INVALID_SIZE;
    if (A->rows > 0 && !A->row_data) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    if (A->nnz > 0 && (!A->col_data || !A->val_data)) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparseStatus_t check_spmv(alphasparseHandle_t handle, alphasparseOperation_t opA,
                               const void *alpha, alphasparseSpMatDescr_t A,
                               alphasparseDnVecDescr_t X, const void *beta, alphasparseDnVecDescr_t Y,
                               alphasparseDataType computeType)
{
    if (!handle) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
    if (!alpha || !beta || !A || !X || !Y) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    alphasparseStatus_t s = check_csr(A, opA);
    if (s) return s;
    if (!X->init || !Y->init) return ALPHA_SPARSE_STATUS_NOT_INITIALIZED;
    if (X->data_type != A->data_type || Y->data_type != A->data_type || computeType != A->data_type)
        return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    if (X->size < A->cols || Y->size < A->rows) return ALPHA_SPARSE_STATUS_INVALID_SIZE;
    if ((A->rows > 0 && !Y->values) || (A->nnz > 0 && !X->values))
        return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparseStatus_t check_spmm(alphasparseHandle_t handle, alphasparseOperation_t opA,
                               alphasparseOperation_t opB, const void *alpha,
                               alphasparseSpMatDescr_t A, alphasparseDnMatDescr_t B, const void *beta,
                               alphasparseDnMatDescr_t Cm, alphasparseDataType computeType)
{
    if (!handle) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
    if (!alpha || !beta || !A || !B || !Cm) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    alphasparseStatus_t s = check_csr(A, opA);
    if (s) return s;
    if (opB != ALPHA_SPARSE_OPERATION_NON_TRANSPOSE) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    if (!B->init || !Cm->init) return ALPHA_SPARSE_STATUS_NOT_INITIALIZED;
    if (B->order != ALPHASPARSE_ORDER_ROW || Cm->order != ALPHASPARSE_ORDER_ROW)
        return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    if (B->data_type != A->data_type || Cm->data_type != A->data_type || computeType != A->data_type)
        return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    if (B->rows < A->cols || Cm->rows < A->rows || B->cols != Cm->cols)
        return ALPHA_SPARSE_STATUS_INVALID_SIZE;
    if (B->ld < B->cols || Cm->ld < Cm->cols || Cm->cols > INT32_MAX)
        return ALPHA_SPARSE_STATUS_INVALID_SIZE;
    if (!B->values || !Cm->values) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

// Picks the workspace for a call: the caller's buffer, or the handle's own scratch when the
// caller passed none and the need fits.
void *pick_workspace(alphasparseHandle_t h, void *external, size_t need, bool *ok)
{
    *ok = true;
    if (need == 0) return external;
    if (external) return external;
    if (h->buffer && h->buffer_size >= need) return h->buffer;
    *ok = false;
    return nullptr;
}

}  // namespace

// ------------------------------------------------------------------------------------ handle
alphasparseStatus_t initHandle(alphasparseHandle_t *handle)
{
    if (!handle) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    alphasparse_handle *h = new (std::nothrow) alphasparse_handle();
    if (!h) return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
    h->stream = nullptr;
    for (int i = 0; i < 6; ++i) {
        hipError_t e = hipStreamCreate(&h->streams[i]);  // default priority
        if (e != hipSuccess) {
            for (int j = 0; j < i; ++j) (void)hipStreamDestroy(h->streams[j]);
            delete h;
            return from_hip(e);
        }
    }
    *handle = h;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparseStatus_t alphasparseGetHandle(alphasparseHandle_t *handle)
{
    if (!handle) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    if (*handle == nullptr) {
        alphasparseStatus_t s = initHandle(handle);
        if (s) return s;
    }
    alphasparse_handle *h = *handle;
    hipError_t e = hipGetDevice(&h->device);
    if (e != hipSuccess) return from_hip(e);
    e = hipGetDeviceProperties(&h->properties, h->device);
    if (e != hipSuccess) return from_hip(e);
    h->wavefront_size = h->properties.warpSize;
    const char *layer = std::getenv("ALPHA_SPARSE_LAYER");
    h->layer_mode = layer ? (alphasparse_layer_mode_t)std::atoi(layer) : ALPHA_SPARSE_LAYER_MODE_NONE;
    if (!h->buffer) {  // calling GetHandle again on a live handle keeps its scratch
        h->buffer_size = 1024 * 1024;
        e = hipMalloc(&h->buffer, h->buffer_size);
        if (e != hipSuccess) return from_hip(e);
        e = hipMalloc((void **)&h->sone, sizeof(float));
        if (e != hipSuccess) return from_hip(e);
        e = hipMalloc((void **)&h->done, sizeof(double));
        if (e != hipSuccess) return from_hip(e);
        const float one_f = 1.0f;
        const double one_d = 1.0;
        e = hipMemcpyAsync(h->sone, &one_f, sizeof one_f, hipMemcpyHostToDevice, h->stream);
        if (e != hipSuccess) return from_hip(e);
        e = hipMemcpyAsync(h->done, &one_d, sizeof one_d, hipMemcpyHostToDevice, h->stream);
        if (e != hipSuccess) return from_hip(e);
        e = hipStreamSynchronize(h->stream);
        if (e != hipSuccess) return from_hip(e);
    }
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparseStatus_t alphasparse_destory_handle(alphasparseHandle_t handle)
{
    if (!handle) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
    drop_plans(handle, false, 0, true);
    delete (HandlePlans *)handle->pflat_analysis_data;
    handle->pflat_analysis_data = nullptr;
    if (handle->buffer) (void)hipFree(handle->buffer);
    if (handle->sone) (void)hipFree(handle->sone);
    if (handle->done) (void)hipFree(handle->done);
    for (int i = 0; i < 6; ++i)
        if (handle->streams[i]) (void)hipStreamDestroy(handle->streams[i]);
    delete handle;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

// ------------------------------------------------------------------------------------ descriptors
alphasparseStatus_t alphasparseCreateDnVec(alphasparseDnVecDescr_t *descr, int64_t size, void *values,
                                           alphasparseDataType data_type)
{
    if (!descr) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    if (size < 0) return ALPHA_SPARSE_STATUS_INVALID_SIZE;
    if (size > 0 && !values) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    *descr = new (std::nothrow) _alphasparse_dnvec_descr();
    if (!*descr) return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
    (*descr)->init = true;
    (*descr)->size = size;
    (*descr)->values = values;
    (*descr)->data_type = data_type;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparseStatus_t alphasparseCreateDnMat(alphasparseDnMatDescr_t *dnMatDescr, int64_t rows, int64_t cols,
                                           int64_t ld, void *values, alphasparseDataType valueType,
                                           alphasparseOrder_t order)
{
    if (!dnMatDescr) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    if (rows < 0 || cols < 0) return ALPHA_SPARSE_STATUS_INVALID_SIZE;
    if (!values) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    *dnMatDescr = new (std::nothrow) _alphasparse_dnmat_descr();
    if (!*dnMatDescr) return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
    (*dnMatDescr)->init = true;
    (*dnMatDescr)->rows = rows;
    (*dnMatDescr)->cols = cols;
    (*dnMatDescr)->ld = ld;
    (*dnMatDescr)->values = values;
    (*dnMatDescr)->data_type = valueType;
    (*dnMatDescr)->order = order;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparseStatus_t alphasparseCreateCsrUntyped(alphasparseSpMatDescr_t *spMatDescr, int64_t rows,
                                                int64_t cols, int64_t nnz, int *csrRowOffsets,
                                                int *col_data, void *val_data,
                                                alphasparseIndexType_t csrRowOffsetsType,
                                                alphasparseIndexType_t csrColIndType,
                                                alphasparseIndexBase_t idxBase,
                                                alphasparseDataType valueType)
{
    if (!spMatDescr) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    *spMatDescr = nullptr;
    _alphasparseSpMatDescr *d = new (std::nothrow) _alphasparseSpMatDescr();
    _alphasparse_mat_descr *md = new (std::nothrow) _alphasparse_mat_descr();
    if (!d || !md) {
        delete d;
        delete md;
        return ALPHA_SPARSE_STATUS_NOT_INITIALIZED;  // the reference's catch-all for a failed new
    }
    d->init = true;
    d->rows = rows;
    d->cols = cols;
    d->nnz = nnz;
    d->row_data = csrRowOffsets;
    d->col_data = col_data;
    d->val_data = val_data;
    d->const_row_data = csrRowOffsets;
    d->const_col_data = col_data;
    d->const_val_data = val_data;
    d->row_type = csrRowOffsetsType;
    d->col_type = csrColIndType;
    d->data_type = valueType;
    d->idx_base = idxBase;
    d->format = ALPHA_SPARSE_FORMAT_CSR;
    md->base = idxBase;
    d->descr = md;
    d->batch_count = 1;
    *spMatDescr = d;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparseStatus_t alphasparseDestroySpMat(alphasparseSpMatDescr_t descr)
{
    if (!descr) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    delete descr->descr;
    delete descr;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}
alphasparseStatus_t alphasparseDestroyDnVec(alphasparseDnVecDescr_t descr)
{
    if (!descr) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    delete descr;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}
alphasparseStatus_t alphasparseDestroyDnMat(alphasparseDnMatDescr_t descr)
{
    if (!descr) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    delete descr;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

// ------------------------------------------------------------------------------------ SpMV
alphasparseStatus_t alphasparseSpMV_bufferSize(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                               const void *alpha, alphasparseSpMatDescr_t matA,
                                               alphasparseDnVecDescr_t vecX, const void *beta,
                                               alphasparseDnVecDescr_t vecY,
                                               alphasparseDataType computeType,
                                               alphasparseSpMVAlg_t alg, size_t *bufferSize)
{
    if (!bufferSize) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    alphasparseStatus_t s = check_spmv(handle, opA, alpha, matA, vecX, beta, vecY, computeType);
    if (s) return s;
    if (asx_spmv_resolve_alg((int)alg, (int32_t)matA->rows, (int32_t)matA->nnz) < 0)
        return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    // sized for a call without kept analysis; a call with kept analysis needs no more than this
    *bufferSize = asx_spmv_workspace_bytes((int)alg, (int)matA->data_type, (int32_t)matA->rows,
                                           (int32_t)matA->nnz);
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparseStatus_t alphasparseSpMV_analysis(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                             alphasparseSpMatDescr_t matA, alphasparseSpMVAlg_t alg)
{
    if (!handle) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
    if (!matA) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    alphasparseStatus_t s = check_csr(matA, opA);
    if (s) return s;
    if (find_plan(handle, false, (int)alg, matA, 1)) return ALPHA_SPARSE_STATUS_SUCCESS;
    HandlePlans *hp = plans_of(handle, true);
    if (!hp) return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
    asx_plan *plan = nullptr;
    int rc = asx_plan_create(&plan, 0, (int)alg, (int)matA->data_type, (int32_t)matA->rows,
                             (int32_t)matA->cols, (int32_t)matA->nnz, matA->row_data, 1,
                             (void *)handle->stream);
    if (rc) return st(rc);
    hp->plans.push_back(KeptPlan{false, (int)alg, matA->row_data, matA->rows, matA->nnz,
                                 (int)matA->data_type, 1, plan});
    matA->analysed = true;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparseStatus_t alphasparseSpMV_clear(alphasparseHandle_t handle, alphasparseSpMVAlg_t alg)
{
    if (!handle) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
    drop_plans(handle, false, (int)alg, false);
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparseStatus_t alphasparseSpMV(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                    const void *alpha, alphasparseSpMatDescr_t matA,
                                    alphasparseDnVecDescr_t vecX, const void *beta,
                                    alphasparseDnVecDescr_t vecY, alphasparseDataType computeType,
                                    alphasparseSpMVAlg_t alg, void *externalBuffer)
{
    alphasparseStatus_t s = check_spmv(handle, opA, alpha, matA, vecX, beta, vecY, computeType);
    if (s) return s;
    const int32_t m = (int32_t)matA->rows, n = (int32_t)matA->cols, nnz = (int32_t)matA->nnz;
    if (asx_spmv_resolve_alg((int)alg, m, nnz) < 0) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    const asx_plan *plan = find_plan(handle, false, (int)alg, matA, 1);
    const size_t need = plan ? asx_plan_workspace_bytes(plan)
                             : asx_spmv_workspace_bytes((int)alg, (int)matA->data_type, m, nnz);
    bool ok;
    void *ws = pick_workspace(handle, externalBuffer, need, &ok);
    if (!ok) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    // the size of a caller's buffer is not part of the signature: it is trusted to be what
    // alphasparseSpMV_bufferSize reported
    const size_t ws_bytes = need;
    int rc;
    if (matA->data_type == ALPHA_R_64F)
        rc = asx_spmv_csr_f64(plan, (int)alg, m, n, nnz, *(const double *)alpha, matA->row_data,
                              matA->col_data, (const double *)matA->val_data,
                              (const double *)vecX->values, *(const double *)beta,
                              (double *)vecY->values, ws, ws_bytes, (void *)handle->stream);
    else
        rc = asx_spmv_csr_f32(plan, (int)alg, m, n, nnz, *(const float *)alpha, matA->row_data,
                              matA->col_data, (const float *)matA->val_data,
                              (const float *)vecX->values, *(const float *)beta,
                              (float *)vecY->values, ws, ws_bytes, (void *)handle->stream);
    return st(rc);
}

alphasparseStatus_t alphasparse_spmv(alphasparseHandle_t handle, alphasparseOperation_t trans,
                                     const void *alpha, const alphasparseSpMatDescr_t mat,
                                     const alphasparseDnVecDescr_t x, const void *beta,
                                     const alphasparseDnVecDescr_t y, alphasparse_datatype_t compute_type,
                                     alphasparse_dcu_spmv_alg_t alg, size_t *buffer_size,
                                     void *temp_buffer)
{
    alphasparseDataType ct;
    switch (compute_type) {
    case ALPHA_SPARSE_DATATYPE_FLOAT: ct = ALPHA_R_32F; break;
    case ALPHA_SPARSE_DATATYPE_DOUBLE: ct = ALPHA_R_64F; break;
    default: return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    }
    // the five ids of this enumeration carry the same values in alphasparseSpMVAlg_t
    const alphasparseSpMVAlg_t a = (alphasparseSpMVAlg_t)(int)alg;
    if (temp_buffer == nullptr) {
        if (!buffer_size) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
        return alphasparseSpMV_bufferSize(handle, trans, alpha, mat, x, beta, y, ct, a, buffer_size);
    }
    return alphasparseSpMV(handle, trans, alpha, mat, x, beta, y, ct, a, temp_buffer);
}

// ------------------------------------------------------------------------------------ SpMM
alphasparseStatus_t alphasparseSpMM_bufferSize(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                               alphasparseOperation_t opB, const void *alpha,
                                               alphasparseSpMatDescr_t matA,
                                               alphasparseDnMatDescr_t matB, const void *beta,
                                               alphasparseDnMatDescr_t matC,
                                               alphasparseDataType computeType,
                                               alphasparseSpMMAlg_t alg, size_t *bufferSize)
{
    if (!bufferSize) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    alphasparseStatus_t s = check_spmm(handle, opA, opB, alpha, matA, matB, beta, matC, computeType);
    if (s) return s;
    if (asx_spmm_resolve_alg((int)alg, (int32_t)matA->rows, (int32_t)matA->nnz, (int32_t)matC->cols) < 0)
        return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    *bufferSize = asx_spmm_workspace_bytes((int)alg, (int)matA->data_type, (int32_t)matA->rows,
                                           (int32_t)matA->nnz, (int32_t)matC->cols);
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

// Builds and keeps the analysis for (matA, N = matC->cols, alg): merge split points, or for
// ALPHASPARSE_SPMM_CSR_ALG6 (and for DEFAULT when the 16x4 blocks of A are at least 1/8 full) the
// blocked copy of A for the MFMA kernel, which holds A's values: call again after changing them.
// *bufferSize, when given, receives the workspace a later alphasparseSpMM call needs (never more
// than alphasparseSpMM_bufferSize reports).
alphasparseStatus_t alphasparseSpMM_preprocess(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                               alphasparseOperation_t opB, const void *alpha,
                                               alphasparseSpMatDescr_t matA,
                                               alphasparseDnMatDescr_t matB, const void *beta,
                                               alphasparseDnMatDescr_t matC,
                                               alphasparseDataType computeType,
                                               alphasparseSpMMAlg_t alg, size_t *bufferSize)
{
    alphasparseStatus_t s = check_spmm(handle, opA, opB, alpha, matA, matB, beta, matC, computeType);
    if (s) return s;
    const int ncols = (int)matC->cols;
    if (asx_spmm_resolve_alg((int)alg, (int32_t)matA->rows, (int32_t)matA->nnz, ncols) < 0)
        return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    const asx_plan *have = find_plan(handle, true, (int)alg, matA, ncols);
    if (!have) {
        HandlePlans *hp = plans_of(handle, true);
        if (!hp) return ALPHA_SPARSE_STATUS_ALLOC_FAILED;
        asx_plan *plan = nullptr;
        int rc = asx_spmm_plan_create(&plan, (int)alg, (int)matA->data_type, (int32_t)matA->rows,
                                      (int32_t)matA->cols, (int32_t)matA->nnz, matA->row_data,
                                      matA->col_data, matA->val_data, ncols, (void *)handle->stream);
        if (rc) return st(rc);
        hp->plans.push_back(KeptPlan{true, (int)alg, matA->row_data, matA->rows, matA->nnz,
                                     (int)matA->data_type, ncols, plan});
        have = plan;
        matA->analysed = true;
    }
    if (bufferSize) *bufferSize = asx_plan_workspace_bytes(have);
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

alphasparseStatus_t alphasparseSpMM(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                    alphasparseOperation_t opB, const void *alpha,
                                    alphasparseSpMatDescr_t matA, alphasparseDnMatDescr_t matB,
                                    const void *beta, alphasparseDnMatDescr_t matC,
                                    alphasparseDataType computeType, alphasparseSpMMAlg_t alg,
                                    void *externalBuffer)
{
    alphasparseStatus_t s = check_spmm(handle, opA, opB, alpha, matA, matB, beta, matC, computeType);
    if (s) return s;
    const int32_t m = (int32_t)matA->rows, k = (int32_t)matA->cols, nnz = (int32_t)matA->nnz;
    const int32_t ncols = (int32_t)matC->cols;
    if (asx_spmm_resolve_alg((int)alg, m, nnz, ncols) < 0) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    const asx_plan *plan = find_plan(handle, true, (int)alg, matA, ncols);
    const size_t need = plan ? asx_plan_workspace_bytes(plan)
                             : asx_spmm_workspace_bytes((int)alg, (int)matA->data_type, m, nnz, ncols);
    bool ok;
    void *ws = pick_workspace(handle, externalBuffer, need, &ok);
    if (!ok) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    int rc;
    if (matA->data_type == ALPHA_R_64F)
        rc = asx_spmm_csr_f64(plan, (int)alg, m, k, nnz, ncols, *(const double *)alpha, matA->row_data,
                              matA->col_data, (const double *)matA->val_data,
                              (const double *)matB->values, matB->ld, *(const double *)beta,
                              (double *)matC->values, matC->ld, ws, need, (void *)handle->stream);
    else
        rc = asx_spmm_csr_f32(plan, (int)alg, m, k, nnz, ncols, *(const float *)alpha, matA->row_data,
                              matA->col_data, (const float *)matA->val_data,
                              (const float *)matB->values, matB->ld, *(const float *)beta,
                              (float *)matC->values, matC->ld, ws, need, (void *)handle->stream);
    return st(rc);
}
