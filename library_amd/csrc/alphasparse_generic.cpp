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
// kernels run on handle->stream; opA = TRANSPOSE runs on a device-built transposed copy and
// leaves the caller's arrays alone (the reference transposes on the host, writes the result
// over the caller's arrays and so toggles A between calls, hip/format/transpose_csr.h:9-71);
// one-based CSR is honoured (the reference's CSR kernels ignore idx_base); column-major B / C
// and opB go through a tiled device transpose into the call's workspace (the reference
// transposes B and C in place and rewrites their descriptors, alphasparse_spmm.hip:186-216).
#include <algorithm>
#include <cstddef>
#include <cstdlib>
#include <mutex>
#include <new>
#include <unordered_set>
#include <vector>

#include "../../include/alphasparse.h"

// Layout checks.  The numbers are those of the reference's own headers compiled with the same
// ROCm headers (tests/golden/layout.json, written by tests/golden/make_layout.py).
#define ASX_OFF(T, f, v) static_assert(offsetof(T, f) == (v), #T "::" #f " moved")
static_assert(sizeof(alphasparse_handle_s) == 1608, "handle layout");
ASX_OFF(alphasparse_handle_s, properties, 16);
ASX_OFF(alphasparse_handle_s, stream, 1488);
ASX_OFF(alphasparse_handle_s, streams, 1496);
ASX_OFF(alphasparse_handle_s, pointer_mode, 1544);
ASX_OFF(alphasparse_handle_s, layer_mode, 1548);
ASX_OFF(alphasparse_handle_s, buffer_size, 1552);
ASX_OFF(alphasparse_handle_s, buffer, 1560);
ASX_OFF(alphasparse_handle_s, sone, 1568);
ASX_OFF(alphasparse_handle_s, done, 1576);
ASX_OFF(alphasparse_handle_s, check_flag, 1584);
ASX_OFF(alphasparse_handle_s, process, 1592);
ASX_OFF(alphasparse_handle_s, pflat_analysis_data, 1600);
static_assert(sizeof(_alphasparseSpMatDescr) == 208, "SpMat layout");
ASX_OFF(_alphasparseSpMatDescr, rows, 8);
ASX_OFF(_alphasparseSpMatDescr, row_data, 40);
ASX_OFF(_alphasparseSpMatDescr, col_data, 48);
ASX_OFF(_alphasparseSpMatDescr, val_data, 64);
ASX_OFF(_alphasparseSpMatDescr, const_row_data, 72);
ASX_OFF(_alphasparseSpMatDescr, row_type, 104);
ASX_OFF(_alphasparseSpMatDescr, data_type, 112);
ASX_OFF(_alphasparseSpMatDescr, idx_base, 116);
ASX_OFF(_alphasparseSpMatDescr, format, 120);
ASX_OFF(_alphasparseSpMatDescr, descr, 128);
ASX_OFF(_alphasparseSpMatDescr, info, 136);
ASX_OFF(_alphasparseSpMatDescr, batch_count, 176);
static_assert(sizeof(_alphasparse_mat_descr) == 144, "mat_descr layout");
ASX_OFF(_alphasparse_mat_descr, base, 12);
ASX_OFF(_alphasparse_mat_descr, max_nnz_per_row, 16);
ASX_OFF(_alphasparse_mat_descr, row_map, 32);
ASX_OFF(_alphasparse_mat_descr, h_level_size, 96);
ASX_OFF(_alphasparse_mat_descr, h_chain_size, 104);
ASX_OFF(_alphasparse_mat_descr, csr_rdiag, 128);
ASX_OFF(_alphasparse_mat_descr, rcsr_rdiag, 136);
static_assert(sizeof(_alphasparse_dnvec_descr) == 32, "DnVec layout");
ASX_OFF(_alphasparse_dnvec_descr, values, 16);
ASX_OFF(_alphasparse_dnvec_descr, data_type, 24);
static_assert(sizeof(_alphasparse_dnmat_descr) == 48, "DnMat layout");
ASX_OFF(_alphasparse_dnmat_descr, ld, 24);
ASX_OFF(_alphasparse_dnmat_descr, values, 32);
ASX_OFF(_alphasparse_dnmat_descr, order, 44);
static_assert(sizeof(_alphasparse_csrmv_info) == 168, "csrmv_info layout");
ASX_OFF(_alphasparse_csrmv_info, row_blocks, 24);
ASX_OFF(_alphasparse_csrmv_info, partition, 48);
ASX_OFF(_alphasparse_csrmv_info, coordinate, 64);
ASX_OFF(_alphasparse_csrmv_info, trans, 128);
ASX_OFF(_alphasparse_csrmv_info, csr_row_ptr, 152);
static_assert(sizeof(_alphasparse_mat_info) == 176, "mat_info layout");
ASX_OFF(_alphasparse_mat_info, csrmv_info, 48);
ASX_OFF(_alphasparse_mat_info, csrgemm_info, 136);
ASX_OFF(_alphasparse_mat_info, boost_val, 168);
#undef ASX_OFF

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

// What analysis keeps, per matrix.  The object sits behind matA->info: its first member is the
// reference's _alphasparse_mat_info (include/alphasparse/handle.h:216-248), whose csrmv_info
// points at the second (handle.h:158-198); the kernels' plans follow.  The matrix owns it
// (alphasparseDestroySpMat releases it); the handle that made it lists it, so that
// alphasparseSpMV_clear and the handle's destruction can release the device memory of callers
// who, like the reference's, never destroy a descriptor.
struct KeptPlan {
    bool spmm;
    int requested_alg;
    // the arrays the plan was built from (the caller's, or a kept zero-based / transposed copy)
    const int *row_data;
    const int *col_data;
    const void *val_data;
    int64_t rows, cols, nnz;
    int value_type;
    int ncols;
    asx_plan *plan;
    bool reads_callers_values_only;  // made by analysis on first use: no copy of A's values, or one guarded by checksums
};
// A zero-based and/or transposed device copy of a caller's CSR matrix.
struct DerivedCsr {
    const int *src_row;
    const int *src_col;
    const void *src_val;
    int64_t rows, cols, nnz;
    int value_type, base;
    bool transposed;
    int *row_ptr, *col;
    void *val;  // owned only when transposed (otherwise the caller's values)
};
// What alphasparseSpMV_bufferSize last reported for (matrix, algorithm): the size the caller's
// externalBuffer is taken to have (its size is not part of alphasparseSpMV's signature).
struct PromisedBuffer {
    int alg;
    size_t bytes;
};
struct MatInfoExt {
    _alphasparse_mat_info info;
    _alphasparse_csrmv_info csrmv;
    alphasparseHandle_t owner;  // null once that handle is gone
    std::vector<KeptPlan> plans;
    std::vector<PromisedBuffer> promised;
    std::vector<DerivedCsr> derived;  // kept by alphasparseSpMV_analysis / alphasparseSpMM_preprocess
};
struct HandleRegistry {
    std::vector<MatInfoExt *> mats;
};
HandleRegistry *registry_of(alphasparseHandle_t h, bool create)
{
    if (!h->pflat_analysis_data && create) h->pflat_analysis_data = new (std::nothrow) HandleRegistry();
    return (HandleRegistry *)h->pflat_analysis_data;
}
// The objects this library has put behind a matA->info, by address: a pointer found there is
// only taken for one of them after it was looked up here (a caller compiled against the
// reference's header may have put its own, smaller _alphasparse_mat_info there, which must not
// be read past its end).
struct LiveInfos {
    std::mutex lock;
    std::unordered_set<const void *> set;
};
LiveInfos &live_infos()
{
    static LiveInfos *l = new LiveInfos();  // never destroyed: descriptors may outlive static destructors
    return *l;
}
MatInfoExt *ext_of(const _alphasparseSpMatDescr *A)
{
    if (!A->info) return nullptr;
    LiveInfos &l = live_infos();
    std::lock_guard<std::mutex> g(l.lock);
    return l.set.count(A->info) ? (MatInfoExt *)A->info : nullptr;
}
// The matrix's store, made on first use (a foreign object already behind matA->info is left alone:
// analysis then reports NOT_SUPPORTED).
MatInfoExt *ext_create(alphasparseHandle_t h, _alphasparseSpMatDescr *A)
{
    if (MatInfoExt *e = ext_of(A)) {
        if (!e->owner) {  // the handle that made it is gone: this one takes it over
            HandleRegistry *reg = registry_of(h, true);
            if (!reg) return nullptr;
            reg->mats.push_back(e);
            e->owner = h;
        }
        return e;
    }
    if (A->info) return nullptr;
    HandleRegistry *reg = registry_of(h, true);
    if (!reg) return nullptr;
    MatInfoExt *e = new (std::nothrow) MatInfoExt();
    if (!e) return nullptr;
    e->info = _alphasparse_mat_info{};
    e->csrmv = _alphasparse_csrmv_info{};
    e->info.csrmv_info = &e->csrmv;
    e->owner = h;
    {
        LiveInfos &l = live_infos();
        std::lock_guard<std::mutex> g(l.lock);
        l.set.insert(&e->info);
    }
    reg->mats.push_back(e);
    A->info = &e->info;
    return e;
}
void free_derived(DerivedCsr &d);
// Releases plans: those of one (kind, algorithm), or everything the matrix keeps.
void ext_drop(MatInfoExt *e, bool spmm, int alg, bool all)
{
    std::vector<KeptPlan> keep;
    for (KeptPlan &k : e->plans) {
        if (all || (k.spmm == spmm && k.requested_alg == alg))
            asx_plan_destroy(k.plan);
        else
            keep.push_back(k);
    }
    e->plans.swap(keep);
    if (all) {
        for (DerivedCsr &d : e->derived) free_derived(d);
        e->derived.clear();
    }
}
asx_plan *find_plan(const _alphasparseSpMatDescr *owner, bool spmm, int alg, const _alphasparseSpMatDescr *A,
                    int ncols)
{
    MatInfoExt *e = ext_of(owner);
    if (!e) return nullptr;
    for (const KeptPlan &k : e->plans)
        if (k.spmm == spmm && k.requested_alg == alg && k.row_data == A->row_data && k.col_data == A->col_data &&
            k.val_data == A->val_data && k.rows == A->rows && k.cols == A->cols && k.nnz == A->nnz &&
            k.value_type == (int)A->data_type && k.ncols == ncols)
            return k.plan;
    return nullptr;
}
size_t promised_bytes(const _alphasparseSpMatDescr *A, int alg)
{
    if (MatInfoExt *e = ext_of(A))
        for (const PromisedBuffer &p : e->promised)
            if (p.alg == alg) return p.bytes;
    return 0;
}
bool kept_is_restricted(const _alphasparseSpMatDescr *A, const asx_plan *plan)
{
    if (MatInfoExt *e = ext_of(A))
        for (const KeptPlan &k : e->plans)
            if (k.plan == plan) return k.reads_callers_values_only;
    return false;
}
void drop_one_plan(const _alphasparseSpMatDescr *A, asx_plan *plan)
{
    MatInfoExt *e = ext_of(A);
    if (!e) return;
    for (size_t i = 0; i < e->plans.size(); ++i)
        if (e->plans[i].plan == plan) {
            asx_plan_destroy(plan);
            e->plans.erase(e->plans.begin() + (long)i);
            return;
        }
}
void drop_plans(alphasparseHandle_t h, bool spmm, int alg, bool all)
{
    HandleRegistry *reg = registry_of(h, false);
    if (!reg) return;
    for (MatInfoExt *e : reg->mats) ext_drop(e, spmm, alg, all);
}

bool is_transpose(alphasparseOperation_t op)
{
    // real value types only: the conjugate transpose is the transpose
    return op == ALPHA_SPARSE_OPERATION_TRANSPOSE || op == ALPHA_SPARSE_OPERATION_CONJUGATE_TRANSPOSE;
}
bool same_source(const DerivedCsr &d, const _alphasparseSpMatDescr *A, bool transposed);
// The kept plan a call with (A, opA, alg) would find, without building anything.
const asx_plan *kept_plan(const _alphasparseSpMatDescr *A, alphasparseOperation_t opA, bool spmm, int alg, int ncols)
{
    MatInfoExt *x = ext_of(A);
    if (!x) return nullptr;
    const bool tr = is_transpose(opA);
    if (!tr && A->idx_base == ALPHA_SPARSE_INDEX_BASE_ZERO) return find_plan(A, spmm, alg, A, ncols);
    for (const DerivedCsr &d : x->derived) {
        if (!same_source(d, A, tr)) continue;
        _alphasparseSpMatDescr e = *A;
        e.row_data = d.row_ptr;
        e.col_data = d.col;
        e.val_data = d.val;
        if (tr) e.rows = A->cols, e.cols = A->rows;
        return find_plan(A, spmm, alg, &e, ncols);
    }
    return nullptr;
}

void free_derived(DerivedCsr &d)
{
    if (d.row_ptr) (void)hipFree(d.row_ptr);
    if (d.col) (void)hipFree(d.col);
    if (d.transposed && d.val) (void)hipFree(d.val);
    d.row_ptr = d.col = nullptr;
    d.val = nullptr;
}

bool same_source(const DerivedCsr &d, const _alphasparseSpMatDescr *A, bool transposed)
{
    return d.src_row == A->row_data && d.src_col == A->col_data && d.src_val == A->val_data &&
           d.rows == A->rows && d.cols == A->cols && d.nnz == A->nnz && d.value_type == (int)A->data_type &&
           d.base == (int)A->idx_base && d.transposed == transposed;
}

// Builds the zero-based (and, if asked, transposed) device copy of A.
alphasparseStatus_t build_derived(alphasparseHandle_t h, const _alphasparseSpMatDescr *A, bool transposed,
                                  DerivedCsr *out)
{
    DerivedCsr d{};
    d.src_row = A->row_data;
    d.src_col = A->col_data;
    d.src_val = A->val_data;
    d.rows = A->rows;
    d.cols = A->cols;
    d.nnz = A->nnz;
    d.value_type = (int)A->data_type;
    d.base = (int)A->idx_base;
    d.transposed = transposed;
    const size_t sv = A->data_type == ALPHA_R_64F ? 8 : 4;
    const size_t nrow = (size_t)(transposed ? A->cols : A->rows) + 1;
    const size_t nnz1 = A->nnz > 0 ? (size_t)A->nnz : 1;
    hipError_t e = hipMalloc((void **)&d.row_ptr, nrow * sizeof(int));
    if (e == hipSuccess) e = hipMalloc((void **)&d.col, nnz1 * sizeof(int));
    if (e == hipSuccess && transposed) e = hipMalloc(&d.val, nnz1 * sv);
    if (e != hipSuccess) {
        free_derived(d);
        return from_hip(e);
    }
    int rc;
    if (transposed) {
        rc = asx_csr_transpose((int)A->data_type, (int32_t)A->rows, (int32_t)A->cols, (int32_t)A->nnz,
                               (int32_t)A->idx_base, A->row_data, A->col_data, A->val_data, d.row_ptr, d.col,
                               d.val, (void *)h->stream);
    } else {
        d.val = A->val_data;
        rc = asx_csr_rebase((int32_t)A->rows, (int32_t)A->nnz, (int32_t)A->idx_base, A->row_data, A->col_data,
                            d.row_ptr, d.col, (void *)h->stream);
    }
    if (rc) {
        free_derived(d);
        return st(rc);
    }
    *out = d;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

// The matrix the kernels run on for (A, opA): A itself, a kept derived copy, or a copy made for
// this call alone (`temporary`, released by release_effective once the call's work is queued).
struct Effective {
    _alphasparseSpMatDescr d;
    DerivedCsr temp;
    bool temporary;
};
alphasparseStatus_t make_effective(alphasparseHandle_t h, const _alphasparseSpMatDescr *A,
                                   alphasparseOperation_t opA, Effective *e)
{
    e->d = *A;
    e->temporary = false;
    e->temp = DerivedCsr{};
    const bool tr = is_transpose(opA);
    if (!tr && A->idx_base == ALPHA_SPARSE_INDEX_BASE_ZERO) return ALPHA_SPARSE_STATUS_SUCCESS;
    const DerivedCsr *use = nullptr;
    if (MatInfoExt *x = ext_of(A))
        for (const DerivedCsr &d : x->derived)
            if (same_source(d, A, tr)) use = &d;
    if (!use) {
        alphasparseStatus_t s = build_derived(h, A, tr, &e->temp);
        if (s) return s;
        e->temporary = true;
        use = &e->temp;
    }
    e->d.row_data = use->row_ptr;
    e->d.col_data = use->col;
    e->d.val_data = use->val;
    e->d.idx_base = ALPHA_SPARSE_INDEX_BASE_ZERO;
    if (tr) {
        e->d.rows = A->cols;
        e->d.cols = A->rows;
    }
    return ALPHA_SPARSE_STATUS_SUCCESS;
}
void release_effective(alphasparseHandle_t h, Effective *e)
{
    if (!e->temporary) return;
    (void)hipStreamSynchronize(h->stream);  // the call's kernels read the copy
    free_derived(e->temp);
    e->temporary = false;
}

// Makes (or remakes, picking up changed values or structure) the kept derived copy for (A, opA);
// plans built on the copy it replaces are dropped.
alphasparseStatus_t keep_derived(alphasparseHandle_t h, _alphasparseSpMatDescr *A, alphasparseOperation_t opA)
{
    const bool tr = is_transpose(opA);
    if (!tr && A->idx_base == ALPHA_SPARSE_INDEX_BASE_ZERO) return ALPHA_SPARSE_STATUS_SUCCESS;
    MatInfoExt *x = ext_create(h, A);
    if (!x) return A->info ? ALPHA_SPARSE_STATUS_NOT_SUPPORTED : ALPHA_SPARSE_STATUS_ALLOC_FAILED;
    (void)hipStreamSynchronize(h->stream);
    for (size_t i = 0; i < x->derived.size();) {
        if (!same_source(x->derived[i], A, tr)) {
            ++i;
            continue;
        }
        std::vector<KeptPlan> keep;
        for (KeptPlan &k : x->plans) {
            if (k.row_data == x->derived[i].row_ptr)
                asx_plan_destroy(k.plan);
            else
                keep.push_back(k);
        }
        x->plans.swap(keep);
        free_derived(x->derived[i]);
        x->derived.erase(x->derived.begin() + (long)i);
    }
    DerivedCsr d{};
    alphasparseStatus_t s = build_derived(h, A, tr, &d);
    if (s) return s;
    x->derived.push_back(d);
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

// Checks shared by SpMV and SpMM on the sparse operand.
alphasparseStatus_t check_csr(const _alphasparseSpMatDescr *A, alphasparseOperation_t opA)
{
    if (!A->init) return ALPHA_SPARSE_STATUS_NOT_INITIALIZED;
    if (A->format != ALPHA_SPARSE_FORMAT_CSR) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    if (opA != ALPHA_SPARSE_OPERATION_NON_TRANSPOSE && !is_transpose(opA)) return ALPHA_SPARSE_STATUS_INVALID_VALUE;
    if (A->idx_base != ALPHA_SPARSE_INDEX_BASE_ZERO && A->idx_base != ALPHA_SPARSE_INDEX_BASE_ONE)
        return ALPHA_SPARSE_STATUS_INVALID_VALUE;
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
    const int64_t out_len = is_transpose(opA) ? A->cols : A->rows;
    const int64_t in_len = is_transpose(opA) ? A->rows : A->cols;
    if (X->size < in_len || Y->size < out_len) return ALPHA_SPARSE_STATUS_INVALID_SIZE;
    if ((out_len > 0 && !Y->values) || (A->nnz > 0 && !X->values))
        return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

// How a dense SpMM operand reaches the kernels, which take row-major k x N (B) and m x N (C).
// A column-major matrix is a row-major matrix of the transposed shape in memory, and op = T
// swaps the two readings, so each operand is either usable in place or needs one transpose.
struct DenseUse {
    int64_t rows, cols;  // of op(matrix)
    bool direct;         // memory already is row-major rows x cols with stride ld
};
DenseUse dense_use(const _alphasparse_dnmat_descr *M, bool transposed)
{
    DenseUse u;
    u.rows = transposed ? M->cols : M->rows;
    u.cols = transposed ? M->rows : M->cols;
    u.direct = (M->order == ALPHASPARSE_ORDER_ROW) != transposed;
    return u;
}
size_t align256(size_t v) { return (v + 255) / 256 * 256; }

alphasparseStatus_t check_spmm(alphasparseHandle_t handle, alphasparseOperation_t opA,
                               alphasparseOperation_t opB, const void *alpha,
                               alphasparseSpMatDescr_t A, alphasparseDnMatDescr_t B, const void *beta,
                               alphasparseDnMatDescr_t Cm, alphasparseDataType computeType)
{
    if (!handle) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
    if (!alpha || !beta || !A || !B || !Cm) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    alphasparseStatus_t s = check_csr(A, opA);
    if (s) return s;
    if (opB != ALPHA_SPARSE_OPERATION_NON_TRANSPOSE && !is_transpose(opB)) return ALPHA_SPARSE_STATUS_INVALID_VALUE;
    if (!B->init || !Cm->init) return ALPHA_SPARSE_STATUS_NOT_INITIALIZED;
    if ((B->order != ALPHASPARSE_ORDER_ROW && B->order != ALPHASPARSE_ORDER_COL) ||
        (Cm->order != ALPHASPARSE_ORDER_ROW && Cm->order != ALPHASPARSE_ORDER_COL))
        return ALPHA_SPARSE_STATUS_INVALID_VALUE;
    if (B->data_type != A->data_type || Cm->data_type != A->data_type || computeType != A->data_type)
        return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    const int64_t m = is_transpose(opA) ? A->cols : A->rows, k = is_transpose(opA) ? A->rows : A->cols;
    const DenseUse ub = dense_use(B, is_transpose(opB)), uc = dense_use(Cm, false);
    if (ub.rows < k || uc.rows < m || ub.cols != uc.cols) return ALPHA_SPARSE_STATUS_INVALID_SIZE;
    // the leading dimension spans a row of the row-major reading of the memory
    if (B->ld < (ub.direct ? ub.cols : ub.rows) || Cm->ld < (uc.direct ? uc.cols : uc.rows) ||
        uc.cols > INT32_MAX)
        return ALPHA_SPARSE_STATUS_INVALID_SIZE;
    if (!B->values || !Cm->values) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

// Bytes of the row-major copies a call needs after its kernel workspace.
void spmm_copy_bytes(const _alphasparseSpMatDescr *A, alphasparseOperation_t opA,
                     const _alphasparse_dnmat_descr *B, alphasparseOperation_t opB,
                     const _alphasparse_dnmat_descr *Cm, size_t *b_bytes, size_t *c_bytes)
{
    const size_t sv = A->data_type == ALPHA_R_64F ? 8 : 4;
    const int64_t m = is_transpose(opA) ? A->cols : A->rows, k = is_transpose(opA) ? A->rows : A->cols;
    const int64_t N = Cm->cols;
    *b_bytes = dense_use(B, is_transpose(opB)).direct ? 0 : align256((size_t)k * (size_t)N * sv);
    *c_bytes = dense_use(Cm, false).direct ? 0 : align256((size_t)m * (size_t)N * sv);
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
    // the device memory of everything analysed through this handle goes with it; the (small)
    // host objects stay with their matrices
    drop_plans(handle, false, 0, true);
    if (HandleRegistry *reg = registry_of(handle, false)) {
        for (MatInfoExt *e : reg->mats) e->owner = nullptr;
        delete reg;
    }
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
    if (MatInfoExt *e = ext_of(descr)) {
        ext_drop(e, false, 0, true);
        if (e->owner)
            if (HandleRegistry *reg = registry_of(e->owner, false))
                for (size_t i = 0; i < reg->mats.size(); ++i)
                    if (reg->mats[i] == e) {
                        reg->mats.erase(reg->mats.begin() + (long)i);
                        break;
                    }
        {
            LiveInfos &l = live_infos();
            std::lock_guard<std::mutex> g(l.lock);
            l.set.erase(&e->info);
        }
        delete e;
        descr->info = nullptr;
    }
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
    const int32_t m_eff = (int32_t)(is_transpose(opA) ? matA->cols : matA->rows);
    if (asx_spmv_resolve_alg((int)alg, m_eff, (int32_t)matA->nnz) < 0)
        return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    // sized for a call without kept analysis, and for DEFAULT for the row-ordered kernels a later
    // alphasparseSpMV_analysis may settle on.  Kept analysis that regrouped A (column slices, row
    // blocks) needs room for the partial sums or carries of a call: reported when the analysis is
    // there already (call this after alphasparseSpMV_analysis to run calls with buffers of their
    // own at the same time; a buffer sized before the analysis is too small for them and such
    // calls use the buffer the analysis keeps, one at a time)
    size_t need = asx_spmv_workspace_bytes((int)alg, (int)matA->data_type, m_eff, (int32_t)matA->nnz);
    if (const asx_plan *plan = kept_plan(matA, opA, false, (int)alg, 1))
        need = std::max(need, asx_plan_workspace_bytes(plan));
    *bufferSize = need;
    // remember what the caller's buffer is now taken to hold
    if (MatInfoExt *x = ext_create(handle, matA)) {
        bool found = false;
        for (PromisedBuffer &p : x->promised)
            if (p.alg == (int)alg) p.bytes = need, found = true;
        if (!found) x->promised.push_back(PromisedBuffer{(int)alg, need});
    }
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

// Analysis on first use, for callers written against the reference, where alphasparseSpMV_analysis
// and alphasparseSpMM_preprocess are stubs or cheap and therefore often never called
// (hip/kernel/level2/alphasparse_spmv.hip:229-256; its own test loops go from _bufferSize straight to
// the timed alphasparseSpMV, hip/test/level2/spmv_csr_r_f64_test.hip:183-198): the first
// alphasparseSpMV / alphasparseSpMM on a descriptor runs an analysis itself (allocates and
// synchronises once; later calls are kernels only).  ALPHASPARSE_AMD_AUTO_ANALYSIS selects how far
// it goes; read once per process:
//   unset, "checked"    SpMV: the full analysis, which may keep a regrouped copy of A's values, guarded:
//                       every call takes two 64-bit checksums of the caller's values (one read of them
//                       on the device, counted when the kernel is chosen) and refreshes the copy where
//                       they differ from the kept ones, so a caller who changes values in place is
//                       served as by the reference.  SpMM, and SpMV with opA = TRANSPOSE: as "structure".
//   "structure"         only analysis that reads the caller's values in every call (split points
//                       of the row-ordered kernels): sound whenever the row offsets and columns
//                       behind a descriptor stay as they are, which holds for a caller who
//                       changes values in place.  Not done for opA = TRANSPOSE (the kept copy of
//                       the transposed matrix would hold values).
//   "1", "values"       the full analysis without the checksums: for callers who do not change
//                       values in place without calling the analysis again
//   "0", "off"          none: every call recomputes its split points, as the reference does
// In every mode the sparsity pattern behind a descriptor is taken to stay as it is.
enum AutoAnalysis { kAutoOff = 0, kAutoStructure = 1, kAutoValues = 2, kAutoChecked = 3 };
static AutoAnalysis auto_analysis()
{
    static const AutoAnalysis mode = [] {
        const char *e = std::getenv("ALPHASPARSE_AMD_AUTO_ANALYSIS");
        if (!e || !e[0] || e[0] == 'c' || e[0] == 'C') return kAutoChecked;
        if (e[0] == 's' || e[0] == 'S') return kAutoStructure;
        if (e[0] == '0' || e[0] == 'o' || e[0] == 'O' || e[0] == 'n' || e[0] == 'N') return kAutoOff;
        return kAutoValues;
    }();
    return mode;
}

// what an analysis may keep: anything (the caller's own analysis call), only what reads the
// caller's values in every call, or a copy of the values guarded by checksums
enum Keeps { kKeepsAnything = 0, kKeepsStructure = 1, kKeepsCheckedValues = 2 };
static alphasparseStatus_t spmv_analysis(alphasparseHandle_t handle, alphasparseOperation_t opA, alphasparseSpMatDescr_t matA,
                                         alphasparseSpMVAlg_t alg, Keeps keeps);

alphasparseStatus_t alphasparseSpMV_analysis(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                             alphasparseSpMatDescr_t matA, alphasparseSpMVAlg_t alg)
{
    return spmv_analysis(handle, opA, matA, alg, kKeepsAnything);
}

static alphasparseStatus_t spmv_analysis(alphasparseHandle_t handle, alphasparseOperation_t opA, alphasparseSpMatDescr_t matA,
                                         alphasparseSpMVAlg_t alg, Keeps keeps)
{
    const bool callers_values_only = keeps != kKeepsAnything;  // made on first use: gives way to the caller's own analysis
    if (!handle) return ALPHA_SPARSE_STATUS_INVALID_HANDLE;
    if (!matA) return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    alphasparseStatus_t s = check_csr(matA, opA);
    if (s) return s;
    // for opA = TRANSPOSE or one-based A this (re)builds the kept device copy the kernels run on:
    // call again after changing A's values or structure
    s = keep_derived(handle, matA, opA);
    if (s) return s;
    Effective eff;
    s = make_effective(handle, matA, opA, &eff);
    if (s) return s;
    const _alphasparseSpMatDescr *A = &eff.d;
    if (asx_plan *have = find_plan(matA, false, (int)alg, A, 1)) {
        // analysed before: the sparsity pattern is taken to be the same (alphasparseSpMV_clear first
        // if it is not); a plan that holds a copy of the values picks up the current ones.  What
        // analysis on first use left there makes way for the caller's own, full analysis.
        if (callers_values_only || !kept_is_restricted(matA, have))
            return st(asx_plan_update_values(have, A->val_data, (void *)handle->stream));
        (void)hipStreamSynchronize(handle->stream);
        drop_one_plan(matA, have);
    }
    MatInfoExt *x = ext_create(handle, matA);
    if (!x) return matA->info ? ALPHA_SPARSE_STATUS_NOT_SUPPORTED : ALPHA_SPARSE_STATUS_ALLOC_FAILED;
    asx_plan *plan = nullptr;
    // may keep a regrouped copy of A's columns and values (column slices, row blocks): call again
    // after changing the values.  Without the columns and values the plan stays row-ordered.
    int rc = keeps == kKeepsCheckedValues
                 ? asx_spmv_plan_create_checked(&plan, (int)alg, (int)A->data_type, (int32_t)A->rows, (int32_t)A->cols,
                                                (int32_t)A->nnz, A->row_data, A->col_data, A->val_data, (void *)handle->stream)
                 : asx_spmv_plan_create(&plan, (int)alg, (int)A->data_type, (int32_t)A->rows, (int32_t)A->cols,
                                        (int32_t)A->nnz, A->row_data, keeps == kKeepsStructure ? nullptr : A->col_data,
                                        keeps == kKeepsStructure ? nullptr : A->val_data, (void *)handle->stream);
    if (rc) return st(rc);
    x->plans.push_back(KeptPlan{false, (int)alg, A->row_data, A->col_data, A->val_data, A->rows, A->cols, A->nnz,
                                (int)A->data_type, 1, plan, callers_values_only});
    // the reference's own record of what was analysed (include/alphasparse/handle.h:190-197)
    x->csrmv.trans = opA;
    x->csrmv.m = (int)matA->rows;
    x->csrmv.n = (int)matA->cols;
    x->csrmv.nnz = (int)matA->nnz;
    x->csrmv.csr_row_ptr = matA->row_data;
    x->csrmv.csr_col_ind = matA->col_data;
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
    const int32_t m_eff = (int32_t)(is_transpose(opA) ? matA->cols : matA->rows);
    if (asx_spmv_resolve_alg((int)alg, m_eff, (int32_t)matA->nnz) < 0) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    // without a copy kept by alphasparseSpMV_analysis, opA = TRANSPOSE and one-based A build their
    // device copy for this call alone (from the values A holds now, as the reference does)
    Effective eff;
    s = make_effective(handle, matA, opA, &eff);
    if (s) return s;
    const _alphasparseSpMatDescr *A = &eff.d;
    const int32_t m = (int32_t)A->rows, n = (int32_t)A->cols, nnz = (int32_t)A->nnz;
    const asx_plan *plan = find_plan(matA, false, (int)alg, A, 1);
    const AutoAnalysis mode = auto_analysis();
    if (!plan && (mode == kAutoValues || (mode != kAutoOff && !is_transpose(opA))) && (!matA->info || ext_of(matA))) {
        release_effective(handle, &eff);
        s = spmv_analysis(handle, opA, matA, alg,
                          mode == kAutoValues ? kKeepsAnything : mode == kAutoChecked ? kKeepsCheckedValues : kKeepsStructure);
        if (s) return s;
        s = make_effective(handle, matA, opA, &eff);
        if (s) return s;
        plan = find_plan(matA, false, (int)alg, A, 1);
    }
    const size_t need = plan ? asx_plan_workspace_bytes(plan)
                             : asx_spmv_workspace_bytes((int)alg, (int)A->data_type, m, nnz);
    // the size of a caller's buffer is not part of the signature: it is trusted to be what
    // alphasparseSpMV_bufferSize last reported for this matrix and algorithm (never queried: what
    // a call without kept analysis needs)
    void *ws;
    size_t ws_bytes = need;
    if (plan && asx_plan_own_scratch_bytes(plan) >= need && need > 0) {
        // kept analysis with a buffer of its own for the partial sums / carries of a call: the
        // caller's buffer is used only when it was sized after the analysis
        const size_t have = externalBuffer ? promised_bytes(matA, (int)alg) : 0;
        ws = have >= need ? externalBuffer : nullptr;
        ws_bytes = have >= need ? have : 0;
    } else {
        bool ok;
        ws = pick_workspace(handle, externalBuffer, need, &ok);
        if (!ok) {
            release_effective(handle, &eff);
            return ALPHA_SPARSE_STATUS_INVALID_POINTER;
        }
    }
    int rc = plan && asx_plan_is_checked(plan)
                 ? asx_plan_refresh_if_changed(const_cast<asx_plan *>(plan), A->val_data, (void *)handle->stream)
                 : ASX_STATUS_SUCCESS;
    if (rc) {
        release_effective(handle, &eff);
        return st(rc);
    }
    if (A->data_type == ALPHA_R_64F)
        rc = asx_spmv_csr_f64(plan, (int)alg, m, n, nnz, *(const double *)alpha, A->row_data, A->col_data,
                              (const double *)A->val_data, (const double *)vecX->values,
                              *(const double *)beta, (double *)vecY->values, ws, ws_bytes,
                              (void *)handle->stream);
    else
        rc = asx_spmv_csr_f32(plan, (int)alg, m, n, nnz, *(const float *)alpha, A->row_data, A->col_data,
                              (const float *)A->val_data, (const float *)vecX->values,
                              *(const float *)beta, (float *)vecY->values, ws, ws_bytes,
                              (void *)handle->stream);
    release_effective(handle, &eff);
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

const char *alphasparseAmdKeptKernel(alphasparseSpMatDescr_t matA, alphasparseOperation_t opA, int is_spmm, int alg, int ncols)
{
    if (!matA) return "none";
    const asx_plan *plan = kept_plan(matA, opA, is_spmm != 0, alg, is_spmm ? ncols : 1);
    return plan ? asx_kernel_name(is_spmm, asx_plan_alg(plan)) : "none";
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
    const int32_t m_eff = (int32_t)(is_transpose(opA) ? matA->cols : matA->rows);
    if (asx_spmm_resolve_alg((int)alg, m_eff, (int32_t)matA->nnz, (int32_t)matC->cols) < 0)
        return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    size_t b_bytes, c_bytes;
    spmm_copy_bytes(matA, opA, matB, opB, matC, &b_bytes, &c_bytes);
    *bufferSize = align256(asx_spmm_workspace_bytes((int)alg, (int)matA->data_type, m_eff, (int32_t)matA->nnz,
                                                    (int32_t)matC->cols)) +
                  b_bytes + c_bytes;
    return ALPHA_SPARSE_STATUS_SUCCESS;
}

// Builds and keeps the analysis for (matA, N = matC->cols, alg): merge split points, or for
// ALPHASPARSE_SPMM_CSR_ALG6 (and for DEFAULT when the 16x4 blocks of A are at least 1/8 full) the
// blocked copy of A for the MFMA kernel, which holds A's values: call again after changing them.
// *bufferSize, when given, receives the workspace a later alphasparseSpMM call needs (never more
// than alphasparseSpMM_bufferSize reports).
static alphasparseStatus_t spmm_preprocess(alphasparseHandle_t handle, alphasparseOperation_t opA, alphasparseOperation_t opB,
                                           const void *alpha, alphasparseSpMatDescr_t matA, alphasparseDnMatDescr_t matB,
                                           const void *beta, alphasparseDnMatDescr_t matC, alphasparseDataType computeType,
                                           alphasparseSpMMAlg_t alg, size_t *bufferSize, bool callers_values_only);

alphasparseStatus_t alphasparseSpMM_preprocess(alphasparseHandle_t handle, alphasparseOperation_t opA,
                                               alphasparseOperation_t opB, const void *alpha,
                                               alphasparseSpMatDescr_t matA,
                                               alphasparseDnMatDescr_t matB, const void *beta,
                                               alphasparseDnMatDescr_t matC,
                                               alphasparseDataType computeType,
                                               alphasparseSpMMAlg_t alg, size_t *bufferSize)
{
    return spmm_preprocess(handle, opA, opB, alpha, matA, matB, beta, matC, computeType, alg, bufferSize, false);
}

static alphasparseStatus_t spmm_preprocess(alphasparseHandle_t handle, alphasparseOperation_t opA, alphasparseOperation_t opB,
                                           const void *alpha, alphasparseSpMatDescr_t matA, alphasparseDnMatDescr_t matB,
                                           const void *beta, alphasparseDnMatDescr_t matC, alphasparseDataType computeType,
                                           alphasparseSpMMAlg_t alg, size_t *bufferSize, bool callers_values_only)
{
    alphasparseStatus_t s = check_spmm(handle, opA, opB, alpha, matA, matB, beta, matC, computeType);
    if (s) return s;
    const int ncols = (int)matC->cols;
    const int32_t m_eff = (int32_t)(is_transpose(opA) ? matA->cols : matA->rows);
    if (asx_spmm_resolve_alg((int)alg, m_eff, (int32_t)matA->nnz, ncols) < 0)
        return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    s = keep_derived(handle, matA, opA);  // (re)builds the kept copy for opA = T / one-based A
    if (s) return s;
    Effective eff;
    s = make_effective(handle, matA, opA, &eff);
    if (s) return s;
    const _alphasparseSpMatDescr *A = &eff.d;
    asx_plan *have = find_plan(matA, true, (int)alg, A, ncols);
    if (have && !callers_values_only && kept_is_restricted(matA, have)) {
        // what analysis on first use left there makes way for the caller's own, full preprocessing
        (void)hipStreamSynchronize(handle->stream);
        drop_one_plan(matA, have);
        have = nullptr;
    }
    if (have) {
        // preprocessed before: a plan that holds a copy of A's values picks up the current ones
        int rc = asx_plan_update_values(have, A->val_data, (void *)handle->stream);
        if (rc) return st(rc);
    } else {
        MatInfoExt *x = ext_create(handle, matA);
        if (!x) return matA->info ? ALPHA_SPARSE_STATUS_NOT_SUPPORTED : ALPHA_SPARSE_STATUS_ALLOC_FAILED;
        asx_plan *plan = nullptr;
        // without the columns and values: split points only, never the blocked copy of A's values
        int rc = callers_values_only
                     ? asx_plan_create(&plan, 1, (int)alg, (int)A->data_type, (int32_t)A->rows, (int32_t)A->cols,
                                       (int32_t)A->nnz, A->row_data, ncols, (void *)handle->stream)
                     : asx_spmm_plan_create(&plan, (int)alg, (int)A->data_type, (int32_t)A->rows, (int32_t)A->cols,
                                            (int32_t)A->nnz, A->row_data, A->col_data, A->val_data, ncols,
                                            (void *)handle->stream);
        if (rc) return st(rc);
        x->plans.push_back(KeptPlan{true, (int)alg, A->row_data, A->col_data, A->val_data, A->rows, A->cols, A->nnz,
                                    (int)A->data_type, ncols, plan, callers_values_only});
        have = plan;
        matA->analysed = true;
    }
    if (bufferSize) {
        size_t b_bytes, c_bytes;
        spmm_copy_bytes(matA, opA, matB, opB, matC, &b_bytes, &c_bytes);
        *bufferSize = align256(asx_plan_workspace_bytes(have)) + b_bytes + c_bytes;
    }
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
    const int32_t ncols = (int32_t)matC->cols;
    const int32_t m_eff = (int32_t)(is_transpose(opA) ? matA->cols : matA->rows);
    if (asx_spmm_resolve_alg((int)alg, m_eff, (int32_t)matA->nnz, ncols) < 0) return ALPHA_SPARSE_STATUS_NOT_SUPPORTED;
    Effective eff;
    s = make_effective(handle, matA, opA, &eff);
    if (s) return s;
    const _alphasparseSpMatDescr *A = &eff.d;
    const int32_t m = (int32_t)A->rows, k = (int32_t)A->cols, nnz = (int32_t)A->nnz;
    const int vt = (int)A->data_type;
    const asx_plan *plan = find_plan(matA, true, (int)alg, A, ncols);
    const AutoAnalysis mode = auto_analysis();
    const bool structure_only = mode == kAutoStructure || mode == kAutoChecked;  // no checksums for SpMM plans
    if (!plan && (mode == kAutoValues || (structure_only && !is_transpose(opA))) && (!matA->info || ext_of(matA))) {
        release_effective(handle, &eff);
        size_t unused = 0;
        s = spmm_preprocess(handle, opA, opB, alpha, matA, matB, beta, matC, computeType, alg, &unused, structure_only);
        // the blocked algorithm has no analysis without A's values: the call goes on without one
        if (s && !(structure_only && s == ALPHA_SPARSE_STATUS_NOT_SUPPORTED)) return s;
        s = make_effective(handle, matA, opA, &eff);
        if (s) return s;
        plan = find_plan(matA, true, (int)alg, A, ncols);
    }
    const size_t kernel_need =
        plan ? asx_plan_workspace_bytes(plan) : asx_spmm_workspace_bytes((int)alg, vt, m, nnz, ncols);
    size_t b_bytes, c_bytes;
    spmm_copy_bytes(matA, opA, matB, opB, matC, &b_bytes, &c_bytes);
    const size_t need = b_bytes + c_bytes ? align256(kernel_need) + b_bytes + c_bytes : kernel_need;
    bool ok;
    void *ws = pick_workspace(handle, externalBuffer, need, &ok);
    if (!ok) {
        release_effective(handle, &eff);
        return ALPHA_SPARSE_STATUS_INVALID_POINTER;
    }
    void *stream = (void *)handle->stream;
    const bool beta_zero = vt == ALPHA_R_64F ? *(const double *)beta == 0.0 : *(const float *)beta == 0.0f;
    // row-major views of B and C: the caller's memory, or copies behind the kernel workspace
    const void *Bv = matB->values;
    int64_t ldb = matB->ld;
    void *Cv = matC->values;
    int64_t ldc = matC->ld;
    int rc = 0;
    if (b_bytes) {
        void *Bc = (char *)ws + align256(kernel_need);
        rc = asx_dense_transpose(vt, ncols, k, matB->values, matB->ld, Bc, ncols, stream);
        Bv = Bc;
        ldb = ncols;
    }
    if (!rc && c_bytes) {
        Cv = (char *)ws + align256(kernel_need) + b_bytes;
        ldc = ncols;
        if (!beta_zero) rc = asx_dense_transpose(vt, ncols, m, matC->values, matC->ld, Cv, ncols, stream);
    }
    if (!rc) {
        if (vt == ALPHA_R_64F)
            rc = asx_spmm_csr_f64(plan, (int)alg, m, k, nnz, ncols, *(const double *)alpha, A->row_data,
                                  A->col_data, (const double *)A->val_data, (const double *)Bv, ldb,
                                  *(const double *)beta, (double *)Cv, ldc, ws, kernel_need, stream);
        else
            rc = asx_spmm_csr_f32(plan, (int)alg, m, k, nnz, ncols, *(const float *)alpha, A->row_data,
                                  A->col_data, (const float *)A->val_data, (const float *)Bv, ldb,
                                  *(const float *)beta, (float *)Cv, ldc, ws, kernel_need, stream);
    }
    if (!rc && c_bytes) rc = asx_dense_transpose(vt, m, ncols, Cv, ncols, matC->values, matC->ld, stream);
    release_effective(handle, &eff);
    return st(rc);
}
