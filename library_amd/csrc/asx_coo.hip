// COO -> CSR on the device: row offsets from sorted row indices, and the (row, column) sort
// that callers run before it.  The reference does the first through hipSPARSE
// (hip/format/coo2csr.h:7-16) and the second on the host with qsort (hip/format/coo_order.h:24-43).
#include <rocprim/device/device_radix_sort.hpp>

#include "asx_internal.hpp"

namespace asx {

// row_ptr[r] = first i with row_ind[i] >= r (r in [0, m]); row_ptr[m] = nnz.
__global__ __launch_bounds__(kBlock) void k_coo2csr(const int32_t *__restrict__ row_ind, int32_t nnz,
                                                    int32_t m, int32_t *__restrict__ row_ptr)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r > m) return;
    int32_t lo = 0, hi = nnz;
    while (lo < hi) {
        const int32_t mid = (lo + hi) / 2;
        if (row_ind[mid] < r)
            lo = mid + 1;
        else
            hi = mid;
    }
    row_ptr[r] = lo;
}

__global__ __launch_bounds__(kBlock) void k_coo_keys(const int32_t *__restrict__ row, const int32_t *__restrict__ col,
                                                     int32_t nnz, uint64_t *__restrict__ keys,
                                                     int32_t *__restrict__ idx)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    keys[i] = ((uint64_t)(uint32_t)row[i] << 32) | (uint32_t)col[i];
    idx[i] = (int32_t)i;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_coo_apply(const uint64_t *__restrict__ keys, const int32_t *__restrict__ idx,
                                                      const T *__restrict__ val_in, int32_t nnz,
                                                      int32_t *__restrict__ row, int32_t *__restrict__ col,
                                                      T *__restrict__ val_out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    const uint64_t k = keys[i];
    row[i] = (int32_t)(k >> 32);
    col[i] = (int32_t)(k & 0xFFFFFFFFu);
    val_out[i] = val_in[idx[i]];
}

template <typename T>
int coo_sort(int32_t *row, int32_t *col, T *val, int32_t nnz, hipStream_t s)
{
    if (nnz <= 1) return ASX_STATUS_SUCCESS;
    int st = ASX_STATUS_SUCCESS;
    uint64_t *keys = nullptr, *keys2 = nullptr;
    int32_t *idx = nullptr, *idx2 = nullptr;
    T *val2 = nullptr;
    void *tmp = nullptr;
    size_t tmp_bytes = 0;
    const unsigned grid = (unsigned)ceil_div64(nnz, kBlock);
#define ASX_TRY(expr)             \
    do {                          \
        st = status_of(expr);     \
        if (st) goto done;        \
    } while (0)
    ASX_TRY(hipMalloc((void **)&keys, sizeof(uint64_t) * (size_t)nnz));
    ASX_TRY(hipMalloc((void **)&keys2, sizeof(uint64_t) * (size_t)nnz));
    ASX_TRY(hipMalloc((void **)&idx, sizeof(int32_t) * (size_t)nnz));
    ASX_TRY(hipMalloc((void **)&idx2, sizeof(int32_t) * (size_t)nnz));
    ASX_TRY(hipMalloc((void **)&val2, sizeof(T) * (size_t)nnz));
    ASX_TRY(rocprim::radix_sort_pairs(nullptr, tmp_bytes, keys, keys2, idx, idx2, (size_t)nnz, 0u, (unsigned)64, s));
    ASX_TRY(hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1));
    hipLaunchKernelGGL(k_coo_keys, dim3(grid), dim3(kBlock), 0, s, row, col, nnz, keys, idx);
    ASX_TRY(rocprim::radix_sort_pairs(tmp, tmp_bytes, keys, keys2, idx, idx2, (size_t)nnz, 0u, (unsigned)64, s));
    ASX_TRY(hipMemcpyAsync(val2, val, sizeof(T) * (size_t)nnz, hipMemcpyDeviceToDevice, s));
    hipLaunchKernelGGL((k_coo_apply<T>), dim3(grid), dim3(kBlock), 0, s, keys2, idx2, val2, nnz, row, col, val);
    ASX_TRY(hipGetLastError());
    ASX_TRY(hipStreamSynchronize(s));
#undef ASX_TRY
done:
    for (void *p : {(void *)keys, (void *)keys2, (void *)idx, (void *)idx2, (void *)val2, tmp})
        if (p) (void)hipFree(p);
    return st;
}

}  // namespace asx

extern "C" int asx_coo2csr(const int32_t *d_row_ind, int32_t nnz, int32_t m, int32_t *d_row_ptr, void *stream)
{
    if (nnz < 0 || m < 0) return ASX_STATUS_INVALID_SIZE;
    if (!d_row_ptr || (nnz > 0 && !d_row_ind)) return ASX_STATUS_INVALID_POINTER;
    hipLaunchKernelGGL(asx::k_coo2csr, dim3((unsigned)asx::ceil_div64((int64_t)m + 1, asx::kBlock)),
                       dim3(asx::kBlock), 0, (hipStream_t)stream, d_row_ind, nnz, m, d_row_ptr);
    return asx::check_launch();
}

extern "C" int asx_coo_sort(int value_type, int32_t *d_row_ind, int32_t *d_col_ind, void *d_val, int32_t nnz,
                            void *stream)
{
    if (nnz < 0) return ASX_STATUS_INVALID_SIZE;
    if (nnz > 0 && (!d_row_ind || !d_col_ind || !d_val)) return ASX_STATUS_INVALID_POINTER;
    if (value_type == ASX_R_64F)
        return asx::coo_sort<double>(d_row_ind, d_col_ind, (double *)d_val, nnz, (hipStream_t)stream);
    if (value_type == ASX_R_32F)
        return asx::coo_sort<float>(d_row_ind, d_col_ind, (float *)d_val, nnz, (hipStream_t)stream);
    return ASX_STATUS_NOT_SUPPORTED;
}
