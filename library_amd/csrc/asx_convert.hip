// Operand conversions around the CSR kernels, all on the device:
//   asx_csr_transpose   A -> A^T as zero-based CSR (what opA = TRANSPOSE runs on).  The reference
//                       does this on the host with two copies across PCIe per call and writes the
//                       result over the caller's arrays (hip/format/transpose_csr.h:9-71).
//   asx_csr_rebase      one-based row offsets / column indices -> zero-based copies.
//   asx_dense_transpose out[c][r] = in[r][c] for a strided dense matrix (column-major B and C of
//                       SpMM; the reference: hip/format/transpose_dn_mat.h:4-35, one element per
//                       thread with uncoalesced writes).
#include <rocprim/device/device_radix_sort.hpp>

#include "asx_internal.hpp"

namespace asx {

// key = (zero-based column << 32) | row, payload = position of the stored element.  A stable sort
// of the keys orders the elements of each column by row, duplicates in their stored order: the
// order the reference's counting transpose produces.
__global__ __launch_bounds__(kBlock) void k_transpose_keys(const int32_t *__restrict__ row_ptr,
                                                           const int32_t *__restrict__ col, int32_t m,
                                                           int32_t nnz, int32_t base,
                                                           uint64_t *__restrict__ keys,
                                                           int32_t *__restrict__ idx)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    const int32_t e = (int32_t)i + base;  // position in the numbering row_ptr uses
    int32_t lo = 0, hi = m;               // largest r with row_ptr[r] <= e
    while (lo < hi) {
        const int32_t mid = lo + (hi - lo + 1) / 2;
        if (row_ptr[mid] <= e)
            lo = mid;
        else
            hi = mid - 1;
    }
    keys[i] = ((uint64_t)(uint32_t)(col[i] - base) << 32) | (uint32_t)lo;
    idx[i] = (int32_t)i;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_transpose_apply(const uint64_t *__restrict__ keys,
                                                            const int32_t *__restrict__ idx,
                                                            const T *__restrict__ val, int32_t nnz,
                                                            int32_t *__restrict__ trow,
                                                            int32_t *__restrict__ col_t,
                                                            T *__restrict__ val_t)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    const uint64_t k = keys[i];
    trow[i] = (int32_t)(k >> 32);
    col_t[i] = (int32_t)(k & 0xFFFFFFFFu);
    val_t[i] = val[idx[i]];
}

// row_ptr_t[r] = first i with trow[i] >= r, r in [0, n]
__global__ __launch_bounds__(kBlock) void k_offsets_from_sorted(const int32_t *__restrict__ trow, int32_t nnz,
                                                                int32_t n, int32_t *__restrict__ row_ptr_t)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r > n) return;
    int32_t lo = 0, hi = nnz;
    while (lo < hi) {
        const int32_t mid = (lo + hi) / 2;
        if (trow[mid] < r)
            lo = mid + 1;
        else
            hi = mid;
    }
    row_ptr_t[r] = lo;
}

int launch_offsets_from_sorted(const int32_t *sorted, int32_t count, int32_t n, int32_t *out, hipStream_t s)
{
    hipLaunchKernelGGL(k_offsets_from_sorted, dim3((unsigned)ceil_div64((int64_t)n + 1, kBlock)), dim3(kBlock), 0, s,
                       sorted, count, n, out);
    return check_launch();
}

static int bits_for(int64_t v)
{
    int b = 1;
    while (b < 32 && ((int64_t)1 << b) < v) ++b;
    return b;
}

template <typename T>
int csr_transpose(int32_t m, int32_t n, int32_t nnz, int32_t base, const int32_t *row_ptr, const int32_t *col,
                  const T *val, int32_t *row_ptr_t, int32_t *col_t, T *val_t, hipStream_t s)
{
    int st = ASX_STATUS_SUCCESS;
    if (nnz == 0) {
        hipLaunchKernelGGL(k_offsets_from_sorted, dim3((unsigned)ceil_div64((int64_t)n + 1, kBlock)), dim3(kBlock), 0,
                           s, (const int32_t *)nullptr, 0, n, row_ptr_t);
        return check_launch();
    }
    uint64_t *keys = nullptr, *keys2 = nullptr;
    int32_t *idx = nullptr, *idx2 = nullptr, *trow = nullptr;
    void *tmp = nullptr;
    size_t tmp_bytes = 0;
    const unsigned grid = (unsigned)ceil_div64(nnz, kBlock);
    const int end_bit = 32 + bits_for(n);
#define ASX_TRY(expr)             \
    do {                          \
        st = status_of(expr);     \
        if (st) goto done;        \
    } while (0)
    ASX_TRY(hipMalloc((void **)&keys, sizeof(uint64_t) * (size_t)nnz));
    ASX_TRY(hipMalloc((void **)&keys2, sizeof(uint64_t) * (size_t)nnz));
    ASX_TRY(hipMalloc((void **)&idx, sizeof(int32_t) * (size_t)nnz));
    ASX_TRY(hipMalloc((void **)&idx2, sizeof(int32_t) * (size_t)nnz));
    ASX_TRY(hipMalloc((void **)&trow, sizeof(int32_t) * (size_t)nnz));
    ASX_TRY(rocprim::radix_sort_pairs(nullptr, tmp_bytes, keys, keys2, idx, idx2, (size_t)nnz, 0u, (unsigned)end_bit, s));
    ASX_TRY(hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1));
    hipLaunchKernelGGL(k_transpose_keys, dim3(grid), dim3(kBlock), 0, s, row_ptr, col, m, nnz, base, keys, idx);
    ASX_TRY(rocprim::radix_sort_pairs(tmp, tmp_bytes, keys, keys2, idx, idx2, (size_t)nnz, 0u, (unsigned)end_bit, s));
    hipLaunchKernelGGL((k_transpose_apply<T>), dim3(grid), dim3(kBlock), 0, s, keys2, idx2, val, nnz, trow, col_t,
                       val_t);
    hipLaunchKernelGGL(k_offsets_from_sorted, dim3((unsigned)ceil_div64((int64_t)n + 1, kBlock)), dim3(kBlock), 0, s,
                       trow, nnz, n, row_ptr_t);
    ASX_TRY(hipGetLastError());
    ASX_TRY(hipStreamSynchronize(s));
#undef ASX_TRY
done:
    for (void *p : {(void *)keys, (void *)keys2, (void *)idx, (void *)idx2, (void *)trow, tmp})
        if (p) (void)hipFree(p);
    return st;
}

__global__ __launch_bounds__(kBlock) void k_rebase(const int32_t *__restrict__ in, int64_t count, int32_t base,
                                                   int32_t *__restrict__ out)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count;
         i += (int64_t)gridDim.x * blockDim.x)
        out[i] = in[i] - base;
}

// 64 x 64 tiles through LDS: reads are coalesced along the input rows, writes along the output
// rows.  256 threads = 64 columns x 4 row groups, 16 rows each.
constexpr int kTrTile = 64;
template <typename T>
__global__ __launch_bounds__(kBlock) void k_dense_transpose(int64_t rows, int64_t cols, const T *__restrict__ in,
                                                            int64_t ld_in, T *__restrict__ out, int64_t ld_out)
{
    __shared__ T tile[kTrTile][kTrTile + 1];
    const int tx = threadIdx.x & (kTrTile - 1), ty = threadIdx.x / kTrTile;
    const int64_t r0 = (int64_t)blockIdx.y * kTrTile, c0 = (int64_t)blockIdx.x * kTrTile;
#pragma unroll 4
    for (int i = ty; i < kTrTile; i += kBlock / kTrTile) {
        const int64_t r = r0 + i, c = c0 + tx;
        if (r < rows && c < cols) tile[i][tx] = in[r * ld_in + c];
    }
    __syncthreads();
#pragma unroll 4
    for (int i = ty; i < kTrTile; i += kBlock / kTrTile) {
        const int64_t c = c0 + i, r = r0 + tx;
        if (r < rows && c < cols) out[c * ld_out + r] = tile[tx][i];
    }
}

template <typename T>
int dense_transpose(int64_t rows, int64_t cols, const T *in, int64_t ld_in, T *out, int64_t ld_out, hipStream_t s)
{
    if (rows == 0 || cols == 0) return ASX_STATUS_SUCCESS;
    const int64_t gx = ceil_div64(cols, kTrTile), gy = ceil_div64(rows, kTrTile);
    if (gy > 65535) {  // grid y limit: walk the rows in slabs
        const int64_t slab = (int64_t)65535 * kTrTile;
        for (int64_t r = 0; r < rows; r += slab) {
            const int64_t nr = rows - r < slab ? rows - r : slab;
            hipLaunchKernelGGL((k_dense_transpose<T>), dim3((unsigned)gx, (unsigned)ceil_div64(nr, kTrTile)),
                               dim3(kBlock), 0, s, nr, cols, in + r * ld_in, ld_in, out + r, ld_out);
        }
    } else {
        hipLaunchKernelGGL((k_dense_transpose<T>), dim3((unsigned)gx, (unsigned)gy), dim3(kBlock), 0, s, rows, cols,
                           in, ld_in, out, ld_out);
    }
    return check_launch();
}

}  // namespace asx

extern "C" int asx_csr_transpose(int value_type, int32_t m, int32_t n, int32_t nnz, int32_t idx_base,
                                 const int32_t *d_row_ptr, const int32_t *d_col, const void *d_val,
                                 int32_t *d_row_ptr_t, int32_t *d_col_t, void *d_val_t, void *stream)
{
    if (m < 0 || n < 0 || nnz < 0) return ASX_STATUS_INVALID_SIZE;
    if (idx_base != 0 && idx_base != 1) return ASX_STATUS_INVALID_VALUE;
    if (!d_row_ptr_t || (m > 0 && !d_row_ptr)) return ASX_STATUS_INVALID_POINTER;
    if (nnz > 0 && (!d_row_ptr || !d_col || !d_val || !d_col_t || !d_val_t)) return ASX_STATUS_INVALID_POINTER;
    if (value_type == ASX_R_64F)
        return asx::csr_transpose<double>(m, n, nnz, idx_base, d_row_ptr, d_col, (const double *)d_val, d_row_ptr_t,
                                          d_col_t, (double *)d_val_t, (hipStream_t)stream);
    if (value_type == ASX_R_32F)
        return asx::csr_transpose<float>(m, n, nnz, idx_base, d_row_ptr, d_col, (const float *)d_val, d_row_ptr_t,
                                         d_col_t, (float *)d_val_t, (hipStream_t)stream);
    return ASX_STATUS_NOT_SUPPORTED;
}

extern "C" int asx_csr_rebase(int32_t m, int32_t nnz, int32_t idx_base, const int32_t *d_row_ptr,
                              const int32_t *d_col, int32_t *d_row_ptr_out, int32_t *d_col_out, void *stream)
{
    if (m < 0 || nnz < 0) return ASX_STATUS_INVALID_SIZE;
    if (!d_row_ptr || !d_row_ptr_out || (nnz > 0 && (!d_col || !d_col_out))) return ASX_STATUS_INVALID_POINTER;
    hipStream_t s = (hipStream_t)stream;
    const auto grid_for = [](int64_t count) {
        int64_t g = asx::ceil_div64(count, asx::kBlock);
        return (unsigned)(g > 8192 ? 8192 : g);
    };
    hipLaunchKernelGGL(asx::k_rebase, dim3(grid_for((int64_t)m + 1)), dim3(asx::kBlock), 0, s, d_row_ptr,
                       (int64_t)m + 1, idx_base, d_row_ptr_out);
    if (nnz > 0)
        hipLaunchKernelGGL(asx::k_rebase, dim3(grid_for(nnz)), dim3(asx::kBlock), 0, s, d_col, (int64_t)nnz, idx_base,
                           d_col_out);
    return asx::check_launch();
}

extern "C" int asx_dense_transpose(int value_type, int64_t rows, int64_t cols, const void *d_in, int64_t ld_in,
                                   void *d_out, int64_t ld_out, void *stream)
{
    if (rows < 0 || cols < 0 || ld_in < cols || ld_out < rows) return ASX_STATUS_INVALID_SIZE;
    if (rows > 0 && cols > 0 && (!d_in || !d_out)) return ASX_STATUS_INVALID_POINTER;
    if (value_type == ASX_R_64F)
        return asx::dense_transpose<double>(rows, cols, (const double *)d_in, ld_in, (double *)d_out, ld_out,
                                            (hipStream_t)stream);
    if (value_type == ASX_R_32F)
        return asx::dense_transpose<float>(rows, cols, (const float *)d_in, ld_in, (float *)d_out, ld_out,
                                           (hipStream_t)stream);
    return ASX_STATUS_NOT_SUPPORTED;
}
