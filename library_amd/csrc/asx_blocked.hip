// Blocked SpMM variant for matrices with dense sub-blocks: A is re-tiled into 16x4 blocks
// (16 rows x 4 consecutive columns, zero filled) and each block meets the matching 4 rows of B
// in one MFMA (v_mfma_f32_16x16x4_f32 / v_mfma_f64_16x16x4_f64), 16 columns of C at a time.
//
// It pays only where blocks are dense: per stored element it streams 4/fill bytes of A (fp32)
// instead of 8, and reads 4 rows of B per block instead of one row per stored element
// (16/fill vs 256 bytes per element at N = 64).  fill = nnz / (64 * blocks); below about 1/8
// the merge kernel moves fewer bytes, so DEFAULT picks this variant only above that.
//
// The reference's counterpart (hip/kernel/level3/alphasparse_spmm_tc4csr.h:38-256) builds the
// blocks on the host through a dense ceil(M/16) x ceil(K/4) bitmap, keeps them in a global, and
// multiplies with Hygon `mmac` builtins.  Here the blocks are built on the device by sorting
// (block row, column quad) keys; they live in the plan.
//
// The zero fill of a block is multiplied with real rows of B: a non-finite value in a row of B
// that some row of the block does not reference reaches that row of C as NaN (0 * Inf), where a
// row-wise kernel would not have read it.  As for any padded block format, B must be finite.
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

#include "asx_internal.hpp"

namespace asx {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef double doublex4 __attribute__((ext_vector_type(4)));

// key = block row (28 bits) | column quad (30 bits) | row in block (4) | column in quad (2)
__global__ __launch_bounds__(kBlock) void k_block_keys(const int32_t *__restrict__ row_ptr,
                                                       const int32_t *__restrict__ col, int32_t m,
                                                       int32_t nnz, uint64_t *__restrict__ keys,
                                                       int32_t *__restrict__ idx)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    int32_t lo = 0, hi = m;  // row holding stored element i: largest r with row_ptr[r] <= i
    while (lo < hi) {
        const int32_t mid = lo + (hi - lo + 1) / 2;
        if (row_ptr[mid] <= i)
            lo = mid;
        else
            hi = mid - 1;
    }
    const uint32_t r = (uint32_t)lo, c = (uint32_t)col[i];
    keys[i] = ((uint64_t)(r >> 4) << 36) | ((uint64_t)(c >> 2) << 6) | ((uint64_t)(r & 15) << 2) | (c & 3);
    idx[i] = (int32_t)i;
}

__global__ __launch_bounds__(kBlock) void k_block_heads(const uint64_t *__restrict__ keys, int32_t nnz,
                                                        int32_t *__restrict__ head)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    head[i] = (i == 0 || (keys[i] >> 6) != (keys[i - 1] >> 6)) ? 1 : 0;
}

// Where every stored element goes: upd_src[i] = its position in A's arrays, upd_dst[i] = its slot
// in bval (lane order of the MFMA A operand), sign bit set when the element repeats the (row,
// column) of the element before it (CSR may hold duplicates; they are summed, as every other
// kernel here and the reference do).
__global__ __launch_bounds__(kBlock) void k_block_slots(const uint64_t *__restrict__ keys,
                                                        const int32_t *__restrict__ idx,
                                                        const int32_t *__restrict__ block_of, int32_t nnz,
                                                        uint64_t *__restrict__ bkey, int32_t *__restrict__ upd_src,
                                                        int64_t *__restrict__ upd_dst)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    const uint64_t key = keys[i];
    const int64_t b = block_of[i] - 1;  // inclusive scan of the head flags
    if (i == 0 || (key >> 6) != (keys[i - 1] >> 6)) bkey[b] = key >> 6;
    const int r16 = (int)((key >> 2) & 15), c4 = (int)(key & 3);
    const bool repeat = i > 0 && keys[i - 1] == key;
    upd_src[i] = idx[i];
    upd_dst[i] = (b * 64 + c4 * 16 + r16) | (repeat ? (int64_t)1 << 63 : 0);
}

// bval[slot] = sum of the values stored for that (row, column), in stored order
template <typename T>
__global__ __launch_bounds__(kBlock) void k_block_values(const int32_t *__restrict__ upd_src,
                                                         const int64_t *__restrict__ upd_dst, int32_t nnz,
                                                         const T *__restrict__ val, T *__restrict__ bval)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    const int64_t dst = upd_dst[i];
    if (dst < 0) return;  // summed by the first element of its run
    T sum = val[upd_src[i]];
    for (int64_t j = i + 1; j < nnz && upd_dst[j] < 0; ++j) sum += val[upd_src[j]];
    bval[dst] = sum;
}

__global__ __launch_bounds__(kBlock) void k_block_rows(const uint64_t *__restrict__ bkey, int32_t nblocks,
                                                       int32_t nbrows, int32_t *__restrict__ brow_ptr,
                                                       int32_t *__restrict__ bcol)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < nblocks) bcol[t] = (int32_t)(bkey[t] & ((1u << 30) - 1));
    if (t > nbrows) return;
    const uint64_t target = (uint64_t)t << 30;  // first block whose block row is >= t
    int32_t lo = 0, hi = nblocks;
    while (lo < hi) {
        const int32_t mid = (lo + hi) / 2;
        if (bkey[mid] < target)
            lo = mid + 1;
        else
            hi = mid;
    }
    brow_ptr[t] = lo;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_fill_zero(T *p, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        p[i] = T(0);
}

#define ASX_TRY(expr)                      \
    do {                                   \
        int _s = status_of(expr);          \
        if (_s) {                          \
            st = _s;                       \
            goto done;                     \
        }                                  \
    } while (0)

// Builds the blocked copy of A.  Synchronises the stream (reads the block count back).
template <typename T>
int build_blocked(int32_t m, int32_t k, int32_t nnz, const int32_t *row_ptr, const int32_t *col,
                  const T *val, BlockedMatrix *out, hipStream_t s)
{
    (void)k;
    int st = ASX_STATUS_SUCCESS;
    uint64_t *keys = nullptr, *keys2 = nullptr, *bkey = nullptr;
    int32_t *idx = nullptr, *idx2 = nullptr, *head = nullptr, *block_of = nullptr;
    void *tmp = nullptr;
    size_t tmp_sort = 0, tmp_scan = 0, tmp_bytes = 0;
    int32_t nblocks = 0;
    const int32_t nbrows = (int32_t)ceil_div64(m, 16);
    out->nbrows = nbrows;
    out->nblocks = 0;
    out->brow_ptr = nullptr;
    out->bcol = nullptr;
    out->bval = nullptr;
    out->upd_src = nullptr;
    out->upd_dst = nullptr;
    out->nnz = nnz;
    const unsigned g_nnz = (unsigned)ceil_div64(nnz > 0 ? nnz : 1, kBlock);
    if (nnz > 0) {
        ASX_TRY(hipMalloc((void **)&keys, sizeof(uint64_t) * (size_t)nnz));
        ASX_TRY(hipMalloc((void **)&keys2, sizeof(uint64_t) * (size_t)nnz));
        ASX_TRY(hipMalloc((void **)&idx, sizeof(int32_t) * (size_t)nnz));
        ASX_TRY(hipMalloc((void **)&idx2, sizeof(int32_t) * (size_t)nnz));
        ASX_TRY(hipMalloc((void **)&head, sizeof(int32_t) * (size_t)nnz));
        ASX_TRY(hipMalloc((void **)&block_of, sizeof(int32_t) * (size_t)nnz));
        ASX_TRY(rocprim::radix_sort_pairs(nullptr, tmp_sort, keys, keys2, idx, idx2, (size_t)nnz, 0u, (unsigned)64, s));
        ASX_TRY(rocprim::inclusive_scan(nullptr, tmp_scan, head, block_of, (size_t)nnz, rocprim::plus<int32_t>(), s));
        tmp_bytes = tmp_sort > tmp_scan ? tmp_sort : tmp_scan;
        ASX_TRY(hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1));
        hipLaunchKernelGGL(k_block_keys, dim3(g_nnz), dim3(kBlock), 0, s, row_ptr, col, m, nnz, keys, idx);
        ASX_TRY(rocprim::radix_sort_pairs(tmp, tmp_sort, keys, keys2, idx, idx2, (size_t)nnz, 0u, (unsigned)64, s));
        hipLaunchKernelGGL(k_block_heads, dim3(g_nnz), dim3(kBlock), 0, s, keys2, nnz, head);
        ASX_TRY(rocprim::inclusive_scan(tmp, tmp_scan, head, block_of, (size_t)nnz, rocprim::plus<int32_t>(), s));
        ASX_TRY(hipMemcpyAsync(&nblocks, block_of + (nnz - 1), sizeof(int32_t), hipMemcpyDeviceToHost, s));
        ASX_TRY(hipStreamSynchronize(s));
    }
    out->nblocks = nblocks;
    ASX_TRY(hipMalloc((void **)&out->brow_ptr, sizeof(int32_t) * ((size_t)nbrows + 1)));
    ASX_TRY(hipMalloc((void **)&out->bcol, sizeof(int32_t) * (size_t)(nblocks > 0 ? nblocks : 1)));
    ASX_TRY(hipMalloc((void **)&out->bval, sizeof(T) * 64 * (size_t)(nblocks > 0 ? nblocks : 1)));
    ASX_TRY(hipMalloc((void **)&bkey, sizeof(uint64_t) * (size_t)(nblocks > 0 ? nblocks : 1)));
    if (nblocks > 0) {
        ASX_TRY(hipMalloc((void **)&out->upd_src, sizeof(int32_t) * (size_t)nnz));
        ASX_TRY(hipMalloc((void **)&out->upd_dst, sizeof(int64_t) * (size_t)nnz));
        hipLaunchKernelGGL((k_fill_zero<T>), dim3(4096), dim3(kBlock), 0, s, (T *)out->bval, (int64_t)nblocks * 64);
        hipLaunchKernelGGL(k_block_slots, dim3(g_nnz), dim3(kBlock), 0, s, keys2, idx2, block_of, nnz, bkey,
                           out->upd_src, out->upd_dst);
        hipLaunchKernelGGL((k_block_values<T>), dim3(g_nnz), dim3(kBlock), 0, s, out->upd_src, out->upd_dst, nnz, val,
                           (T *)out->bval);
    }
    {
        const int64_t span = (int64_t)(nblocks > nbrows + 1 ? nblocks : nbrows + 1);
        hipLaunchKernelGGL(k_block_rows, dim3((unsigned)ceil_div64(span, kBlock)), dim3(kBlock), 0, s, bkey,
                           nblocks, nbrows, out->brow_ptr, out->bcol);
    }
    ASX_TRY(hipGetLastError());
    ASX_TRY(hipStreamSynchronize(s));
done:
    for (void *p : {(void *)keys, (void *)keys2, (void *)idx, (void *)idx2, (void *)head, (void *)block_of, tmp,
                    (void *)bkey})
        if (p) (void)hipFree(p);
    if (st) free_blocked(out);
    return st;
}
#undef ASX_TRY

void free_blocked(BlockedMatrix *b)
{
    if (b->brow_ptr) (void)hipFree(b->brow_ptr);
    if (b->bcol) (void)hipFree(b->bcol);
    if (b->bval) (void)hipFree(b->bval);
    if (b->upd_src) (void)hipFree(b->upd_src);
    if (b->upd_dst) (void)hipFree(b->upd_dst);
    b->brow_ptr = nullptr;
    b->bcol = nullptr;
    b->bval = nullptr;
    b->upd_src = nullptr;
    b->upd_dst = nullptr;
}

// Refreshes the blocks' values from A's (same sparsity pattern); the zero fill is untouched.
template <typename T>
int blocked_update_values(const BlockedMatrix *bm, const T *val, hipStream_t s)
{
    if (bm->nblocks <= 0 || bm->nnz <= 0) return ASX_STATUS_SUCCESS;
    hipLaunchKernelGGL((k_block_values<T>), dim3((unsigned)ceil_div64(bm->nnz, kBlock)), dim3(kBlock), 0, s, bm->upd_src,
                       bm->upd_dst, bm->nnz, val, (T *)bm->bval);
    return check_launch();
}

// ---- MFMA wrappers: A 16x4 (lane l: row l%16, k l/16), B 4x16 (lane l: k l/16, col l%16),
// ---- D 16x16 in 4 registers per lane, col l%16; the row of register r differs by type:
// ----   fp32: 4*(l/16) + r        fp64: 4*r + l/16
__device__ __forceinline__ floatx4 mfma16x16x4(float a, float b, floatx4 c)
{
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ doublex4 mfma16x16x4(double a, double b, doublex4 c)
{
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
}
template <typename T>
struct Acc4;
template <>
struct Acc4<float> {
    typedef floatx4 type;
    static __device__ __forceinline__ int row(int lane_hi, int r) { return lane_hi * 4 + r; }
};
template <>
struct Acc4<double> {
    typedef doublex4 type;
    static __device__ __forceinline__ int row(int lane_hi, int r) { return r * 4 + lane_hi; }
};

// One wave per (block row, group of 64 columns of C): 4 accumulators of 16x16.
template <typename T>
__global__ __launch_bounds__(kBlock) void k_spmm_blocked(int32_t m, int32_t kdim, int32_t ncols, int32_t nbrows,
                                                         T alpha, const int32_t *__restrict__ brow_ptr,
                                                         const int32_t *__restrict__ bcol,
                                                         const T *__restrict__ bval, const T *__restrict__ B,
                                                         int64_t ldb, T beta, T *__restrict__ C, int64_t ldc)
{
    typedef typename Acc4<T>::type acc_t;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t br = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (br >= nbrows) return;  // wave-uniform
    const int kq = lane >> 4, j16 = lane & 15;
    const int64_t n0 = (int64_t)blockIdx.y * 64;
    acc_t acc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[t] = acc_t{0, 0, 0, 0};
    const int32_t b0 = __builtin_amdgcn_readfirstlane(brow_ptr[br]);
    const int32_t b1 = __builtin_amdgcn_readfirstlane(brow_ptr[br + 1]);
    for (int32_t b = b0; b < b1; ++b) {
        const T a = bval[(int64_t)b * 64 + lane];
        const int64_t crow = (int64_t)__builtin_amdgcn_readfirstlane(bcol[b]) * 4 + kq;
        T bv[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int64_t n = n0 + t * 16 + j16;
            bv[t] = (crow < kdim && n < ncols) ? B[crow * ldb + n] : T(0);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t] = mfma16x16x4(a, bv[t], acc[t]);
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int64_t n = n0 + t * 16 + j16;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int64_t row = br * 16 + Acc4<T>::row(kq, r);
            if (row < m && n < ncols) {
                const int64_t idx = row * ldc + n;
                const T v = acc[t][r];
                C[idx] = beta == T(0) ? alpha * v : fma_t<T>(alpha, v, beta * C[idx]);
            }
        }
    }
}

template <typename T>
int launch_spmm_blocked(int32_t m, int32_t k, int32_t ncols, T alpha, const BlockedMatrix *bm, const T *B,
                        int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t s)
{
    if (m <= 0 || ncols <= 0) return ASX_STATUS_SUCCESS;
    dim3 grid((unsigned)ceil_div64(bm->nbrows, kBlock / kWave), (unsigned)ceil_div64(ncols, 64));
    hipLaunchKernelGGL((k_spmm_blocked<T>), grid, dim3(kBlock), 0, s, m, k, ncols, bm->nbrows, alpha, bm->brow_ptr,
                       bm->bcol, (const T *)bm->bval, B, ldb, beta, C, ldc);
    return check_launch();
}

template int build_blocked<float>(int32_t, int32_t, int32_t, const int32_t *, const int32_t *, const float *,
                                  BlockedMatrix *, hipStream_t);
template int build_blocked<double>(int32_t, int32_t, int32_t, const int32_t *, const int32_t *, const double *,
                                   BlockedMatrix *, hipStream_t);
template int blocked_update_values<float>(const BlockedMatrix *, const float *, hipStream_t);
template int blocked_update_values<double>(const BlockedMatrix *, const double *, hipStream_t);
template int launch_spmm_blocked<float>(int32_t, int32_t, int32_t, float, const BlockedMatrix *, const float *,
                                        int64_t, float, float *, int64_t, hipStream_t);
template int launch_spmm_blocked<double>(int32_t, int32_t, int32_t, double, const BlockedMatrix *, const double *,
                                         int64_t, double, double *, int64_t, hipStream_t);

}  // namespace asx
