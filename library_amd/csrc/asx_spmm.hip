// CSR x dense SpMM for gfx950, C = alpha*A*B + beta*C with B (k x N) and C (m x N) row-major.
//
// Lanes of a wavefront are the 64 columns of a column tile, so every read of a row of B and
// every access to a row of C is one fully coalesced 256-byte (fp32) / 512-byte (fp64) access.
// The stored elements of A are read 64 at a time, one per lane, and broadcast lane by lane
// through v_readlane, which also makes the row address of B wave-uniform (scalar base +
// lane offset).
//
//   row   : one wave per (row, column tile).  Simple; long rows serialise.
//   merge : one wave per kSpmmSegment consecutive items of the merge path over
//           (row ends, stored elements): bounded work per wave whatever the row lengths.
//           Rows that end inside a segment are written by that segment, and so is a row
//           that starts in it and ends in the next; of a longer row the part that runs past
//           a segment end is kept as a carry row and added by an ordered pass afterwards.  No atomics (the reference's default SpMM,
//           hip/kernel/level3/alphasparse_spmm_csr_nnz_split.h:283-409, scales C in a
//           separate pass and joins segments with atomicAdd).
#include "asx_internal.hpp"

namespace asx {

template <typename T>
__device__ __forceinline__ T readlane_t(T v, int l);
template <>
__device__ __forceinline__ float readlane_t<float>(float v, int l)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l));
}
template <>
__device__ __forceinline__ double readlane_t<double>(double v, int l)
{
    int lo = __builtin_amdgcn_readlane(__double2loint(v), l);
    int hi = __builtin_amdgcn_readlane(__double2hiint(v), l);
    return __hiloint2double(hi, lo);
}

#ifndef ASX_SPMM_IN_FLIGHT
#define ASX_SPMM_IN_FLIGHT 8
#endif
constexpr int kSpmmInFlight = ASX_SPMM_IN_FLIGHT;  // rows of B a wave has in flight

// acc += sum over stored elements [k_begin, k_end) of one row: a * B[col, c]
template <typename T>
__device__ __forceinline__ T spmm_accumulate(T acc, int32_t k_begin, int32_t k_end, int lane, bool col_ok,
                                             int64_t c, const int32_t *__restrict__ col,
                                             const T *__restrict__ val, const T *__restrict__ B,
                                             int64_t ldb)
{
    for (int32_t k0 = k_begin; k0 < k_end; k0 += kWave) {
        const int32_t kk = k0 + lane;
        const int32_t cl = kk < k_end ? col[kk] : 0;
        const T vl = kk < k_end ? val[kk] : T(0);
        const int cnt = k_end - k0 < kWave ? k_end - k0 : kWave;
        // kSpmmInFlight rows of B at a time
        int j = 0;
        for (; j + kSpmmInFlight <= cnt; j += kSpmmInFlight) {
            int32_t cc[kSpmmInFlight];
            T b[kSpmmInFlight];
#pragma unroll
            for (int u = 0; u < kSpmmInFlight; ++u) cc[u] = __builtin_amdgcn_readlane(cl, j + u);
#pragma unroll
            for (int u = 0; u < kSpmmInFlight; ++u) b[u] = col_ok ? B[(int64_t)cc[u] * ldb + c] : T(0);
#pragma unroll
            for (int u = 0; u < kSpmmInFlight; ++u) acc = fma_t<T>(readlane_t<T>(vl, j + u), b[u], acc);
        }
        if (j < cnt) {  // the last, partial batch: all its loads are issued before the first use
            int32_t cc[kSpmmInFlight];
            T b[kSpmmInFlight];
#pragma unroll
            for (int u = 0; u < kSpmmInFlight; ++u) cc[u] = __builtin_amdgcn_readlane(cl, (j + u) & (kWave - 1));
#pragma unroll
            for (int u = 0; u < kSpmmInFlight; ++u) b[u] = (col_ok && j + u < cnt) ? B[(int64_t)cc[u] * ldb + c] : T(0);
#pragma unroll
            for (int u = 0; u < kSpmmInFlight; ++u)
                if (j + u < cnt) acc = fma_t<T>(readlane_t<T>(vl, (j + u) & (kWave - 1)), b[u], acc);
        }
    }
    return acc;
}

template <typename T>
__device__ __forceinline__ T scaled_out(T alpha, T acc, T beta, const T *C, int64_t idx)
{
    return beta == T(0) ? alpha * acc : fma_t<T>(alpha, acc, beta * C[idx]);
}

// ===========================================================================================
// row: one wave per (row, column tile)
// ===========================================================================================
template <typename T>
__global__ __launch_bounds__(kBlock) void k_spmm_row(int32_t m, int32_t ncols, T alpha,
                                                     const int32_t *__restrict__ row_ptr,
                                                     const int32_t *__restrict__ col,
                                                     const T *__restrict__ val, const T *__restrict__ B,
                                                     int64_t ldb, T beta, T *__restrict__ C,
                                                     int64_t ldc)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (row >= m) return;  // wave-uniform
    const int64_t c = (int64_t)blockIdx.y * kWave + lane;
    const bool col_ok = c < ncols;
    const int32_t s = __builtin_amdgcn_readfirstlane(row_ptr[row]);
    const int32_t e = __builtin_amdgcn_readfirstlane(row_ptr[row + 1]);
    T acc = spmm_accumulate<T>(T(0), s, e, lane, col_ok, c, col, val, B, ldb);
    if (col_ok) C[row * ldc + c] = scaled_out<T>(alpha, acc, beta, C, row * ldc + c);
}

template <typename T>
int launch_spmm_row(int32_t m, int32_t ncols, T alpha, const int32_t *row_ptr, const int32_t *col,
                    const T *val, const T *B, int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t s)
{
    if (m <= 0 || ncols <= 0) return ASX_STATUS_SUCCESS;
    dim3 grid((unsigned)ceil_div64(m, kBlock / kWave), (unsigned)ceil_div64(ncols, kWave));
    hipLaunchKernelGGL((k_spmm_row<T>), grid, dim3(kBlock), 0, s, m, ncols, alpha, row_ptr, col, val, B,
                       ldb, beta, C, ldc);
    return check_launch();
}

// ===========================================================================================
// merge: one wave per kSpmmSegment merge items
// ===========================================================================================
// Boundary g of the merge path lies between segments g-1 and g, at row xs[g], element ys[g].
// The row cut by a boundary is SHORT there if it starts inside segment g-1 and ends inside
// segment g: then the boundary moves to the end of that row, so segment g-1 takes the whole row
// (running up to kSpmmSegment items past its nominal end) and segment g starts after it.  Only
// rows long enough to cover a whole segment are still cut and leave carries.
__global__ __launch_bounds__(kBlock) void k_spmm_snap_splits(int32_t m, int32_t nseg,
                                                             const int32_t *__restrict__ row_ptr,
                                                             const int32_t *__restrict__ xs,
                                                             const int32_t *__restrict__ ys,
                                                             int32_t *__restrict__ xs_out,
                                                             int32_t *__restrict__ ys_out)
{
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g > nseg) return;
    int32_t x = xs[g], y = ys[g];
    if (g > 0 && g < nseg && x < m) {
        const int32_t b = row_ptr[x], e = row_ptr[x + 1];
        if (b < y && b >= ys[g - 1] && e <= ys[g + 1] && x < xs[g + 1]) {
            x += 1;
            y = e;
        }
    }
    xs_out[g] = x;
    ys_out[g] = y;
}

int launch_spmm_snap_splits(int32_t m, int32_t nnz, const int32_t *row_ptr, const int32_t *xs, const int32_t *ys,
                            int32_t *xs_out, int32_t *ys_out, hipStream_t s)
{
    const int32_t nseg = spmm_segments(m, nnz);
    hipLaunchKernelGGL(k_spmm_snap_splits, dim3((unsigned)ceil_div64((int64_t)nseg + 1, kBlock)), dim3(kBlock), 0, s, m,
                       nseg, row_ptr, xs, ys, xs_out, ys_out);
    return check_launch();
}

// A segment's stored elements and row ends, staged in LDS by the wave that owns the segment.
// After snapping a segment holds at most 2 * kSpmmSegment elements and kSpmmSegment + 1 row ends.
constexpr int kSegElems = 2 * kSpmmSegment;
constexpr int kSegRows = kSpmmSegment + kWave;

// acc += sum over staged elements [i0, i1) (positions relative to the segment start): a * B[col, c].
// The LDS reads are broadcasts (every lane reads the same address).
template <typename T>
__device__ __forceinline__ T spmm_accumulate_staged(T acc, int32_t i0, int32_t i1, bool col_ok, int64_t c,
                                                    const int32_t *s_col, const T *s_val,
                                                    const T *__restrict__ B, int64_t ldb)
{
    int32_t i = i0;
    for (; i + kSpmmInFlight <= i1; i += kSpmmInFlight) {
        int32_t cc[kSpmmInFlight];
        T a[kSpmmInFlight], b[kSpmmInFlight];
#pragma unroll
        for (int u = 0; u < kSpmmInFlight; ++u) {
            cc[u] = __builtin_amdgcn_readfirstlane(s_col[i + u]);
            a[u] = s_val[i + u];
        }
#pragma unroll
        for (int u = 0; u < kSpmmInFlight; ++u) b[u] = col_ok ? B[(int64_t)cc[u] * ldb + c] : T(0);
#pragma unroll
        for (int u = 0; u < kSpmmInFlight; ++u) acc = fma_t<T>(a[u], b[u], acc);
    }
    if (i < i1) {  // the last, partial batch: all its loads are issued before the first use
        int32_t cc[kSpmmInFlight];
        T a[kSpmmInFlight], b[kSpmmInFlight];
#pragma unroll
        for (int u = 0; u < kSpmmInFlight; ++u) {
            const int32_t iu = i + u < i1 ? i + u : i1 - 1;
            cc[u] = __builtin_amdgcn_readfirstlane(s_col[iu]);
            a[u] = s_val[iu];
        }
#pragma unroll
        for (int u = 0; u < kSpmmInFlight; ++u) b[u] = (col_ok && i + u < i1) ? B[(int64_t)cc[u] * ldb + c] : T(0);
#pragma unroll
        for (int u = 0; u < kSpmmInFlight; ++u)
            if (i + u < i1) acc = fma_t<T>(a[u], b[u], acc);
    }
    return acc;
}

// xs, ys: the snapped split points.  The wave first stages the segment's column indices, values
// and row ends in LDS (one round trip for all of them), so that the loads of B of one row after
// the other follow without waiting on row offsets or stored elements in between; the old value
// of a row of C (beta != 0) is requested before the row's loads of B.
template <typename T>
__global__ __launch_bounds__(kBlock) void k_spmm_merge(int32_t m, int32_t nnz, int32_t nseg,
                                                       int32_t ncols, T alpha,
                                                       const int32_t *__restrict__ row_ptr,
                                                       const int32_t *__restrict__ col,
                                                       const T *__restrict__ val,
                                                       const T *__restrict__ B, int64_t ldb, T beta,
                                                       T *__restrict__ C, int64_t ldc,
                                                       const int32_t *__restrict__ xs,
                                                       const int32_t *__restrict__ ys,
                                                       T *__restrict__ carry,
                                                       int32_t *__restrict__ carry_row)
{
    __shared__ int32_t s_col_all[kBlock / kWave][kSegElems];
    __shared__ T s_val_all[kBlock / kWave][kSegElems];
    __shared__ int32_t s_end_all[kBlock / kWave][kSegRows];
    const int lane = threadIdx.x & (kWave - 1);
    const int w = threadIdx.x / kWave;
    const int64_t seg = (int64_t)blockIdx.x * (kBlock / kWave) + w;
    if (seg >= nseg) return;  // wave-uniform
    const int64_t c = (int64_t)blockIdx.y * kWave + lane;
    const bool col_ok = c < ncols;
    const int32_t x0 = __builtin_amdgcn_readfirstlane(xs[seg]);
    const int32_t y0 = __builtin_amdgcn_readfirstlane(ys[seg]);
    const int32_t x1 = __builtin_amdgcn_readfirstlane(xs[seg + 1]);
    const int32_t y1 = __builtin_amdgcn_readfirstlane(ys[seg + 1]);
    const int32_t nel = y1 - y0, nrow = x1 - x0;

    if (nel <= kSegElems && nrow <= kSegRows) {
        int32_t *s_col = s_col_all[w];
        T *s_val = s_val_all[w];
        int32_t *s_end = s_end_all[w];
#pragma unroll
        for (int i = lane; i < kSegElems; i += kWave) {
            if (i < nel) {
                s_col[i] = col[y0 + i];
                s_val[i] = val[y0 + i];
            }
        }
#pragma unroll
        for (int i = lane; i < kSegRows; i += kWave)
            if (i < nrow) s_end[i] = row_ptr[x0 + 1 + i] - y0;
        // the staged data is private to this wave: order its LDS writes before its LDS reads
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        int32_t k = 0;
        for (int32_t r = 0; r < nrow; ++r) {  // rows this segment finishes
            const int32_t e = __builtin_amdgcn_readfirstlane(s_end[r]);
            const int64_t idx = (int64_t)(x0 + r) * ldc + c;
            const T c_old = (beta != T(0) && col_ok) ? C[idx] : T(0);
            const T acc = spmm_accumulate_staged<T>(T(0), k, e, col_ok, c, s_col, s_val, B, ldb);
            k = e;
            if (col_ok) C[idx] = beta == T(0) ? alpha * acc : fma_t<T>(alpha, acc, beta * c_old);
        }
        const bool has_tail = nel > k;  // row x1 continues past the segment end
        if (has_tail) {
            const T acc = spmm_accumulate_staged<T>(T(0), k, nel, col_ok, c, s_col, s_val, B, ldb);
            if (col_ok) carry[seg * ncols + c] = acc;
        }
        if (lane == 0 && blockIdx.y == 0) carry_row[seg] = has_tail ? x1 : -1;
        return;
    }

    // a segment too large to stage (cannot happen with snapped merge-path points; kept for safety)
    int32_t k = y0;
    T acc = T(0);
    for (int32_t row = x0; row < x1; ++row) {
        const int32_t e = __builtin_amdgcn_readfirstlane(row_ptr[row + 1]);
        acc = spmm_accumulate<T>(acc, k, e, lane, col_ok, c, col, val, B, ldb);
        k = e;
        if (col_ok) {
            const int64_t idx = (int64_t)row * ldc + c;
            C[idx] = scaled_out<T>(alpha, acc, beta, C, idx);
        }
        acc = T(0);
    }
    const bool has_tail = y1 > k;
    if (has_tail) {
        acc = spmm_accumulate<T>(T(0), k, y1, lane, col_ok, c, col, val, B, ldb);
        if (col_ok) carry[seg * ncols + c] = acc;
    }
    if (lane == 0 && blockIdx.y == 0) carry_row[seg] = has_tail ? x1 : -1;
}

// Every wave looks at kFixupSegs consecutive segments (one lane each) for the first segment of a run
// of segments that left carries for the same row; each such run is then summed by the whole wave
// (lanes = columns), one after the other: few segments per wave, because a run costs three or four
// dependent memory round trips and the runs of a wave are taken in turn (64 segments per wave left
// the pass with 2000 waves, each with five runs in a row: 22 us on the Zipf matrix, 19 us with 8; what
// remains is the longest rows, whose hundreds of carry rows one wave adds 64 at a time).  The run length
// comes from ballots over carry_row (64 segments per step), the carry rows are added in segment
// order with a counted, unrolled loop (many independent loads in flight; a loop that tests
// carry_row before every add would pay one memory round trip per segment).
constexpr int kFixupSegs = 8;
template <typename T>
__global__ __launch_bounds__(kBlock) void k_spmm_merge_fixup(int32_t m, int32_t nseg, int32_t ncols,
                                                             T alpha, const T *__restrict__ carry,
                                                             const int32_t *__restrict__ carry_row,
                                                             T *__restrict__ C, int64_t ldc)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t wave = ((int64_t)blockIdx.x * kBlock + threadIdx.x) / kWave;
    const int64_t t = wave * kFixupSegs + lane;
    int32_t my_row = -1;
    bool head = false;
    if (lane < kFixupSegs && t < nseg) {
        my_row = carry_row[t];
        head = my_row >= 0 && my_row < m && (t == 0 || carry_row[t - 1] != my_row);
    }
    unsigned long long todo = __ballot(head);
    while (todo) {  // wave-uniform
        const int src = __ffsll(todo) - 1;
        todo &= todo - 1;
        const int64_t seg = t - lane + src;
        const int32_t row = __shfl(my_row, src, kWave);
        int64_t len = 1;
        for (int64_t base = seg + 1;; base += kWave) {
            const int64_t idx = base + lane;
            const bool same = idx < nseg && carry_row[idx] == row;
            const unsigned long long mask = __ballot(same);
            const int n = mask == ~0ull ? kWave : __ffsll((unsigned long long)~mask) - 1;
            len += n;
            if (n < kWave) break;
        }
        for (int64_t c = lane; c < ncols; c += kWave) {
            const T *p = carry + seg * ncols + c;
            T sum = T(0);
            int64_t j = 0;
            for (; j + 64 <= len; j += 64) {  // a 50 000-element row leaves 390 carry rows
                T v[64];
#pragma unroll
                for (int u = 0; u < 64; ++u) v[u] = p[(j + u) * ncols];
#pragma unroll
                for (int u = 0; u < 64; ++u) sum += v[u];
            }
            for (; j + 8 <= len; j += 8) {
                T v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = p[(j + u) * ncols];
#pragma unroll
                for (int u = 0; u < 8; ++u) sum += v[u];
            }
            for (; j < len; ++j) sum += p[j * ncols];
            const int64_t idx = (int64_t)row * ldc + c;
            C[idx] = fma_t<T>(alpha, sum, C[idx]);
        }
    }
}

template <typename T>
int launch_spmm_merge(int32_t m, int32_t nnz, int32_t ncols, T alpha, const int32_t *row_ptr,
                      const int32_t *col, const T *val, const T *B, int64_t ldb, T beta, T *C,
                      int64_t ldc, const int32_t *xs, const int32_t *ys, T *carry, int32_t *carry_row,
                      hipStream_t s)
{
    if (m <= 0 || ncols <= 0) return ASX_STATUS_SUCCESS;
    const int32_t nseg = spmm_segments(m, nnz);
    dim3 grid((unsigned)ceil_div64(nseg, kBlock / kWave), (unsigned)ceil_div64(ncols, kWave));
    hipLaunchKernelGGL((k_spmm_merge<T>), grid, dim3(kBlock), 0, s, m, nnz, nseg, ncols, alpha, row_ptr,
                       col, val, B, ldb, beta, C, ldc, xs, ys, carry, carry_row);
    hipLaunchKernelGGL((k_spmm_merge_fixup<T>), dim3((unsigned)ceil_div64(ceil_div64(nseg, kFixupSegs), kBlock / kWave)),
                       dim3(kBlock), 0, s, m,
                       nseg, ncols, alpha, carry, carry_row, C, ldc);
    return check_launch();
}

#define ASX_INST(T)                                                                                  \
    template int launch_spmm_row<T>(int32_t, int32_t, T, const int32_t *, const int32_t *, const T *, \
                                    const T *, int64_t, T, T *, int64_t, hipStream_t);               \
    template int launch_spmm_merge<T>(int32_t, int32_t, int32_t, T, const int32_t *, const int32_t *, \
                                      const T *, const T *, int64_t, T, T *, int64_t, const int32_t *, \
                                      const int32_t *, T *, int32_t *, hipStream_t);
ASX_INST(float)
ASX_INST(double)
#undef ASX_INST

}  // namespace asx
