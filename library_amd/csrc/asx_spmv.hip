// CSR SpMV kernels for gfx950 (wave64), y = alpha*A*x + beta*y.
//
//   vector : aligned sub-groups of a wavefront (2..64 lanes) own one row each; DPP reduction.
//   stream : a workgroup owns the rows that start inside a window of kStreamTile stored
//            elements; products are staged through LDS once (coalesced), rows are reduced
//            from LDS by 1..64 lanes each; the one row that may run past the window is
//            finished by the whole workgroup.  No atomics, no inter-workgroup traffic.
//   flat   : a workgroup owns exactly kFlatTile consecutive stored elements (aligned vector
//            loads, no metadata needed to start them); each thread walks its 4 products in
//            registers, rows spanning threads are joined by a segmented scan, rows spanning
//            tiles by the ordered carry pass.
//   merge  : a workgroup owns kMergeTile consecutive items of the merge path over
//            (row ends, stored elements); each thread walks exactly kMergeItemsPerThread
//            items; partial rows are joined by a segmented scan inside the workgroup and by
//            an ordered carry pass between workgroups.  No atomics: results do not depend on
//            scheduling.
//   (the column-sliced kernel for scattered columns lives in asx_sliced.hip)
//
// The reference's kernels for the same job (hip/kernel/level2/alphasparse_spmv_csr_vector.h,
// _flat.h, _merge_ginkgo.h, _adaptive.h) join partial rows with floating-point atomicAdd and
// recompute their split points in every call; neither is done here.
#include "asx_internal.hpp"

namespace asx {

// Tile order: tile = workgroup id.  Workgroups are dealt to the 8 XCDs round-robin, so
// neighbouring tiles run at the same time on different XCDs.  The alternative (each XCD walks
// one contiguous eighth of the tiles, so that x entries shared by neighbouring rows stay in
// one L2) measured 0-5 % slower on the benchmark workloads (5-point stencil 326 vs 312 us,
// power-law 586 vs 580 us, uniform 16/row equal): the shared x lines are served by the
// Infinity Cache either way, and eight far-apart streams cost more than they save.

// Streaming operands (stored elements, column indices, y) are touched once per call.  When
// they are larger than the Infinity Cache can hold from one call to the next, loading and
// storing them with the non-temporal hint keeps x cached (stencil: 312 -> 305 us); when the
// whole working set fits that cache the hint costs its hits (uniform 16/row fp32, 151 MB:
// 96 -> 114 us), so it is chosen per call from the size of the streamed arrays.
template <bool NT, typename T>
__device__ __forceinline__ T stream_load(const T *p)
{
    return NT ? __builtin_nontemporal_load(p) : *p;
}
template <bool NT, typename T>
__device__ __forceinline__ void stream_store(T *p, T v)
{
    if (NT)
        __builtin_nontemporal_store(v, p);
    else
        *p = v;
}

constexpr int64_t kNonTemporalAboveBytes = (int64_t)128 << 20;
inline bool use_nontemporal(int64_t nnz, size_t sv)
{
    return nnz * (int64_t)(sv + 4) > kNonTemporalAboveBytes;
}

template <typename T>
__device__ __forceinline__ T axpby_out(T alpha, T sum, T beta, const T *y, int64_t r)
{
    return beta == T(0) ? alpha * sum : fma_t<T>(alpha, sum, beta * y[r]);
}

// ===========================================================================================
// vector
// ===========================================================================================
template <typename T, int LANES>
__global__ __launch_bounds__(kBlock) void k_spmv_vector(int32_t m, T alpha,
                                                        const int32_t *__restrict__ row_ptr,
                                                        const int32_t *__restrict__ col,
                                                        const T *__restrict__ val,
                                                        const T *__restrict__ x, T beta,
                                                        T *__restrict__ y)
{
    const int lane = threadIdx.x & (LANES - 1);
    const int64_t row = ((int64_t)blockIdx.x * kBlock + threadIdx.x) / LANES;
    T sum = T(0);
    if (row < m) {
        const int32_t e = row_ptr[row + 1];
        int32_t k = row_ptr[row] + lane;
        // two independent chains per lane keep more gathers in flight on long rows
        T s0 = T(0), s1 = T(0);
        for (; k + LANES < e; k += 2 * LANES) {
            s0 = fma_t<T>(val[k], x[col[k]], s0);
            s1 = fma_t<T>(val[k + LANES], x[col[k + LANES]], s1);
        }
        if (k < e) s0 = fma_t<T>(val[k], x[col[k]], s0);
        sum = s0 + s1;
    }
    sum = group_sum<LANES>(sum);  // all lanes stay active for the cross-lane moves
    if (row < m && lane == 0) y[row] = axpby_out<T>(alpha, sum, beta, y, row);
}

template <typename T>
int launch_spmv_vector(int32_t m, int32_t nnz, T alpha, const int32_t *row_ptr, const int32_t *col,
                       const T *val, const T *x, T beta, T *y, hipStream_t s)
{
    if (m <= 0) return ASX_STATUS_SUCCESS;
    const double mean = (double)nnz / (double)m;
#define ASX_VEC(L)                                                                                   \
    hipLaunchKernelGGL((k_spmv_vector<T, L>), dim3((unsigned)ceil_div64((int64_t)m * L, kBlock)),    \
                       dim3(kBlock), 0, s, m, alpha, row_ptr, col, val, x, beta, y)
    if (mean <= 2.0)
        ASX_VEC(2);
    else if (mean <= 4.0)
        ASX_VEC(4);
    else if (mean <= 8.0)
        ASX_VEC(8);
    else if (mean <= 16.0)
        ASX_VEC(16);
    else if (mean <= 32.0)
        ASX_VEC(32);
    else
        ASX_VEC(64);
#undef ASX_VEC
    return check_launch();
}

// ===========================================================================================
// stream
// ===========================================================================================
// LDS index with one pad slot per 32 entries: rows whose length is a multiple of 16 or 32
// would otherwise put every lane of a wave on the same few banks.
__device__ __forceinline__ int pad32(int j) { return j + (j >> 5); }
constexpr int kStreamLds = kStreamTile + kStreamTile / 32 + 1;
constexpr int kStreamRowCap = kStreamTile / 2;  // row pointers kept in LDS per block (+1)

// Row pointer i of the block (relative to the block's first stored element): from LDS for the
// first kStreamRowCap+1 rows, from memory for the (rare) rows past that.
__device__ __forceinline__ int32_t stream_rp(const int32_t *s_rp, const int32_t *__restrict__ row_ptr,
                                             int32_t r0, int32_t a, int i)
{
    return i <= kStreamRowCap ? s_rp[i] : row_ptr[r0 + i] - a;
}

template <int G, bool NT, typename T>
__device__ __forceinline__ void stream_reduce_rows(const T *s_prod, const int32_t *s_rp, int32_t r0,
                                                   int32_t nrows, int32_t a, int32_t n1, T extra,
                                                   T alpha, T beta, T y_first, bool y_first_ok,
                                                   const int32_t *__restrict__ row_ptr,
                                                   T *__restrict__ y)
{
    const int lane = threadIdx.x & (G - 1);
    const int rows_per_pass = kBlock / G;
    // every lane runs the same number of passes so the cross-lane moves see full waves
    for (int base = 0; base < nrows; base += rows_per_pass) {
        const int g = base + (int)threadIdx.x / G;
        T sum = T(0);
        if (g < nrows) {
            const int32_t s = stream_rp(s_rp, row_ptr, r0, a, g);
            int32_t e = stream_rp(s_rp, row_ptr, r0, a, g + 1);
            e = e < n1 ? e : n1;
            for (int32_t j = s + lane; j < e; j += G) sum += s_prod[pad32(j)];
        }
        sum = group_sum<G>(sum);
        if (g < nrows && lane == 0) {
            const int64_t r = (int64_t)r0 + g;
            if (g == nrows - 1) sum += extra;
            T out;
            if (beta == T(0))
                out = alpha * sum;
            else
                out = fma_t<T>(alpha, sum, beta * ((base == 0 && y_first_ok) ? y_first : y[r]));
            stream_store<NT>(y + r, out);
        }
    }
}

template <typename T, bool NT>
__global__ __launch_bounds__(kBlock) void k_spmv_stream(int32_t m, int32_t nblocks, T alpha,
                                                        const int32_t *__restrict__ row_ptr,
                                                        const int32_t *__restrict__ col,
                                                        const T *__restrict__ val,
                                                        const T *__restrict__ x, T beta,
                                                        T *__restrict__ y,
                                                        const int32_t *__restrict__ blocks)
{
    __shared__ T s_prod[kStreamLds];
    __shared__ int32_t s_rp[kStreamRowCap + 1];
    __shared__ T s_part[kBlock / kWave];
    const int t = blockIdx.x;
    // blocks[2t] = first row of block t, blocks[2t+1] = its first stored element: one hop
    const int2 lo = reinterpret_cast<const int2 *>(blocks)[t];
    const int2 hi = reinterpret_cast<const int2 *>(blocks)[t + 1];
    const int32_t r0 = lo.x, r1 = hi.x;
    const int32_t nrows = r1 - r0;
    if (nrows <= 0) return;
    const int32_t a = lo.y;
    const int32_t bend = hi.y;
    const int32_t c1 = bend - a > kStreamTile ? a + kStreamTile : bend;
    const int32_t n1 = c1 - a;
    const int tid = threadIdx.x;

    // ---- issue every load of the block up front: stored elements, row pointers, y ----
    constexpr int IPT = kStreamTile / kBlock;
    int32_t cj[IPT];
    T vj[IPT];
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
        const int j = tid + i * kBlock;
        cj[i] = j < n1 ? stream_load<NT>(col + (int64_t)a + j) : 0;
    }
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
        const int j = tid + i * kBlock;
        vj[i] = j < n1 ? stream_load<NT>(val + (int64_t)a + j) : T(0);
    }
    constexpr int RPI = (kStreamRowCap + 1 + kBlock - 1) / kBlock;
    const int32_t rp_n = nrows < kStreamRowCap ? nrows : kStreamRowCap;  // pointers 0..rp_n
    int32_t rpv[RPI];
#pragma unroll
    for (int i = 0; i < RPI; ++i) {
        const int j = tid + i * kBlock;
        rpv[i] = j <= rp_n ? row_ptr[r0 + j] : 0;
    }
    // the row this thread writes in the first reduction pass (lanes-per-row is decided below
    // from nrows alone, so the mapping is known here)
    int g_shift = 0;
    if (nrows <= 128) g_shift = nrows > 64 ? 1 : nrows > 32 ? 2 : nrows > 16 ? 3 : nrows > 8 ? 4 : nrows > 4 ? 5 : 6;
    const int my_g = tid >> g_shift;
    const bool y_first_ok = beta != T(0) && my_g < nrows && (tid & ((1 << g_shift) - 1)) == 0;
    const T y_first = y_first_ok ? y[(int64_t)r0 + my_g] : T(0);

#pragma unroll
    for (int i = 0; i < IPT; ++i) {
        const int j = tid + i * kBlock;
        if (j < n1) s_prod[pad32(j)] = vj[i] * x[cj[i]];
    }
#pragma unroll
    for (int i = 0; i < RPI; ++i) {
        const int j = tid + i * kBlock;
        if (j <= rp_n) s_rp[j] = rpv[i] - a;
    }

    // ---- the last row may run past the window: finish it with the whole workgroup ----
    T extra = T(0);
    if (bend > c1) {  // uniform over the workgroup
        T p0 = T(0), p1 = T(0);
        int64_t k = (int64_t)c1 + tid;
        for (; k + kBlock < bend; k += 2 * kBlock) {
            p0 = fma_t<T>(val[k], x[col[k]], p0);
            p1 = fma_t<T>(val[k + kBlock], x[col[k + kBlock]], p1);
        }
        if (k < bend) p0 = fma_t<T>(val[k], x[col[k]], p0);
        T p = group_sum<kWave>(p0 + p1);
        if ((tid & (kWave - 1)) == 0) s_part[tid / kWave] = p;
    }
    __syncthreads();
    if (bend > c1) extra = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);

#define ASX_RED(G) \
    stream_reduce_rows<G, NT, T>(s_prod, s_rp, r0, nrows, a, n1, extra, alpha, beta, y_first, y_first_ok, row_ptr, y)
    switch (g_shift) {
    case 0: ASX_RED(1); break;
    case 1: ASX_RED(2); break;
    case 2: ASX_RED(4); break;
    case 3: ASX_RED(8); break;
    case 4: ASX_RED(16); break;
    case 5: ASX_RED(32); break;
    default: ASX_RED(64); break;
    }
#undef ASX_RED
}

// Row blocks of the stream kernel, as (row, row_ptr[row]) pairs: pair t = first row whose first
// stored element lies at or after t*kStreamTile (t < nb), pair nb = (m, nnz),
// nb = max(1, ceil(nnz / kStreamTile)).  2*(nb+1) int32, 8-byte aligned.
__global__ __launch_bounds__(kBlock) void k_stream_row_blocks(const int32_t *__restrict__ row_ptr,
                                                              int32_t m, int32_t nb,
                                                              int32_t *__restrict__ blocks)
{
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t > nb) return;
    if (t == nb) {
        blocks[2 * nb] = m;
        blocks[2 * nb + 1] = row_ptr[m];
        return;
    }
    const int64_t target = t * kStreamTile;
    int32_t lo = 0, hi = m;  // first r in [0,m] with row_ptr[r] >= target
    while (lo < hi) {
        int32_t mid = (lo + hi) / 2;
        if ((int64_t)row_ptr[mid] < target)
            lo = mid + 1;
        else
            hi = mid;
    }
    blocks[2 * t] = lo;
    blocks[2 * t + 1] = row_ptr[lo];
}

int launch_stream_row_blocks(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t *d_blocks,
                             hipStream_t s)
{
    int32_t nb = stream_blocks(nnz);
    if (nb < 1) nb = 1;
    hipLaunchKernelGGL(k_stream_row_blocks, dim3((unsigned)ceil_div64((int64_t)nb + 1, kBlock)),
                       dim3(kBlock), 0, s, d_row_ptr, m, nb, d_blocks);
    return check_launch();
}

template <typename T>
int launch_spmv_stream(int32_t m, int32_t nnz, T alpha, const int32_t *row_ptr, const int32_t *col,
                       const T *val, const T *x, T beta, T *y, const int32_t *blocks, hipStream_t s)
{
    if (m <= 0) return ASX_STATUS_SUCCESS;
    int32_t nb = stream_blocks(nnz);
    if (nb < 1) nb = 1;
    if (use_nontemporal(nnz, sizeof(T)))
        hipLaunchKernelGGL((k_spmv_stream<T, true>), dim3((unsigned)nb), dim3(kBlock), 0, s, m, nb, alpha,
                           row_ptr, col, val, x, beta, y, blocks);
    else
        hipLaunchKernelGGL((k_spmv_stream<T, false>), dim3((unsigned)nb), dim3(kBlock), 0, s, m, nb, alpha,
                           row_ptr, col, val, x, beta, y, blocks);
    return check_launch();
}

// ===========================================================================================
// merge path
// ===========================================================================================
template <typename T, bool NT>
__global__ __launch_bounds__(kBlock) void k_spmv_merge(int32_t m, int32_t nnz, int32_t ntiles, T alpha,
                                                       const int32_t *__restrict__ row_ptr,
                                                       const int32_t *__restrict__ col,
                                                       const T *__restrict__ val,
                                                       const T *__restrict__ x, T beta,
                                                       T *__restrict__ y,
                                                       const int32_t *__restrict__ xs,
                                                       const int32_t *__restrict__ ys,
                                                       T *__restrict__ carry)
{
    constexpr int IPT = kMergeItemsPerThread;
    // s_val[0..nz) = products, s_val[nz..nz+nr) = finished row sums (nz + nr <= kMergeTile)
    __shared__ T s_val[kMergeTile];
    __shared__ int32_t s_rend[kMergeTile + 1];
    __shared__ T s_wv[kBlock / kWave];
    __shared__ int32_t s_wk[kBlock / kWave];

    const int b = blockIdx.x;
    const int tid = threadIdx.x;
    const int32_t x0 = xs[b], y0 = ys[b], x1 = xs[b + 1], y1 = ys[b + 1];
    const int32_t nr = x1 - x0, nz = y1 - y0, total = nr + nz;

    // ---- stage: stored elements first (the long-latency part), then row ends ----
    int32_t cj[IPT];
    T vj[IPT];
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
        const int j = tid + i * kBlock;
        cj[i] = j < nz ? stream_load<NT>(col + (int64_t)y0 + j) : 0;
        vj[i] = j < nz ? stream_load<NT>(val + (int64_t)y0 + j) : T(0);
    }
    for (int i = tid; i <= nr; i += kBlock) {
        const int32_t r = x0 + i;
        s_rend[i] = (r < m ? row_ptr[r + 1] : nnz) - y0;
    }
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
        const int j = tid + i * kBlock;
        if (j < nz) s_val[j] = vj[i] * x[cj[i]];
    }
    __syncthreads();

    // ---- this thread's start on the tile's merge path ----
    int32_t diag = tid * IPT;
    if (diag > total) diag = total;
    int32_t lo = diag - nz > 0 ? diag - nz : 0;
    int32_t hi = diag < nr ? diag : nr;
    while (lo < hi) {
        const int32_t p = (lo + hi) >> 1;
        if (s_rend[p] < diag - p)
            lo = p + 1;
        else
            hi = p;
    }
    int32_t row = lo, k = diag - lo;
    const int32_t first_row = row;
    int32_t cur_end = s_rend[row];
    bool emitted = false;
    T run = T(0);
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
        if (diag + i < total) {
            if (k < cur_end) {
                run += s_val[k];
                ++k;
            } else {
                s_val[nz + row] = run;
                emitted = true;
                run = T(0);
                ++row;
                cur_end = s_rend[row];
            }
        }
    }

    // ---- join rows that span threads: segmented scan of (row in progress, partial) ----
    const int lane = tid & (kWave - 1), w = tid / kWave;
    const T incl = wave_segscan_incl<T>(row, run);
    const int32_t k0 = __shfl(row, 0, kWave);
    if (lane == kWave - 1) {
        s_wk[w] = row;
        s_wv[w] = incl;
    }
    __syncthreads();
    int32_t pk = -1;
    T pv = T(0);
    for (int j = 0; j < w; ++j) {
        const int32_t kj = s_wk[j];
        const T vjj = s_wv[j];
        if (kj == pk)
            pv += vjj;
        else {
            pk = kj;
            pv = vjj;
        }
    }
    const int32_t up_k = __shfl_up(row, 1, kWave);
    T carry_in = __shfl_up(incl, 1, kWave);
    if (lane == 0) {
        carry_in = (w > 0 && pk == first_row) ? pv : T(0);
    } else {
        if (up_k != first_row) carry_in = T(0);  // cannot happen on a consistent path; keeps it safe
        if (up_k == k0 && pk == up_k) carry_in += pv;
    }
    if (emitted) s_val[nz + first_row] += carry_in;
    if (tid == kBlock - 1) {
        T out = incl;
        if (row == k0 && pk == row) out += pv;
        carry[b] = out;  // partial of row x1 gathered in this tile (0 when none of it is here)
    }
    __syncthreads();

    // ---- finished rows, coalesced ----
    for (int i = tid; i < nr; i += kBlock) {
        const int64_t r = (int64_t)x0 + i;
        stream_store<NT>(y + r, axpby_out<T>(alpha, s_val[nz + i], beta, y, r));
    }
}

// Adds the carries to the rows that continue past a tile end.  One thread per tile.  A tile
// whose open row ends in the very next tile (the common case) is settled by its thread alone.
// A run of several tiles that end inside the same row is settled by the whole wave of the run's
// first tile: it finds the run length with ballots over xs (64 tiles per step), sums the run's
// carries lane-parallel in a fixed order and adds the total to y.  (A single thread walking the
// run pays one memory round trip per tile: 100 round trips for a 200 000-element row.)
template <typename T>
__device__ __forceinline__ void fixup_tiles(int64_t t, int32_t m, int32_t ntiles, T alpha,
                                            const int32_t *__restrict__ xs, const T *__restrict__ carry,
                                            T *__restrict__ y)
{
    const int lane = threadIdx.x & (kWave - 1);
    int32_t row = m;
    bool first = false, run = false;
    if (t < ntiles) {
        row = xs[t + 1];
        first = row < m && (t == 0 || xs[t] != row);
        run = first && t + 1 < ntiles && xs[t + 2] == row;
    }
    if (first && !run) {
        const T c = carry[t];
        if (c != T(0)) y[row] = fma_t<T>(alpha, c, y[row]);
    }
    unsigned long long todo = __ballot(run);
    while (todo) {  // wave-uniform
        const int src = __ffsll(todo) - 1;
        todo &= todo - 1;
        const int64_t b = t - lane + src;
        const int32_t r = __shfl(row, src, kWave);
        int64_t len = 1;
        for (int64_t base = b + 1;; base += kWave) {
            const int64_t j = base + lane;
            const bool same = j < ntiles && xs[j + 1] == r;
            const unsigned long long mask = __ballot(same);
            const int n = mask == ~0ull ? kWave : __ffsll((unsigned long long)~mask) - 1;
            len += n;
            if (n < kWave) break;
        }
        T part = T(0);
        for (int64_t j = lane; j < len; j += kWave) part += carry[b + j];
        const T sum = group_sum<kWave>(part);
        if (lane == 0 && sum != T(0)) y[r] = fma_t<T>(alpha, sum, y[r]);
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_spmv_merge_fixup(int32_t m, int32_t ntiles, T alpha,
                                                             const int32_t *__restrict__ xs,
                                                             const T *__restrict__ carry,
                                                             T *__restrict__ y)
{
    fixup_tiles<T>((int64_t)blockIdx.x * kBlock + threadIdx.x, m, ntiles, alpha, xs, carry, y);
}

template <typename T>
int launch_spmv_merge(int32_t m, int32_t nnz, T alpha, const int32_t *row_ptr, const int32_t *col,
                      const T *val, const T *x, T beta, T *y, const int32_t *xs, const int32_t *ys,
                      T *carry, hipStream_t s)
{
    if (m <= 0) return ASX_STATUS_SUCCESS;
    const int32_t ntiles = merge_tiles(m, nnz);
    if (use_nontemporal(nnz, sizeof(T)))
        hipLaunchKernelGGL((k_spmv_merge<T, true>), dim3((unsigned)ntiles), dim3(kBlock), 0, s, m, nnz,
                           ntiles, alpha, row_ptr, col, val, x, beta, y, xs, ys, carry);
    else
        hipLaunchKernelGGL((k_spmv_merge<T, false>), dim3((unsigned)ntiles), dim3(kBlock), 0, s, m, nnz,
                           ntiles, alpha, row_ptr, col, val, x, beta, y, xs, ys, carry);
    hipLaunchKernelGGL((k_spmv_merge_fixup<T>), dim3((unsigned)ceil_div64(ntiles, kBlock)),
                       dim3(kBlock), 0, s, m, ntiles, alpha, xs, carry, y);
    return check_launch();
}

// ===========================================================================================
// flat: tiles of exactly kFlatTile stored elements
// ===========================================================================================
// Tile t owns stored elements [t*kFlatTile, (t+1)*kFlatTile): its loads need no metadata and are
// 16-byte vector loads on aligned addresses.  seg_row[t] (the row holding the tile's first
// element, asx_nnz_split_rows) arrives while the loads are in flight.  Each thread keeps its 4
// consecutive products in registers and walks them against the tile's row ends (LDS); rows that
// end inside a thread are stored to an LDS row buffer, rows that span threads are joined by a
// segmented scan, the row still open at the tile end leaves a carry that the same ordered pass
// as the merge kernel's adds afterwards.  Work per tile is bounded whatever the row lengths;
// a tile that meets more rows than the LDS row buffer holds (a flood of empty rows) takes a
// slower thread-per-row path.
constexpr int kFlatItemsPerThread = kFlatTile / kBlock;
static_assert(kFlatItemsPerThread == 4, "the vector loads below read 4 elements per thread");
constexpr int kFlatRowCap = 1024;  // rows of one tile kept in LDS
#ifndef ASX_FLAT_TPG
#define ASX_FLAT_TPG 1
#endif
constexpr int kFlatTilesPerGroup = ASX_FLAT_TPG;

template <typename T>
struct Vec4;
template <>
struct Vec4<float> {
    template <bool NT>
    static __device__ __forceinline__ void load(const float *p, float v[4])
    {
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        const f32x4 *q = reinterpret_cast<const f32x4 *>(p);
        const f32x4 t = NT ? __builtin_nontemporal_load(q) : *q;
        v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
    }
};
template <>
struct Vec4<double> {
    template <bool NT>
    static __device__ __forceinline__ void load(const double *p, double v[4])
    {
        typedef double f64x2 __attribute__((ext_vector_type(2)));
        const f64x2 *q = reinterpret_cast<const f64x2 *>(p);
        const f64x2 a = NT ? __builtin_nontemporal_load(q) : q[0];
        const f64x2 b = NT ? __builtin_nontemporal_load(q + 1) : q[1];
        v[0] = a.x, v[1] = a.y, v[2] = b.x, v[3] = b.y;
    }
};

// Row mode of the flat kernel: aligned groups of G lanes own one row each.
template <int G, bool NT, typename T>
__device__ __forceinline__ void flat_reduce_rows(const T *s_prod, const int32_t *s_rend, bool fits, int32_t rs,
                                                 int32_t rcount, int32_t nwritten, int64_t base, int32_t n1,
                                                 int t, T alpha, T beta, const int32_t *__restrict__ row_ptr,
                                                 T *__restrict__ y, T *__restrict__ carry)
{
    const int lane = threadIdx.x & (G - 1);
    const int rows_per_pass = kBlock / G;
    for (int first = 0; first < rcount; first += rows_per_pass) {  // same trip count for every lane
        const int i = first + (int)threadIdx.x / G;
        T sum = T(0);
        if (i < rcount) {
            int32_t s, e;
            if (fits) {
                s = i > 0 ? s_rend[i - 1] : 0;
                e = s_rend[i];
            } else {
                const int64_t gs = (int64_t)row_ptr[rs + i] - base, ge = (int64_t)row_ptr[rs + i + 1] - base;
                s = gs < 0 ? 0 : (int32_t)gs;
                e = ge > n1 ? n1 : (int32_t)ge;
            }
            s = s < 0 ? 0 : s;
            e = e > n1 ? n1 : e;
            for (int32_t k = s + lane; k < e; k += G) sum += s_prod[k + (k >> 5)];
        }
        sum = group_sum<G>(sum);
        if (i < rcount && lane == 0) {
            const int64_t r = (int64_t)rs + i;
            if (i < nwritten)
                stream_store<NT>(y + r, axpby_out<T>(alpha, sum, beta, y, r));
            else
                carry[t] = sum;
        }
    }
}

// Rows no longer than this are summed one thread per row from LDS; a tile that meets a longer
// row takes the register walk, whose cost does not depend on row lengths.
constexpr int kFlatRowModeMaxLen = 32;

// The 4 consecutive stored elements of thread `tid` in tile t.
template <typename T, bool VEC, bool NT>
__device__ __forceinline__ void flat_load(int t, int32_t nnz, const int32_t *__restrict__ col,
                                          const T *__restrict__ val, int32_t c[4], T p[4])
{
    const int64_t base = (int64_t)t * kFlatTile;
    const int32_t n1 = nnz - base < kFlatTile ? (int32_t)(nnz - base) : kFlatTile;
    const int32_t k0 = threadIdx.x * 4;
    if (VEC && n1 == kFlatTile) {
        typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
        const i32x4 *cp = reinterpret_cast<const i32x4 *>(col + base + k0);
        const i32x4 cc = NT ? __builtin_nontemporal_load(cp) : *cp;
        c[0] = cc.x, c[1] = cc.y, c[2] = cc.z, c[3] = cc.w;
        Vec4<T>::template load<NT>(val + base + k0, p);
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            c[j] = k0 + j < n1 ? col[base + k0 + j] : 0;
            p[j] = k0 + j < n1 ? val[base + k0 + j] : T(0);
        }
    }
}

template <typename T>
struct FlatShared {
    int32_t rend[kFlatRowCap + 1];
    T out[kFlatRowCap + 1];
    T prod[kFlatTile + kFlatTile / 32];  // row mode (padded against bank conflicts)
    T wv[kBlock / kWave];
    int32_t wk[kBlock / kWave];
};

// One tile: gathers, reduction, y and carry.  Every thread of the workgroup calls it.
template <typename T, bool NT>
__device__ __forceinline__ void flat_tile(FlatShared<T> &sh, int t, int32_t m, int32_t nnz, T alpha,
                                          const int32_t *__restrict__ row_ptr, const int32_t c[4], T p[4],
                                          const T *__restrict__ x, T beta, T *__restrict__ y,
                                          const int32_t *__restrict__ seg_row, T *__restrict__ carry)
{
    int32_t *s_rend = sh.rend;
    T *s_out = sh.out;
    T *s_prod = sh.prod;
    T *s_wv = sh.wv;
    int32_t *s_wk = sh.wk;
    const int tid = threadIdx.x;
    const int64_t base = (int64_t)t * kFlatTile;
    const int32_t n1 = nnz - base < kFlatTile ? (int32_t)(nnz - base) : kFlatTile;
    const int32_t k0 = tid * 4;
    // ---- rows met by the tile: rs .. re; re (if < m) continues into the next tile ----
    const int32_t rs = t == 0 ? 0 : seg_row[t];
    const int32_t re = seg_row[t + 1];
    const int32_t nwritten = re - rs;                   // rows that end inside this tile
    const int32_t rcount = nwritten + (re < m ? 1 : 0);  // plus the one left open
    const bool fits = rcount <= kFlatRowCap + 1;  // 1024 one-element rows plus the open row still fit
    int has_long = 0;
    if (fits) {
        for (int i = tid; i < rcount; i += kBlock) {
            const int32_t lo = row_ptr[rs + i], hi = row_ptr[rs + i + 1];
            s_rend[i] = (int32_t)(hi - base);
            s_out[i] = T(0);
            has_long |= (hi - lo) > kFlatRowModeMaxLen;
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (k0 + j < n1) p[j] *= x[c[j]];
#pragma unroll
    for (int j = 0; j < 4; ++j) s_prod[k0 + j + ((k0 + j) >> 5)] = k0 + j < n1 ? p[j] : T(0);
    const bool walk = fits && __syncthreads_or(has_long);  // also the barrier after staging
    if (!fits) __syncthreads();

    if (!walk) {
        // ---- row mode: 1..64 lanes per row (from the tile's row count) over the products in LDS ----
#define ASX_FLAT_ROWS(G)                                                                              \
    flat_reduce_rows<G, NT, T>(s_prod, s_rend, fits, rs, rcount, nwritten, base, n1, t, alpha, beta, row_ptr, \
                               y, carry)
        if (rcount > 128)
            ASX_FLAT_ROWS(1);
        else if (rcount > 64)
            ASX_FLAT_ROWS(2);
        else if (rcount > 32)
            ASX_FLAT_ROWS(4);
        else if (rcount > 16)
            ASX_FLAT_ROWS(8);
        else
            ASX_FLAT_ROWS(16);
#undef ASX_FLAT_ROWS
        if (re >= m && tid == 0) carry[t] = T(0);
        return;
    }

    // ---- walk mode.  Row holding this thread's first element: first i with s_rend[i] > k0 ----
    int32_t lo = 0, hi = rcount;
    while (lo < hi) {
        const int32_t mid = (lo + hi) >> 1;
        if (s_rend[mid] > k0)
            hi = mid;
        else
            lo = mid + 1;
    }
    int32_t row = lo;
    const int32_t first_row = row;
    bool emitted = false;
    T run = T(0);
    int32_t cur_end = row < rcount ? s_rend[row] : 0x7fffffff;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int32_t k = k0 + j;
        if (k < n1) {
            while (k >= cur_end) {  // the row ended before k (and any empty rows after it)
                s_out[row] = run;
                emitted = true;
                run = T(0);
                ++row;
                cur_end = row < rcount ? s_rend[row] : 0x7fffffff;
            }
            run += p[j];
        }
    }
    // the row ends exactly where this thread's elements end: nobody after us will see its end
    if (k0 < n1 && (k0 + 4 < n1 ? k0 + 4 : n1) >= cur_end) {
        s_out[row] = run;
        emitted = true;
        run = T(0);
    }

    // ---- join rows that span threads ----
    const int lane = tid & (kWave - 1), w = tid / kWave;
    const T incl = wave_segscan_incl<T>(row, run);
    const int32_t key0 = __shfl(row, 0, kWave);
    if (lane == kWave - 1) {
        s_wk[w] = row;
        s_wv[w] = incl;
    }
    __syncthreads();
    int32_t pk = -1;
    T pv = T(0);
    for (int j = 0; j < w; ++j) {
        const int32_t kj = s_wk[j];
        const T vj = s_wv[j];
        if (kj == pk)
            pv += vj;
        else {
            pk = kj;
            pv = vj;
        }
    }
    const int32_t up_k = __shfl_up(row, 1, kWave);
    T carry_in = __shfl_up(incl, 1, kWave);
    if (lane == 0) {
        carry_in = (w > 0 && pk == first_row) ? pv : T(0);
    } else {
        if (up_k != first_row)
            carry_in = T(0);
        else if (up_k == key0 && pk == up_k)
            carry_in += pv;
    }
    if (emitted) s_out[first_row] += carry_in;
    if (tid == kBlock - 1) {
        T out = T(0);
        if (re < m && row == nwritten) {  // the open row: everything the tile saw of it
            out = incl;
            if (row == key0 && pk == row) out += pv;
        }
        carry[t] = out;
    }
    __syncthreads();

    for (int i = tid; i < nwritten; i += kBlock) {
        const int64_t r = (int64_t)rs + i;
        stream_store<NT>(y + r, axpby_out<T>(alpha, s_out[i], beta, y, r));
    }
}

// kFlatTilesPerGroup consecutive tiles per workgroup: the loads of all of them are issued before
// the first is reduced, so the reduction of one tile overlaps the memory latency of the next.
template <typename T, bool VEC, bool NT, int TPG>
__global__ __launch_bounds__(kBlock) void k_spmv_flat(int32_t m, int32_t nnz, int32_t ntiles, T alpha,
                                                      const int32_t *__restrict__ row_ptr,
                                                      const int32_t *__restrict__ col,
                                                      const T *__restrict__ val,
                                                      const T *__restrict__ x, T beta,
                                                      T *__restrict__ y,
                                                      const int32_t *__restrict__ seg_row,
                                                      T *__restrict__ carry)
{
    __shared__ FlatShared<T> sh;
    const int t0 = blockIdx.x * TPG;
    int32_t c[TPG][4];
    T p[TPG][4];
#pragma unroll
    for (int u = 0; u < TPG; ++u)
        if (t0 + u < ntiles) flat_load<T, VEC, NT>(t0 + u, nnz, col, val, c[u], p[u]);
#pragma unroll
    for (int u = 0; u < TPG; ++u) {
        if (t0 + u < ntiles) {  // uniform over the workgroup
            if (u > 0) __syncthreads();  // the previous tile is done with the LDS buffers
            flat_tile<T, NT>(sh, t0 + u, m, nnz, alpha, row_ptr, c[u], p[u], x, beta, y, seg_row, carry);
        }
    }
}

// seg_row[t] = row holding stored element t*kFlatTile for t < nt, seg_row[nt] = m,
// nt = max(1, ceil(nnz / kFlatTile)): the reference's flat partition
// (hip/kernel/level2/alphasparse_spmv_csr_flat.h:7-38) for 1024 elements per workgroup.
int launch_flat_seg_rows(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t *d_seg_row, hipStream_t s)
{
    return launch_nnz_split_rows_n(d_row_ptr, m, flat_tiles(nnz), kFlatTile, d_seg_row, s);
}

// flag[0] = 1 if any row is cut by a tile boundary (then the carry pass is needed)
__global__ __launch_bounds__(kBlock) void k_flat_has_carry(const int32_t *__restrict__ row_ptr, int32_t m,
                                                           const int32_t *__restrict__ seg_row, int32_t ntiles,
                                                           int32_t *__restrict__ flag)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x + 1;
    if (t >= ntiles) return;
    const int32_t r = seg_row[t];
    if (r < m && (int64_t)row_ptr[r] < t * kFlatTile) flag[0] = 1;
}

int launch_flat_has_carry(const int32_t *d_row_ptr, int32_t m, int32_t nnz, const int32_t *d_seg_row,
                          int32_t *d_flag, hipStream_t s)
{
    const int32_t ntiles = flat_tiles(nnz);
    if (ntiles > 1)
        hipLaunchKernelGGL(k_flat_has_carry, dim3((unsigned)ceil_div64(ntiles - 1, kBlock)), dim3(kBlock), 0, s,
                           d_row_ptr, m, d_seg_row, ntiles, d_flag);
    return check_launch();
}

template <typename T>
int launch_spmv_flat(int32_t m, int32_t nnz, T alpha, const int32_t *row_ptr, const int32_t *col,
                     const T *val, const T *x, T beta, T *y, const int32_t *seg_row, T *carry,
                     bool carry_pass, hipStream_t s)
{
    if (m <= 0) return ASX_STATUS_SUCCESS;
    const int32_t ntiles = flat_tiles(nnz);
    // the 16-byte loads need 16-byte aligned arrays (true for anything a device allocator returns;
    // a caller may pass an offset view)
    const bool aligned = ((uintptr_t)col % 16 == 0) && ((uintptr_t)val % 16 == 0);
    const bool nt = use_nontemporal(nnz, sizeof(T));
#define ASX_FLAT(VEC, NT)                                                                             \
    hipLaunchKernelGGL((k_spmv_flat<T, VEC, NT, kFlatTilesPerGroup>),                                 \
                       dim3((unsigned)ceil_div64(ntiles, kFlatTilesPerGroup)), dim3(kBlock), 0, s, m, nnz, \
                       ntiles, alpha, row_ptr, col, val, x, beta, y, seg_row, carry)
    if (aligned && nt) ASX_FLAT(true, true);
    else if (aligned) ASX_FLAT(true, false);
    else if (nt) ASX_FLAT(false, true);
    else ASX_FLAT(false, false);
#undef ASX_FLAT
    if (carry_pass)
        hipLaunchKernelGGL((k_spmv_merge_fixup<T>), dim3((unsigned)ceil_div64(ntiles, kBlock)),
                           dim3(kBlock), 0, s, m, ntiles, alpha, seg_row, carry, y);
    return check_launch();
}

#define ASX_INST(T)                                                                                  \
    template int launch_spmv_vector<T>(int32_t, int32_t, T, const int32_t *, const int32_t *,        \
                                       const T *, const T *, T, T *, hipStream_t);                   \
    template int launch_spmv_stream<T>(int32_t, int32_t, T, const int32_t *, const int32_t *,        \
                                       const T *, const T *, T, T *, const int32_t *, hipStream_t);  \
    template int launch_spmv_merge<T>(int32_t, int32_t, T, const int32_t *, const int32_t *,         \
                                      const T *, const T *, T, T *, const int32_t *, const int32_t *, \
                                      T *, hipStream_t);                                             \
    template int launch_spmv_flat<T>(int32_t, int32_t, T, const int32_t *, const int32_t *, const T *, \
                                     const T *, T, T *, const int32_t *, T *, bool, hipStream_t);
ASX_INST(float)
ASX_INST(double)
#undef ASX_INST

}  // namespace asx
