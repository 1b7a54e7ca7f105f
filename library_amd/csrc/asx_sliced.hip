// Column-sliced CSR SpMV for matrices whose columns are scattered over a large x.
//
// A random gather of x that is served by an L2 costs one 128-byte L2 request per stored element,
// and that request rate, not HBM, bounds the row-ordered kernels on such matrices.  Here the
// stored elements are regrouped once (plan build) by column slice, a slice of x being at most
// 128 KiB, and each workgroup of pass 1 copies its slice of x into LDS before it streams the
// slice's stored elements: every gather is an LDS read.  What crosses slices is one partial sum
// per (row, slice) pair with at least one stored element, written by pass 1 in slice order and
// added up per row by pass 2.
//
//   pass 1  k_sliced_products : workgroup = (slice, range of tiles); wave = one tile of 256 stored
//           elements per step (4 consecutive elements per lane, row order inside the slice).
//           16-bit column-in-slice + "first element of a run" flag per element, values in the
//           order the 16-byte loads deliver them.  In-lane running sums, one segmented wave scan,
//           partial sums stored at tile_base[tile] + rank of the run.  A run is cut at every tile
//           start, so a tile needs nothing from its neighbours (a row with 1000 elements in one
//           slice leaves 4 or 5 partial sums there instead of 1).
//   pass 2  k_sliced_reduce   : wave = block of rows_per_wave rows of A with an accumulator per row
//           in LDS.  The partial sums of the block inside slice s are the contiguous range
//           chunk_lo[b][s] .. chunk_lo[b+1][s]; the wave walks the slices in order and adds each
//           range with LDS adds (only this wave touches its accumulators and a wave's LDS
//           operations execute in order, so the order of additions is fixed), then writes
//           y = alpha * acc + beta * y.
//
// No global atomics; results are bit-reproducible.  The reference has no counterpart (its CSR
// kernels gather x from global memory: hip/kernel/level2/alphasparse_spmv_csr_vector.h:99-126).
#include <hipcub/hipcub.hpp>

#include <rocprim/rocprim.hpp>

#include <algorithm>
#include <vector>

#include "asx_internal.hpp"
#include "asx_tiles.hpp"

namespace asx {

namespace {

constexpr int32_t kPadRow = 0x7fffffff;

__global__ __launch_bounds__(kBlock) void k_sliced_keys(const int32_t *__restrict__ col, int32_t nnz, int32_t width,
                                                        int32_t *__restrict__ keys, int32_t *__restrict__ idx)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    keys[i] = col[i] / width;
    idx[i] = (int32_t)i;
}

// srow[p] = row of A that holds stored element sidx[p]
__global__ __launch_bounds__(kBlock) void k_sliced_rows(const int32_t *__restrict__ sidx, int32_t nnz,
                                                        const int32_t *__restrict__ row_ptr, int32_t m,
                                                        int32_t *__restrict__ srow)
{
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= nnz) return;
    const int32_t src = sidx[p];
    int32_t lo = 0, hi = m;  // largest r with row_ptr[r] <= src
    while (lo < hi) {
        const int32_t mid = lo + (hi - lo + 1) / 2;
        if (row_ptr[mid] <= src)
            lo = mid;
        else
            hi = mid - 1;
    }
    srow[p] = lo;
}

// Every slot of the padded element space starts as a pad: a run of its own with value 0 whose
// partial sum no row block reads.
template <typename T>
__global__ __launch_bounds__(kBlock) void k_sliced_fill_pads(int64_t slots, int32_t *__restrict__ lrow,
                                                             int32_t *__restrict__ lhead, uint16_t *__restrict__ cf,
                                                             T *__restrict__ val, int32_t *__restrict__ perm)
{
    const int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (d >= slots) return;
    lrow[d] = kPadRow;
    lhead[d] = 1;
    cf[d] = 0x8000u;
    val[d] = T(0);
    perm[d] = -1;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_sliced_place(const int32_t *__restrict__ skey, const int32_t *__restrict__ sidx,
                                                         const int32_t *__restrict__ srow, int32_t nnz, int32_t width,
                                                         const int32_t *__restrict__ pstart,
                                                         const int32_t *__restrict__ tile_off,
                                                         const int32_t *__restrict__ col, const T *__restrict__ val,
                                                         int32_t *__restrict__ lrow, int32_t *__restrict__ lhead,
                                                         uint16_t *__restrict__ cf, T *__restrict__ val_out,
                                                         int32_t *__restrict__ perm)
{
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= nnz) return;
    const int32_t sl = skey[p];
    const int32_t q = (int32_t)(p - pstart[sl]);
    const int64_t d = (int64_t)tile_off[sl] * kSlicedTile + q;
    const int32_t src = sidx[p];
    const int32_t row = srow[p];
    const bool head = (q % kSlicedTile) == 0 || srow[p - 1] != row;
    lrow[d] = row;
    lhead[d] = head ? 1 : 0;
    cf[d] = (uint16_t)((col[src] - sl * width) | (head ? 0x8000 : 0));
    const int64_t t = d / kSlicedTile;
    const int64_t phys = t * kSlicedTile + tile_val_pos<T>((int)(d % kSlicedTile));
    val_out[phys] = val[src];
    perm[phys] = src;
}

__global__ __launch_bounds__(kBlock) void k_sliced_tile_base(const int32_t *__restrict__ hscan, int32_t ntiles,
                                                             int32_t *__restrict__ tile_base)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t > ntiles) return;
    tile_base[t] = t < ntiles ? hscan[t * kSlicedTile] - 1 : hscan[(int64_t)ntiles * kSlicedTile - 1];
}

__global__ __launch_bounds__(kBlock) void k_sliced_partial_rows(const int32_t *__restrict__ lrow,
                                                                const int32_t *__restrict__ lhead,
                                                                const int32_t *__restrict__ hscan, int64_t slots,
                                                                int32_t rows_per_wave, int32_t *__restrict__ prow_full,
                                                                uint16_t *__restrict__ prow)
{
    const int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (d >= slots || !lhead[d]) return;
    const int32_t id = hscan[d] - 1;
    const int32_t r = lrow[d];
    prow_full[id] = r;
    // bit 15: this partial sum may belong to the same row as the one before it (a run cut at a tile
    // start); pass 2 must not add the two with one read-modify-write
    const bool cont = d > 0 && d % kSlicedTile == 0 && lrow[d - 1] == r;
    prow[id] = (uint16_t)((r % rows_per_wave) | (cont ? 0x8000 : 0));
}

// chunk_lo[b * nslices + s] = first partial sum of slice s whose row is >= b * rows_per_wave
__global__ __launch_bounds__(kBlock) void k_sliced_chunks(const int32_t *__restrict__ prow_full,
                                                          const int32_t *__restrict__ tile_base,
                                                          const int32_t *__restrict__ tile_off, int32_t nslices,
                                                          int32_t nrb, int32_t rows_per_wave,
                                                          int32_t *__restrict__ chunk_lo)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= ((int64_t)nrb + 1) * nslices) return;
    const int32_t b = (int32_t)(i / nslices), sl = (int32_t)(i % nslices);
    const int64_t target = (int64_t)b * rows_per_wave;
    int32_t lo = tile_base[tile_off[sl]], hi = tile_base[tile_off[sl + 1]];
    while (lo < hi) {
        const int32_t mid = lo + (hi - lo) / 2;
        if ((int64_t)prow_full[mid] < target)
            lo = mid + 1;
        else
            hi = mid;
    }
    chunk_lo[i] = lo;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_sliced_regather(const int32_t *__restrict__ perm, int64_t slots,
                                                            const T *__restrict__ val, T *__restrict__ val_out)
{
    const int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (d >= slots) return;
    const int32_t src = perm[d];
    val_out[d] = src >= 0 ? val[src] : T(0);
}

// ---- pass 1 ------------------------------------------------------------------------------
// A run's sum goes, at the run's rank, into the wave's staging area in LDS; the tile's sums then
// leave as stores of consecutive lanes to consecutive partial sums.
constexpr int kStageRuns = kSlicedTile;  // every run of a tile
template <typename T>
struct StageRun {
    T *stage;
    __device__ __forceinline__ void operator()(int rank, T v) const { stage[rank] = v; }
};
template <typename T>
__device__ __forceinline__ void store_staged(const T *stage, int lane, int total, T *__restrict__ out)
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int k = 0; k < kStageRuns / kWave; ++k) {
        const int i = k * kWave + lane;
        if (k * kWave < total) {  // uniform
            if (i < total) out[i] = stage[i];
        }
    }
    __builtin_amdgcn_wave_barrier();
}

template <typename T, int WIDTH, int NW, int D>
__global__ __launch_bounds__(NW *kWave) void k_sliced_products(int32_t n, const int4 *__restrict__ wg_tab,
                                                               const uint16_t *__restrict__ cf,
                                                               const T *__restrict__ val,
                                                               const int32_t *__restrict__ tile_base,
                                                               const T *__restrict__ x, T *__restrict__ partial)
{
    __shared__ T xs[WIDTH];
    __shared__ T stage_all[NW * kStageRuns];
    const int4 wg = wg_tab[blockIdx.x];
    const int64_t c0 = (int64_t)wg.x * WIDTH;
    const int32_t cnt = n - c0 < WIDTH ? (int32_t)(n - c0) : WIDTH;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    T *stage = stage_all + wave * kStageRuns;
    // the first tiles' loads go out before the slice of x is fetched (they do not need it)
    const int32_t last = wg.z - 1;
    Tile<T> tl[D];
    int32_t t = wg.y + wave;
#pragma unroll
    for (int d = 0; d < D; ++d) tile_load<T>(tl[d], t + d * NW < last ? t + d * NW : last, lane, cf, val, tile_base);
    load_x_window<T, WIDTH, NW * kWave>(xs, x, c0, cnt);
    __syncthreads();
    // D tiles in turn; a tile's loads are issued D steps ahead, right after the stores of the tile
    // that used the buffer before it.  The loads are unconditional (past the end they re-read the
    // last tile), so that the number of memory operations issued after them is known and a step
    // waits for its own loads only.
    while (t < wg.z) {  // uniform over the wave
#pragma unroll
        for (int d = 0; d < D; ++d) {
            if (t + d * NW < wg.z) {
                const int total = tile_reduce<T>(tl[d], lane, xs, StageRun<T>{stage});
                store_staged<T>(stage, lane, total, partial + tl[d].base);
            }
            tile_load<T>(tl[d], t + (D + d) * NW < last ? t + (D + d) * NW : last, lane, cf, val, tile_base);
        }
        t += D * NW;
    }
}

// ---- pass 2 ------------------------------------------------------------------------------
// The partial sums of a row block, range after range in slice order, are cut (when the plan is
// built) into steps of up to 64 entries.  A step takes its entries from up to kPieces consecutive
// pieces of ranges (a range may be split between steps); lane l reads entry base[p] + l of the
// piece p it falls in.  Descriptor of a step: base[0..2], then
// first lane of piece 1 | first lane of piece 2 << 8 | entries << 16.
constexpr int kPieces = 3;
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));

// One thread per row block walks the block's ranges; `psteps == nullptr`: only count.
__global__ __launch_bounds__(kBlock) void k_sliced_pack(const int32_t *__restrict__ chunk_lo, int32_t nrb,
                                                         int32_t nslices, const int32_t *__restrict__ pstep_ptr,
                                                         int32_t *__restrict__ count, i32x4 *__restrict__ psteps)
{
    const int32_t b = (int32_t)(blockIdx.x * blockDim.x + threadIdx.x);
    if (b >= nrb) return;
    const int32_t *lo_row = chunk_lo + (int64_t)b * nslices, *hi_row = lo_row + nslices;
    i32x4 *out = psteps ? psteps + pstep_ptr[b] : nullptr;
    int32_t nsteps = 0, fill = 0, pieces = 0;
    int32_t base[kPieces] = {0, 0, 0}, first[kPieces] = {0, kWave, kWave};
    for (int32_t sl = 0; sl < nslices; ++sl) {
        int32_t lo = lo_row[sl], len = hi_row[sl] - lo;
        while (len > 0) {
            if (pieces == kPieces || fill == kWave) {
                if (out) out[nsteps] = i32x4{base[0], base[1], base[2], first[1] | first[2] << 8 | fill << 16};
                ++nsteps;
                fill = pieces = 0;
                first[1] = first[2] = kWave;
            }
            const int32_t take = len < kWave - fill ? len : kWave - fill;
            base[pieces] = lo - fill;
            first[pieces] = fill;
            ++pieces;
            fill += take;
            lo += take;
            len -= take;
        }
    }
    if (fill > 0) {
        if (out) out[nsteps] = i32x4{base[0], base[1], base[2], first[1] | first[2] << 8 | fill << 16};
        ++nsteps;
    }
    if (!psteps) count[b] = nsteps;
}

// U steps whose loads are issued together.
template <typename T, int U>
struct StepBatch {
    uint16_t id[U];
    T pv[U];
    uint32_t valid;  // bit u: the lane's entry of step u counts
};

template <int U>
__device__ __forceinline__ void steps_describe(i32x4 (&d)[U], int32_t first, const i32x4 *__restrict__ psteps)
{
#pragma unroll
    for (int u = 0; u < U; ++u) d[u] = psteps[first + u];  // uniform addresses: scalar loads
}

// Every load is unconditional: a step past the block's last one reads entries 0..63 and counts
// nothing; a lane past a step's entries reads a neighbour's entry (prow and partial are readable
// for kSlicedReducePad entries past the last partial sum) and drops it at the add.
template <typename T, int U>
__device__ __forceinline__ void steps_issue(StepBatch<T, U> &bt, const i32x4 (&d)[U], int32_t first, int32_t end,
                                            int lane, const uint16_t *__restrict__ prow, const T *__restrict__ partial)
{
    uint32_t valid = 0;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const bool live = first + u < end;
        const int32_t w = live ? d[u].w : (kWave | kWave << 8);
        const int32_t f1 = w & 0xff, f2 = (w >> 8) & 0xff, total = w >> 16;
        int32_t base = d[u].x;
        base = lane >= f1 ? d[u].y : base;
        base = lane >= f2 ? d[u].z : base;
        const int64_t at = live ? (int64_t)base + lane : lane;
        bt.id[u] = prow[at];
        bt.pv[u] = partial[at];
        valid |= (uint32_t)(lane < total) << u;
    }
    bt.valid = valid;
}

// Entries that do not count go to a spare accumulator of the lane's own behind the block's rows
// (64 lanes adding to one address would be serialised).
template <typename T, int U>
__device__ __forceinline__ void steps_add(const StepBatch<T, U> &bt, double *acc, int32_t spare)
{
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const bool on = (bt.valid >> u) & 1;
        double *p = acc + (on ? (int32_t)(bt.id[u] & 0x7fff) : spare);
        __hip_atomic_fetch_add(p, (double)bt.pv[u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);  // ds_add_f64
    }
}

// One wave (= one workgroup) per row block.  The wave reads its steps' descriptors with scalar
// loads, one batch ahead, and keeps NB batches of U steps in flight, so that a batch waits for its
// own loads only.  Accumulators are fp64 for both value types: the LDS has a native fp64 atomic
// add (no dependent read in the wave's instruction stream), and the fp32 one measured 2.5 times
// slower.  Only this wave touches its accumulators and a wave's LDS operations execute in order,
// so the order of additions is fixed.
template <typename T, int U, int NB>
__global__ __launch_bounds__(kWave) void k_sliced_reduce(int32_t m, int32_t nrb, int32_t rw, T alpha, T beta,
                                                         const int32_t *__restrict__ pstep_ptr,
                                                         const i32x4 *__restrict__ psteps,
                                                         const uint16_t *__restrict__ prow,
                                                         const T *__restrict__ partial, T *__restrict__ y)
{
    extern __shared__ __align__(16) unsigned char sliced_lds[];
    double *acc = reinterpret_cast<double *>(sliced_lds);
    const int lane = threadIdx.x;
    // neighbouring row blocks share the cache lines at the ends of their ranges: keep them on one XCD
    // (the grid is a multiple of kXcds workgroups, dealt to the XCDs round-robin)
    const int32_t per_xcd = (int32_t)gridDim.x / kXcds;
    const int32_t b = ((int32_t)blockIdx.x % kXcds) * per_xcd + (int32_t)blockIdx.x / kXcds;
    if (b >= nrb) return;
    const int32_t s0 = pstep_ptr[b], s1 = pstep_ptr[b + 1];
    StepBatch<T, U> bt[NB];
    i32x4 d[U];
    steps_describe<U>(d, s0, psteps);
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        steps_issue<T, U>(bt[j], d, s0 + j * U, s1, lane, prow, partial);
        steps_describe<U>(d, s0 + (j + 1) * U, psteps);
        __builtin_amdgcn_sched_barrier(0);
    }
    for (int i = lane; i < rw + kWave; i += kWave) acc[i] = 0.0;  // rw + lane: the lane's spare accumulator
    int32_t k = s0;
    for (; k + NB * U < s1; k += NB * U) {  // uniform
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            steps_add<T, U>(bt[j], acc, rw + lane);
            __builtin_amdgcn_sched_barrier(0);  // keep a later batch's address arithmetic (and its wait) behind these adds
            steps_issue<T, U>(bt[j], d, k + (NB + j) * U, s1, lane, prow, partial);
            steps_describe<U>(d, k + (NB + j + 1) * U, psteps);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int j = 0; j < NB; ++j) steps_add<T, U>(bt[j], acc, rw + lane);
    const int64_t r0 = (int64_t)b * rw;
    constexpr int Q = 8;  // rows of y per lane whose old values are requested together
    for (int i0 = 0; i0 < rw; i0 += Q * kWave) {
        T yv[Q];
        if (beta != T(0)) {
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const int i = i0 + q * kWave + lane;
                yv[q] = (i < rw && r0 + i < m) ? y[r0 + i] : T(0);
            }
        }
#pragma unroll
        for (int q = 0; q < Q; ++q) {
            const int i = i0 + q * kWave + lane;
            if (i < rw && r0 + i < m) {
                const T a = (T)acc[i];
                y[r0 + i] = beta == T(0) ? alpha * a : fma_t<T>(alpha, a, beta * yv[q]);
            }
        }
    }
}

}  // namespace

void free_sliced(SlicedMatrix *p)
{
    for (void *q : {p->val, p->partial, (void *)p->cf, (void *)p->perm, (void *)p->tile_base, (void *)p->wg_tab,
                    (void *)p->prow, (void *)p->chunk_lo, (void *)p->pstep_ptr, (void *)p->psteps})
        if (q) (void)hipFree(q);
    p->val = p->partial = nullptr;
    p->cf = p->prow = nullptr;
    p->perm = p->tile_base = p->wg_tab = p->chunk_lo = p->pstep_ptr = p->psteps = nullptr;
}

template <typename T>
int build_sliced(int32_t m, int32_t n, int32_t nnz, int32_t width, int32_t rows_per_wave, int32_t target_wgs,
                 const int32_t *row_ptr, const int32_t *col, const T *val, SlicedMatrix *out, hipStream_t s)
{
    SlicedMatrix sm{};
    if (m <= 0 || nnz <= 0 || n <= 0) return ASX_STATUS_INVALID_SIZE;
    if (width < 1 || width > 32768 || rows_per_wave < 1 || rows_per_wave > 65536 || target_wgs < 1)
        return ASX_STATUS_INVALID_VALUE;
    sm.width = width;
    sm.nslices = (int32_t)ceil_div64(n, width);
    sm.rows_per_wave = rows_per_wave;
    sm.nrb = (int32_t)ceil_div64(m, rows_per_wave);
    int key_bits = 1;
    while ((1 << key_bits) < sm.nslices) ++key_bits;

    int st = ASX_STATUS_SUCCESS;
    // Scratch of the build, in one allocation (every hipMalloc / hipFree of this size costs a
    // fraction of a millisecond): five arrays of `cap` ints, cap = the most slots there can be
    // (every slice padded to whole tiles), used in turn as
    //   a: sort keys in, then row of each sorted element, then (after the placing) the scan of run starts
    //   b: sorted keys = slice of each sorted element, then (after the placing) the row of each partial sum
    //   c: sort values in, then row of each slot
    //   d: sorted values = position in A of each sorted element
    //   e: run-start flag of each slot
    // followed by the slice offsets (elements, tiles) and the sort / scan workspace.
    int32_t *arena = nullptr;
    int32_t *a = nullptr, *b = nullptr, *c = nullptr, *d = nullptr, *e = nullptr;
    int32_t *lrow = nullptr, *lhead = nullptr, *hscan = nullptr, *prow_full = nullptr;
    int32_t *d_pstart = nullptr, *d_tile_off = nullptr;
    void *tmp = nullptr;
    int32_t *pack_tmp = nullptr;
    void *pack_scan_tmp = nullptr;
    size_t tmp_sort = 0, tmp_scan = 0, tmp_bytes = 0;
    std::vector<int32_t> pstart((size_t)sm.nslices + 1), tile_off((size_t)sm.nslices + 1, 0);
    std::vector<int32_t> tab;
    int64_t slots = 0;
    const unsigned grid = (unsigned)ceil_div64(nnz, kBlock);
    const int64_t cap64 = (int64_t)nnz + (int64_t)(kSlicedTile - 1) * sm.nslices;
    if (cap64 > 0x7fffffff) return ASX_STATUS_INVALID_SIZE;
    const size_t cap = ((size_t)cap64 + 63) & ~(size_t)63;
    const size_t noff = ((size_t)sm.nslices + 1 + 63) & ~(size_t)63;
#define ASX_TRY(expr)         \
    do {                      \
        st = status_of(expr); \
        if (st) goto done;    \
    } while (0)
#define ASX_TRY_ST(expr)   \
    do {                   \
        st = (expr);       \
        if (st) goto done; \
    } while (0)
    ASX_TRY(hipcub::DeviceRadixSort::SortPairs(nullptr, tmp_sort, a, b, c, d, nnz, 0, key_bits, s));
    ASX_TRY(hipcub::DeviceScan::InclusiveSum(nullptr, tmp_scan, lhead, hscan, (int)cap64, s));
    tmp_bytes = std::max<size_t>(std::max(tmp_sort, tmp_scan), 256);
    ASX_TRY(hipMalloc((void **)&arena, sizeof(int32_t) * (5 * cap + 2 * noff) + tmp_bytes));
    a = arena, b = a + cap, c = b + cap, d = c + cap, e = d + cap;
    d_pstart = e + cap;
    d_tile_off = d_pstart + noff;
    tmp = d_tile_off + noff;

    // 1. stored elements by slice (stable: row order, then column order, survives inside a slice)
    hipLaunchKernelGGL(k_sliced_keys, dim3(grid), dim3(kBlock), 0, s, col, nnz, width, a, c);
    ASX_TRY(hipcub::DeviceRadixSort::SortPairs(tmp, tmp_bytes, a, b, c, d, nnz, 0, key_bits, s));
    // b = slice of each sorted element, d = its position in A; a = its row
    hipLaunchKernelGGL(k_sliced_rows, dim3(grid), dim3(kBlock), 0, s, d, nnz, row_ptr, m, a);
    ASX_TRY_ST(launch_offsets_from_sorted(b, nnz, sm.nslices, d_pstart, s));
    ASX_TRY(hipMemcpyAsync(pstart.data(), d_pstart, sizeof(int32_t) * pstart.size(), hipMemcpyDeviceToHost, s));
    ASX_TRY(hipStreamSynchronize(s));

    // 2. tiles: every slice starts a new tile
    for (int32_t sl = 0; sl < sm.nslices; ++sl)
        tile_off[sl + 1] = tile_off[sl] + (int32_t)ceil_div64(pstart[sl + 1] - pstart[sl], kSlicedTile);
    sm.ntiles = tile_off[sm.nslices];
    slots = (int64_t)sm.ntiles * kSlicedTile;
    if (slots > 0x7fffffff) {
        st = ASX_STATUS_INVALID_SIZE;
        goto done;
    }
    ASX_TRY(hipMemcpyAsync(d_tile_off, tile_off.data(), sizeof(int32_t) * tile_off.size(), hipMemcpyHostToDevice, s));
    ASX_TRY(hipMalloc(&sm.val, sizeof(T) * (size_t)slots));
    ASX_TRY(hipMalloc((void **)&sm.cf, sizeof(uint16_t) * (size_t)slots));
    ASX_TRY(hipMalloc((void **)&sm.perm, sizeof(int32_t) * (size_t)slots));
    lrow = c;   // the sort's input values are spent
    lhead = e;
    {
        const unsigned sgrid = (unsigned)ceil_div64(slots, kBlock);
        hipLaunchKernelGGL((k_sliced_fill_pads<T>), dim3(sgrid), dim3(kBlock), 0, s, slots, lrow, lhead, sm.cf,
                           (T *)sm.val, sm.perm);
        hipLaunchKernelGGL((k_sliced_place<T>), dim3(grid), dim3(kBlock), 0, s, b, d, a, nnz, width, d_pstart, d_tile_off,
                           col, val, lrow, lhead, sm.cf, (T *)sm.val, sm.perm);
        // 3. partial sums: one per run start
        hscan = a;      // the placing has read the rows, slices and positions of the sorted elements:
        prow_full = b;  // their arrays are free (kernels run in stream order)
        ASX_TRY(hipcub::DeviceScan::InclusiveSum(tmp, tmp_bytes, lhead, hscan, (int)slots, s));
        ASX_TRY(hipMemcpyAsync(&sm.npartials, hscan + (slots - 1), sizeof(int32_t), hipMemcpyDeviceToHost, s));
        ASX_TRY(hipStreamSynchronize(s));
        ASX_TRY(hipMalloc((void **)&sm.tile_base, sizeof(int32_t) * ((size_t)sm.ntiles + 1)));
        ASX_TRY(hipMalloc((void **)&sm.prow, sizeof(uint16_t) * ((size_t)sm.npartials + kSlicedReducePad)));
        ASX_TRY(hipMemsetAsync(sm.prow, 0, sizeof(uint16_t) * ((size_t)sm.npartials + kSlicedReducePad), s));
        ASX_TRY(hipMalloc(&sm.partial, sizeof(T) * ((size_t)sm.npartials + kSlicedReducePad)));
        ASX_TRY(hipMemsetAsync(sm.partial, 0, sizeof(T) * ((size_t)sm.npartials + kSlicedReducePad), s));
        ASX_TRY(hipMalloc((void **)&sm.chunk_lo, sizeof(int32_t) * ((size_t)sm.nrb + 1) * (size_t)sm.nslices));
        hipLaunchKernelGGL(k_sliced_tile_base, dim3((unsigned)ceil_div64((int64_t)sm.ntiles + 1, kBlock)), dim3(kBlock),
                           0, s, hscan, sm.ntiles, sm.tile_base);
        hipLaunchKernelGGL(k_sliced_partial_rows, dim3(sgrid), dim3(kBlock), 0, s, lrow, lhead, hscan, slots,
                           rows_per_wave, prow_full, sm.prow);
        // 4. where each row block starts inside each slice's partial sums
        const int64_t nchunks = ((int64_t)sm.nrb + 1) * sm.nslices;
        hipLaunchKernelGGL(k_sliced_chunks, dim3((unsigned)ceil_div64(nchunks, kBlock)), dim3(kBlock), 0, s, prow_full,
                           sm.tile_base, d_tile_off, sm.nslices, sm.nrb, rows_per_wave, sm.chunk_lo);
    }
    // 4b. the steps in which pass 2 reads each row block's ranges
    {
        size_t scan_bytes = 0;
        int32_t *cnt = nullptr;
        ASX_TRY(hipMalloc((void **)&pack_tmp, sizeof(int32_t) * ((size_t)sm.nrb + 1)));
        cnt = pack_tmp;
        ASX_TRY(hipMalloc((void **)&sm.pstep_ptr, sizeof(int32_t) * ((size_t)sm.nrb + 1)));
        ASX_TRY(hipMemsetAsync(cnt, 0, sizeof(int32_t) * ((size_t)sm.nrb + 1), s));
        ASX_TRY(rocprim::exclusive_scan(nullptr, scan_bytes, cnt, sm.pstep_ptr, 0, (size_t)sm.nrb + 1, rocprim::plus<int32_t>(), s));
        ASX_TRY(hipMalloc(&pack_scan_tmp, std::max<size_t>(scan_bytes, 256)));
        const unsigned pgrid = (unsigned)ceil_div64(sm.nrb, kBlock);
        hipLaunchKernelGGL(k_sliced_pack, dim3(pgrid), dim3(kBlock), 0, s, sm.chunk_lo, sm.nrb, sm.nslices, nullptr, cnt,
                           nullptr);
        ASX_TRY(rocprim::exclusive_scan(pack_scan_tmp, scan_bytes, cnt, sm.pstep_ptr, 0, (size_t)sm.nrb + 1, rocprim::plus<int32_t>(), s));
        ASX_TRY(hipMemcpyAsync(&sm.npsteps, sm.pstep_ptr + sm.nrb, sizeof(int32_t), hipMemcpyDeviceToHost, s));
        ASX_TRY(hipStreamSynchronize(s));
        ASX_TRY(hipMalloc((void **)&sm.psteps, sizeof(int32_t) * 4 * ((size_t)sm.npsteps + kSlicedStepPad)));
        ASX_TRY(hipMemsetAsync(sm.psteps, 0, sizeof(int32_t) * 4 * ((size_t)sm.npsteps + kSlicedStepPad), s));
        hipLaunchKernelGGL(k_sliced_pack, dim3(pgrid), dim3(kBlock), 0, s, sm.chunk_lo, sm.nrb, sm.nslices, sm.pstep_ptr,
                           nullptr, reinterpret_cast<i32x4 *>(sm.psteps));
    }
    // 5. workgroups of pass 1: every slice gets its share of about `target_wgs` workgroups (at
    //    least one, and no workgroup smaller than 32 tiles unless the slice is), its tiles in equal
    //    pieces
    {
        for (int32_t sl = 0; sl < sm.nslices; ++sl) {
            const int32_t tiles = tile_off[sl + 1] - tile_off[sl];
            if (tiles == 0) continue;
            int32_t pieces = (int32_t)(((int64_t)tiles * target_wgs + sm.ntiles / 2) / sm.ntiles);
            pieces = std::min<int32_t>(pieces, tiles / 32);
            pieces = std::max<int32_t>(pieces, 1);
            for (int32_t k = 0; k < pieces; ++k) {
                tab.push_back(sl);
                tab.push_back(tile_off[sl] + (int32_t)((int64_t)tiles * k / pieces));
                tab.push_back(tile_off[sl] + (int32_t)((int64_t)tiles * (k + 1) / pieces));
                tab.push_back(0);
            }
        }
        sm.nwg = (int32_t)(tab.size() / 4);
        // The workgroups of a slice all fetch that slice of x: keep them on one XCD, whose L2 then
        // fetches it once (workgroup i runs on XCD i mod kXcds; entry j of the list above goes to
        // position (j mod per_xcd) * kXcds + j / per_xcd, so consecutive entries share an XCD).
        if (sm.nwg > sm.nslices && sm.nwg % kXcds == 0) {
            const int32_t per_xcd = sm.nwg / kXcds;
            std::vector<int32_t> placed(tab.size());
            for (int32_t j = 0; j < sm.nwg; ++j) {
                const int32_t i = (j % per_xcd) * kXcds + j / per_xcd;
                for (int q = 0; q < 4; ++q) placed[(size_t)i * 4 + q] = tab[(size_t)j * 4 + q];
            }
            tab.swap(placed);
        }
        ASX_TRY(hipMalloc((void **)&sm.wg_tab, sizeof(int32_t) * std::max<size_t>(tab.size(), 4)));
        ASX_TRY(hipMemcpyAsync(sm.wg_tab, tab.data(), sizeof(int32_t) * tab.size(), hipMemcpyHostToDevice, s));
    }
    ASX_TRY(hipStreamSynchronize(s));
    ASX_TRY(hipGetLastError());
#undef ASX_TRY
#undef ASX_TRY_ST
done:
    if (arena) (void)hipFree(arena);
    if (pack_tmp) (void)hipFree(pack_tmp);
    if (pack_scan_tmp) (void)hipFree(pack_scan_tmp);
    if (st) {
        free_sliced(&sm);
        return st;
    }
    *out = sm;
    return ASX_STATUS_SUCCESS;
}

template <typename T>
int sliced_update_values(const SlicedMatrix *sm, const T *val, hipStream_t s)
{
    const int64_t slots = (int64_t)sm->ntiles * kSlicedTile;
    if (slots == 0) return ASX_STATUS_SUCCESS;
    hipLaunchKernelGGL((k_sliced_regather<T>), dim3((unsigned)ceil_div64(slots, kBlock)), dim3(kBlock), 0, s, sm->perm,
                       slots, val, (T *)sm->val);
    return check_launch();
}

template <typename T>
int launch_spmv_sliced(int32_t m, int32_t n, T alpha, const SlicedMatrix *sm, const T *x, T beta, T *y, T *partial,
                       hipStream_t s)
{
    if (m <= 0) return ASX_STATUS_SUCCESS;
    if (!partial) return ASX_STATUS_INVALID_POINTER;
    constexpr int kSmall = 65536 / sizeof(T), kLarge = 131072 / sizeof(T);
    const int4 *tab = reinterpret_cast<const int4 *>(sm->wg_tab);
    constexpr int kDepth = 2;  // tiles in flight per wave (3 and 4 measured the same or slower)
#define ASX_PROD(W)                                                                                                 \
    hipLaunchKernelGGL((k_sliced_products<T, W, 16, kDepth>), dim3((unsigned)sm->nwg), dim3(16 * kWave), 0, s, n, tab, \
                       sm->cf, (const T *)sm->val, sm->tile_base, x, partial)
    if (sm->nwg > 0) {
        if (sm->width == kLarge)
            ASX_PROD(kLarge);
        else if (sm->width == kSmall)
            ASX_PROD(kSmall);
        else
            return ASX_STATUS_INVALID_VALUE;
    }
#undef ASX_PROD
    // steps per batch and batches in flight: 4 x 2 measured best (8 x 2, 4 x 4: the same or 1-3 % slower)
    constexpr int kSteps = 4, kBatches = 2;
    static_assert((kBatches + 1) * kSteps <= kSlicedStepPad, "descriptors are read this far past a block's last step");
    const int32_t rw = sm->rows_per_wave;
    const size_t lds = align_up(((size_t)rw + kWave) * sizeof(double), 16);
    if (rw < 1 || rw > 32767 || lds > 65536) return ASX_STATUS_INVALID_VALUE;
    const unsigned rgrid = (unsigned)(ceil_div64(sm->nrb, kXcds) * kXcds);
    hipLaunchKernelGGL((k_sliced_reduce<T, kSteps, kBatches>), dim3(rgrid), dim3(kWave), lds, s, m, sm->nrb, rw, alpha, beta,
                       sm->pstep_ptr, reinterpret_cast<const i32x4 *>(sm->psteps), sm->prow, partial, y);
    return check_launch();
}

#define ASX_INST(T)                                                                                              \
    template int build_sliced<T>(int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, const int32_t *,          \
                                 const int32_t *, const T *, SlicedMatrix *, hipStream_t);                       \
    template int sliced_update_values<T>(const SlicedMatrix *, const T *, hipStream_t);                          \
    template int launch_spmv_sliced<T>(int32_t, int32_t, T, const SlicedMatrix *, const T *, T, T *, T *, hipStream_t);
ASX_INST(float)
ASX_INST(double)
#undef ASX_INST

}  // namespace asx
