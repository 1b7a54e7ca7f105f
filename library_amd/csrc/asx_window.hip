// Row-block CSR SpMV with a sliding window of x in LDS, for matrices whose rows reach only
// nearby columns (stencils, banded and finite-element matrices).
//
// The row-ordered kernels read 4 bytes of column index per stored element, the row offsets, and
// gather x through the L2 (one request per stored element).  Here the rows are cut, once (plan
// build), into blocks of R consecutive rows whose columns all lie inside a window of fewer than
// kWindowCols columns, and consecutive blocks are chained: a workgroup walks its chain of blocks
// with LDS as a ring over the columns of x (column c lives at c mod kWindowCols), so that from
// one block to the next only the columns that are new are fetched - while the block before is
// still being multiplied - and x crosses the L2 once.  The block's stored elements stream as
// tiles of 256 with a 16-bit column-mod-window and a "first element of a row" flag per element
// (10 instead of 12.8 bytes per stored element in fp64; no row offsets are read).  Every row owns
// at least one slot (an empty row gets a zero that points at a zero in LDS), so the runs of a tile
// are consecutive rows and a run's sum goes straight to y.  Rows of up to 16 stored elements are
// never cut by a tile start (the tile is padded instead); a longer row that is cut leaves its
// later pieces in carry slots, which an ordered pass adds to y afterwards (no atomics; results are
// bit-reproducible).
//
// The reference has no counterpart (its CSR kernels read 32-bit columns and gather x from global
// memory: hip/kernel/level2/alphasparse_spmv_csr_vector.h:99-126).
#include <hipcub/hipcub.hpp>

#include <algorithm>
#include <vector>

#include "asx_internal.hpp"
#include "asx_tiles.hpp"

namespace asx {

namespace {

constexpr int32_t kNoCol = 0x7fffffff;
constexpr int kWindowCols = 16384;    // ring size in columns: 128 KiB of fp64, 64 KiB of fp32
constexpr int kWindowSlack = 8;       // a block's window is kept this much narrower (aligned fetches)
constexpr int kWindowWaves = 16;
constexpr int32_t kAlignRowLen = 16;  // rows up to this length are not cut by tile starts

// first and last column of every row (cmin = kNoCol, cmax = -1 for an empty row)
__global__ __launch_bounds__(kBlock) void k_window_row_span(const int32_t *__restrict__ row_ptr,
                                                            const int32_t *__restrict__ col, int32_t m,
                                                            int32_t *__restrict__ cmin, int32_t *__restrict__ cmax)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= m) return;
    int32_t lo = kNoCol, hi = -1;
    for (int32_t k = row_ptr[r]; k < row_ptr[r + 1]; ++k) {
        const int32_t c = col[k];
        lo = c < lo ? c : lo;
        hi = c > hi ? c : hi;
    }
    cmin[r] = lo;
    cmax[r] = hi;
}

// bmin / bmax of every block of `rows` rows (bmin preset to kNoCol, bmax to -1)
__global__ __launch_bounds__(kBlock) void k_window_block_span(const int32_t *__restrict__ cmin,
                                                              const int32_t *__restrict__ cmax, int32_t m,
                                                              int32_t rows, int32_t *__restrict__ bmin,
                                                              int32_t *__restrict__ bmax)
{
    // `rows` is a multiple of 256, so the 64 rows of a wave lie in one block: one pair of atomics a wave
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int32_t lo = kNoCol, hi = -1;
    if (r < m && cmax[r] >= 0) lo = cmin[r], hi = cmax[r];
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        lo = min(lo, __shfl_xor(lo, d, kWave));
        hi = max(hi, __shfl_xor(hi, d, kWave));
    }
    if (__lane_id() != 0 || hi < 0) return;
    atomicMin(bmin + r / rows, lo);
    atomicMax(bmax + r / rows, hi);
}
__global__ __launch_bounds__(kBlock) void k_window_fill_i32(int32_t *p, int64_t n, int32_t v)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}
// widest window any block needs once its start is rounded down to a multiple of 4 columns
__global__ __launch_bounds__(kBlock) void k_window_max_span(const int32_t *__restrict__ bmin,
                                                            const int32_t *__restrict__ bmax, int32_t nblocks,
                                                            int32_t *__restrict__ out)
{
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks || bmax[b] < 0) return;
    atomicMax(out, bmax[b] - (bmin[b] & ~3) + 1);
}

// Slot (from the start of its block) at which every row starts, and the tiles of every block.  A
// row takes max(1, length) slots; a row of at most kAlignRowLen slots that would cross a tile
// start begins at that tile start instead.  One thread walks one block's rows in order.
__global__ __launch_bounds__(kBlock) void k_window_row_starts(const int32_t *__restrict__ row_ptr, int32_t m,
                                                              int32_t rows, int32_t nblocks,
                                                              int32_t *__restrict__ row_start,
                                                              int32_t *__restrict__ block_tiles)
{
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const int32_t r0 = (int32_t)(b * rows);
    const int32_t r1 = (int64_t)r0 + rows < m ? r0 + rows : m;
    int32_t pos = 0;
    int32_t next = row_ptr[r0];
    for (int32_t r = r0; r < r1; ++r) {
        const int32_t cur = next;
        next = row_ptr[r + 1];
        const int32_t len = next - cur > 0 ? next - cur : 1;
        const int32_t in_tile = pos % kSlicedTile;
        if (len <= kAlignRowLen && in_tile + len > kSlicedTile) pos += kSlicedTile - in_tile;
        row_start[r] = pos;
        pos += len;
    }
    block_tiles[b] = (pos + kSlicedTile - 1) / kSlicedTile;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_window_fill_pads(int64_t slots, uint16_t pad, uint16_t *__restrict__ cf,
                                                             T *__restrict__ val, int32_t *__restrict__ perm)
{
    const int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (d >= slots) return;
    cf[d] = pad;
    val[d] = T(0);
    perm[d] = -1;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_window_place(const int32_t *__restrict__ row_ptr,
                                                         const int32_t *__restrict__ col, const T *__restrict__ val,
                                                         int32_t m, int32_t nnz, int32_t rows,
                                                         const int32_t *__restrict__ row_start,
                                                         const int32_t *__restrict__ tile_off, uint16_t *__restrict__ cf,
                                                         T *__restrict__ val_out, int32_t *__restrict__ perm)
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
    const int32_t r = lo, b = r / rows;
    const int32_t o = row_start[r] + (int32_t)(i - row_ptr[r]);
    const int64_t d = (int64_t)tile_off[b] * kSlicedTile + o;
    const bool head = i == row_ptr[r] || o % kSlicedTile == 0;
    cf[d] = (uint16_t)((col[i] % kWindowCols) | (head ? 0x8000 : 0));
    const int64_t phys = d / kSlicedTile * kSlicedTile + tile_val_pos<T>((int)(d % kSlicedTile));
    val_out[phys] = val[i];
    perm[phys] = (int32_t)i;
}

// per tile: x = the row its first slot belongs to, bit 31 set when the tile starts inside that
// row; y = the number of runs of the tile that are rows (the slots behind them are padding)
__global__ __launch_bounds__(kBlock) void k_window_tile_info(const int32_t *__restrict__ row_start, int32_t m,
                                                             int32_t rows, int32_t nblocks,
                                                             const int32_t *__restrict__ tile_off, int32_t ntiles,
                                                             int2 *__restrict__ tile_info, int32_t *__restrict__ any_cont)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= ntiles) return;
    int32_t lo = 0, hi = nblocks - 1;  // block of tile t: largest b with tile_off[b] <= t
    while (lo < hi) {
        const int32_t mid = lo + (hi - lo + 1) / 2;
        if (tile_off[mid] <= t)
            lo = mid;
        else
            hi = mid - 1;
    }
    const int32_t b = lo, r0 = b * rows;
    const int32_t r1 = (int64_t)r0 + rows < m ? r0 + rows : m;
    const int32_t o = (int32_t)(t - tile_off[b]) * kSlicedTile;
    int32_t a = r0, z = r1 - 1;  // largest row whose start is <= o
    while (a < z) {
        const int32_t mid = a + (z - a + 1) / 2;
        if (row_start[mid] <= o)
            a = mid;
        else
            z = mid - 1;
    }
    int32_t u = a + 1, v = r1;  // first row that starts at or behind the end of the tile
    while (u < v) {
        const int32_t mid = u + (v - u) / 2;
        if (row_start[mid] < o + kSlicedTile)
            u = mid + 1;
        else
            v = mid;
    }
    const bool cont = row_start[a] != o;
    tile_info[t] = make_int2(a | (cont ? (int32_t)0x80000000 : 0), u - a);
    if (cont) *any_cont = 1;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_window_regather(const int32_t *__restrict__ perm, int64_t slots,
                                                            const T *__restrict__ val, T *__restrict__ val_out)
{
    const int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (d >= slots) return;
    const int32_t src = perm[d];
    val_out[d] = src >= 0 ? val[src] : T(0);
}

// ---- the kernel ----------------------------------------------------------------------------
// Run k of a tile is row (first row of the tile) + k, for the `limit` runs that are rows; the
// first sum of a tile that starts inside a row goes to the tile's carry slot.  The sums of the
// first kStageRows rows of a tile pass through a staging area of the wave in LDS and leave as
// stores of consecutive lanes to consecutive rows: stored straight from the lanes that close the
// runs (4 or 5 masked stores a tile, 8 bytes every 32 to 40), the same 134 MB of y cost 66 us of
// the 5-point stencil's 220; staged, a third of that.  Rows past kStageRows (a tile of rows shorter
// than 2 on average) are stored directly.
constexpr int kStageRows = 128;
template <typename T>
struct StoreRows {
    T *y, *carry_slot, *stage;
    int32_t row0, limit;
    bool cont;
    T alpha, beta;
    __device__ __forceinline__ void operator()(int rank, T v) const
    {
        if (rank == 0 && cont) {
            *carry_slot = v;
            return;
        }
        if (rank < kStageRows) {
            stage[rank] = v;  // ranks at or past `limit` are written too and never read
        } else if (rank < limit) {
            const int64_t r = (int64_t)row0 + rank;
            y[r] = beta == T(0) ? alpha * v : fma_t<T>(alpha, v, beta * y[r]);
        }
    }
    // after the tile's runs are staged: the wave's LDS writes and reads execute in order
    __device__ __forceinline__ void flush(int lane) const
    {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const int32_t first = cont ? 1 : 0, end = limit < kStageRows ? limit : kStageRows;
#pragma unroll
        for (int k = 0; k < kStageRows / kWave; ++k) {
            const int32_t i = k * kWave + lane;
            if (k * kWave < end) {  // uniform
                if (i >= first && i < end) {
                    const int64_t r = (int64_t)row0 + i;
                    const T v = stage[i];
                    y[r] = beta == T(0) ? alpha * v : fma_t<T>(alpha, v, beta * y[r]);
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
};

template <typename T>
struct WindowTile : Tile<T> {
    int32_t limit;
};
template <typename T>
__device__ __forceinline__ void window_tile_load(WindowTile<T> &tl, int32_t t, int lane, const uint16_t *__restrict__ cf,
                                                 const T *__restrict__ val, const int2 *__restrict__ tile_info)
{
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 cw = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(cf + (int64_t)t * kSlicedTile) + lane);
    tl.c01 = cw.x;
    tl.c23 = cw.y;
    TileValues<T>::load(val + (int64_t)t * kSlicedTile, lane, tl.v);
    const int2 info = tile_info[t];
    tl.base = info.x;
    tl.limit = info.y;
}

// The columns [lo, hi) of x (lo a multiple of 4, hi - lo <= kWindowCols) into registers, one
// 16-byte piece per thread and step; columns at or past n read as 0.  Every register is written by
// one load instruction only (predicated, after a zero fill), never by two alternative ones: with
// alternatives the compiler orders them with a full s_waitcnt between the steps and the fetch
// takes one memory round trip per step.  ALIGNED (x on a 16-byte boundary): whole pieces inside x
// with one 16-byte load; the piece that straddles the end of x (n no multiple of the piece),
// element by element into `tail` by the one thread that owns it.  Otherwise element by element.
template <typename T, int THREADS, bool ALIGNED>
struct XFetch {
    static constexpr int V = 16 / sizeof(T);
    static constexpr int PER = kWindowCols / (THREADS * V);
    typedef T vec_t __attribute__((ext_vector_type(V)));
    vec_t buf[PER];
    vec_t tail;
    __device__ __forceinline__ void load(const T *__restrict__ x, int32_t n, int32_t lo, int32_t hi)
    {
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const int64_t c = (int64_t)lo + ((int64_t)k * THREADS + threadIdx.x) * V;
            buf[k] = vec_t(T(0));
            if (ALIGNED) {
                if (c < hi && c + V <= n) buf[k] = *reinterpret_cast<const vec_t *>(x + c);
            } else {
#pragma unroll
                for (int e = 0; e < V; ++e)
                    if (c + e < hi && c + e < n) buf[k][e] = x[c + e];
            }
        }
        if (ALIGNED) {
            tail = vec_t(T(0));
            const int64_t cs = (int64_t)n & ~(int64_t)(V - 1);  // start of the piece that straddles the end of x
            if (cs < n && cs >= lo && cs < hi && ((cs - lo) / V) % THREADS == (int64_t)threadIdx.x) {
#pragma unroll
                for (int e = 0; e < V - 1; ++e)
                    if (cs + e < n) tail[e] = x[cs + e];
            }
        }
    }
    __device__ __forceinline__ void store(T *xs, int32_t n, int32_t lo, int32_t hi) const
    {
        const int64_t cs = (int64_t)n & ~(int64_t)(V - 1);
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const int64_t c = (int64_t)lo + ((int64_t)k * THREADS + threadIdx.x) * V;
            if (c < hi) *reinterpret_cast<vec_t *>(xs + (c % kWindowCols)) = (ALIGNED && c == cs) ? tail : buf[k];
        }
    }
};

template <typename T, int NW, bool ALIGNED>
__global__ __launch_bounds__(NW *kWave) void k_spmv_window(int32_t n, T alpha, T beta, const int2 *__restrict__ chains,
                                                           const int4 *__restrict__ blocks,
                                                           const uint16_t *__restrict__ cf, const T *__restrict__ val,
                                                           const int2 *__restrict__ tile_info,
                                                           const T *__restrict__ x, T *__restrict__ y,
                                                           T *__restrict__ carry)
{
    // ring over the columns of x, then the zero the pads point at
    __shared__ __align__(16) T xs[kWindowCols + 16 / sizeof(T)];
    __shared__ T stage_all[NW * kStageRows];
    const int2 chain = chains[blockIdx.x];  // first block, end block
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    T *stage = stage_all + wave * kStageRows;
    const int32_t chain_last = blocks[chain.y - 1].y - 1;  // last tile of the chain
    // this wave's tiles are those congruent to its number, across the blocks of the chain; two are
    // in flight (loaded two steps ahead; past the end of the chain the last tile is re-read)
    WindowTile<T> ta, tb;
    int32_t t = blocks[chain.x].x + wave;
    window_tile_load<T>(ta, t < chain_last ? t : chain_last, lane, cf, val, tile_info);
    window_tile_load<T>(tb, t + NW < chain_last ? t + NW : chain_last, lane, cf, val, tile_info);
    if (threadIdx.x == 0) xs[kWindowCols] = T(0);
    XFetch<T, NW * kWave, ALIGNED> xf;
    int4 blk = blocks[chain.x];  // first tile, end tile, columns to fetch before the block: from, to
    xf.load(x, n, blk.z, blk.w);
    int32_t b = chain.x, tile_hi;
    // Start of block b: the columns fetched for it go into the ring once every wave is done with
    // the block before; the next block's new columns are fetched while this one is multiplied.
#define ASX_BLOCK_BEGIN()                      \
    {                                          \
        __syncthreads();                       \
        xf.store(xs, n, blk.z, blk.w);         \
        __syncthreads();                       \
        tile_hi = blk.y;                       \
        if (b + 1 < chain.y) {                 \
            blk = blocks[b + 1];               \
            xf.load(x, n, blk.z, blk.w);       \
        }                                      \
    }
#define ASX_STEP(TL, TT)                                                                                          \
    {                                                                                                             \
        const StoreRows<T> out{y, carry + (TT), stage, TL.base & 0x7fffffff, TL.limit, TL.base < 0, alpha, beta}; \
        tile_reduce<T>(TL, lane, xs, out);                                                                        \
        out.flush(lane);                                                                                          \
    }
#define ASX_NEXT(TL, TT) window_tile_load<T>(TL, (TT) < chain_last ? (TT) : chain_last, lane, cf, val, tile_info)
    // Every wave passes the start of every block of the chain (the barriers count all waves),
    // whether it has tiles in the block or not.  ta and tb take turns without changing places.
    ASX_BLOCK_BEGIN()
    for (;;) {  // all conditions are uniform over the wave
        while (t >= tile_hi) {
            if (++b >= chain.y) return;
            ASX_BLOCK_BEGIN()
        }
        ASX_STEP(ta, t);
        ASX_NEXT(ta, t + 2 * NW);
        t += NW;
        while (t >= tile_hi) {
            if (++b >= chain.y) return;
            ASX_BLOCK_BEGIN()
        }
        ASX_STEP(tb, t);
        ASX_NEXT(tb, t + 2 * NW);
        t += NW;
    }
#undef ASX_BLOCK_BEGIN
#undef ASX_STEP
#undef ASX_NEXT
}

// Adds the carries to their rows, in tile order: the thread of the first tile of a run of tiles
// that start inside the same row sums the run's carries and adds the total once.
template <typename T>
__global__ __launch_bounds__(kBlock) void k_window_fixup(int32_t ntiles, T alpha, const int2 *__restrict__ tile_info,
                                                         const T *__restrict__ carry, T *__restrict__ y)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= ntiles) return;
    const int32_t w = tile_info[t].x;
    if (w >= 0) return;                            // starts at a row start
    if (t > 0 && tile_info[t - 1].x == w) return;  // a later tile of its run
    T s = carry[t];
    for (int64_t j = t + 1; j < ntiles && tile_info[j].x == w; ++j) s += carry[j];
    const int32_t r = w & 0x7fffffff;
    y[r] = fma_t<T>(alpha, s, y[r]);
}

}  // namespace

void free_window(WindowMatrix *p)
{
    for (void *q : {p->val, p->carry, (void *)p->cf, (void *)p->perm, (void *)p->tile_info, (void *)p->blocks,
                    (void *)p->chains})
        if (q) (void)hipFree(q);
    p->val = p->carry = nullptr;
    p->cf = nullptr;
    p->perm = p->tile_info = p->blocks = p->chains = nullptr;
}

template <typename T>
int build_window(int32_t m, int32_t n, int32_t nnz, int32_t target_wgs, const int32_t *row_ptr, const int32_t *col,
                 const T *val, WindowMatrix *out, hipStream_t s)
{
    WindowMatrix wm{};
    if (m <= 0 || nnz <= 0 || n <= 0) return ASX_STATUS_INVALID_SIZE;
    if (target_wgs < 1) return ASX_STATUS_INVALID_VALUE;
    int st = ASX_STATUS_SUCCESS;
    int32_t *cmin = nullptr, *cmax = nullptr, *row_start = nullptr;  // m each
    int32_t *bmin = nullptr, *bmax = nullptr, *btiles = nullptr, *tile_off = nullptr, *d_small = nullptr;
    void *tmp = nullptr;
    size_t tmp_bytes = 0;
    std::vector<int32_t> h_bmin, h_bmax, h_off, blk, chains;
    int64_t slots = 0;
    int32_t h_small[2] = {0, 0};
    const unsigned mgrid = (unsigned)ceil_div64(m, kBlock);
    const int32_t min_blocks = 4 * target_wgs;  // larger blocks only while at least this many blocks remain
    const int32_t max_nb = (int32_t)ceil_div64(m, 256);
#define ASX_TRY(expr)         \
    do {                      \
        st = status_of(expr); \
        if (st) goto done;    \
    } while (0)
    for (int32_t **q : {&cmin, &cmax, &row_start}) ASX_TRY(hipMalloc((void **)q, sizeof(int32_t) * (size_t)m));
    for (int32_t **q : {&bmin, &bmax, &btiles, &tile_off})
        ASX_TRY(hipMalloc((void **)q, sizeof(int32_t) * ((size_t)max_nb + 1)));
    ASX_TRY(hipMalloc((void **)&d_small, sizeof(int32_t) * 2));
    ASX_TRY(hipcub::DeviceScan::ExclusiveSum(nullptr, tmp_bytes, btiles, tile_off, max_nb + 1, s));
    ASX_TRY(hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1));

    // 1. column span of every row
    hipLaunchKernelGGL(k_window_row_span, dim3(mgrid), dim3(kBlock), 0, s, row_ptr, col, m, cmin, cmax);
    // 2. the largest block of rows (a multiple of 256) whose widest window fits the ring
    wm.rows_per_block = 0;
    for (int32_t rows : {8192, 6144, 4096, 3072, 2048, 1536, 1024, 768, 512, 384, 256}) {
        if (rows > 256 && ceil_div64(m, rows) < min_blocks) continue;  // too few blocks to share out
        const int32_t nb = (int32_t)ceil_div64(m, rows);
        const unsigned bgrid = (unsigned)ceil_div64(nb, kBlock);
        hipLaunchKernelGGL(k_window_fill_i32, dim3(bgrid), dim3(kBlock), 0, s, bmin, (int64_t)nb, kNoCol);
        hipLaunchKernelGGL(k_window_fill_i32, dim3(bgrid), dim3(kBlock), 0, s, bmax, (int64_t)nb, -1);
        ASX_TRY(hipMemsetAsync(d_small, 0, sizeof(int32_t) * 2, s));
        hipLaunchKernelGGL(k_window_block_span, dim3(mgrid), dim3(kBlock), 0, s, cmin, cmax, m, rows, bmin, bmax);
        hipLaunchKernelGGL(k_window_max_span, dim3(bgrid), dim3(kBlock), 0, s, bmin, bmax, nb, d_small);
        ASX_TRY(hipMemcpyAsync(h_small, d_small, sizeof(int32_t), hipMemcpyDeviceToHost, s));
        ASX_TRY(hipStreamSynchronize(s));
        if (h_small[0] <= kWindowCols - kWindowSlack) {
            wm.rows_per_block = rows;
            wm.nblocks = nb;
            break;
        }
    }
    if (wm.rows_per_block == 0) {
        st = ASX_STATUS_NOT_SUPPORTED;  // some 256 rows reach further than the ring: not this kernel's matrix
        goto done;
    }
    // 3. where every row starts inside its block; tiles of every block
    hipLaunchKernelGGL(k_window_row_starts, dim3((unsigned)ceil_div64(wm.nblocks, kBlock)), dim3(kBlock), 0, s, row_ptr, m,
                       wm.rows_per_block, wm.nblocks, row_start, btiles);
    ASX_TRY(hipMemsetAsync(btiles + wm.nblocks, 0, sizeof(int32_t), s));
    ASX_TRY(hipcub::DeviceScan::ExclusiveSum(tmp, tmp_bytes, btiles, tile_off, wm.nblocks + 1, s));
    h_bmin.resize((size_t)wm.nblocks);
    h_bmax.resize((size_t)wm.nblocks);
    h_off.resize((size_t)wm.nblocks + 1);
    ASX_TRY(hipMemcpyAsync(h_bmin.data(), bmin, sizeof(int32_t) * h_bmin.size(), hipMemcpyDeviceToHost, s));
    ASX_TRY(hipMemcpyAsync(h_bmax.data(), bmax, sizeof(int32_t) * h_bmax.size(), hipMemcpyDeviceToHost, s));
    ASX_TRY(hipMemcpyAsync(h_off.data(), tile_off, sizeof(int32_t) * h_off.size(), hipMemcpyDeviceToHost, s));
    ASX_TRY(hipStreamSynchronize(s));
    wm.ntiles = h_off[(size_t)wm.nblocks];
    slots = (int64_t)wm.ntiles * kSlicedTile;
    if (slots > 0x7fffffff) {
        st = ASX_STATUS_INVALID_SIZE;
        goto done;
    }
    ASX_TRY(hipMalloc(&wm.val, sizeof(T) * (size_t)slots));
    ASX_TRY(hipMalloc((void **)&wm.cf, sizeof(uint16_t) * (size_t)slots));
    ASX_TRY(hipMalloc((void **)&wm.perm, sizeof(int32_t) * (size_t)slots));
    ASX_TRY(hipMalloc((void **)&wm.tile_info, sizeof(int2) * (size_t)wm.ntiles));
    ASX_TRY(hipMalloc(&wm.carry, sizeof(T) * (size_t)wm.ntiles));
    ASX_TRY(hipMemsetAsync(wm.carry, 0, sizeof(T) * (size_t)wm.ntiles, s));
    // 4. every slot starts as a zero that points at the zero behind the ring and opens a run of its
    //    own (the slots of empty rows and the padding stay that way)
    hipLaunchKernelGGL((k_window_fill_pads<T>), dim3((unsigned)ceil_div64(slots, kBlock)), dim3(kBlock), 0, s, slots,
                       (uint16_t)(0x8000 | kWindowCols), wm.cf, (T *)wm.val, wm.perm);
    hipLaunchKernelGGL((k_window_place<T>), dim3((unsigned)ceil_div64(nnz, kBlock)), dim3(kBlock), 0, s, row_ptr, col, val,
                       m, nnz, wm.rows_per_block, row_start, tile_off, wm.cf, (T *)wm.val, wm.perm);
    // 5. first row and number of rows of every tile
    ASX_TRY(hipMemsetAsync(d_small, 0, sizeof(int32_t) * 2, s));
    hipLaunchKernelGGL(k_window_tile_info, dim3((unsigned)ceil_div64(wm.ntiles, kBlock)), dim3(kBlock), 0, s, row_start, m,
                       wm.rows_per_block, wm.nblocks, tile_off, wm.ntiles, (int2 *)wm.tile_info, d_small);
    ASX_TRY(hipMemcpyAsync(h_small, d_small, sizeof(int32_t), hipMemcpyDeviceToHost, s));
    // 6. chains of blocks, one per workgroup, of about equal numbers of tiles.  Inside a chain a
    //    block fetches only the columns behind those already in the ring; a block whose columns
    //    start before what the ring still holds begins a new chain (and fetches its whole window).
    {
        const int64_t per_chain = std::max<int64_t>(1, ceil_div64(wm.ntiles, target_wgs));
        blk.resize((size_t)wm.nblocks * 4);
        int64_t have = -1;  // columns [.., have) are in the ring (-1: nothing yet)
        int32_t chain_lo = 0;
        int64_t chain_tiles = 0;
        for (int32_t b = 0; b < wm.nblocks; ++b) {
            const bool empty = h_bmax[(size_t)b] < 0;
            const int64_t lo = empty ? 0 : (h_bmin[(size_t)b] & ~3);
            const int64_t hi = empty ? 0 : ((int64_t)h_bmax[(size_t)b] + 4) & ~(int64_t)3;  // past the last, rounded up
            bool fresh = false;
            if (b != chain_lo) {
                if (!empty && have >= 0 && lo < std::max(have, hi) - kWindowCols) fresh = true;  // already overwritten
                if (chain_tiles >= per_chain) fresh = true;
            }
            if (fresh) {
                chains.push_back(chain_lo);
                chains.push_back(b);
                chain_lo = b;
                chain_tiles = 0;
                have = -1;
            }
            int64_t from = 0, to = 0;
            if (!empty) {
                if (have < 0 || lo >= have) {  // nothing useful in the ring: the whole window
                    from = lo;
                    to = hi;
                } else {
                    from = have;
                    to = std::max(have, hi);
                }
                have = to;
            }
            blk[(size_t)b * 4 + 0] = h_off[(size_t)b];
            blk[(size_t)b * 4 + 1] = h_off[(size_t)b + 1];
            blk[(size_t)b * 4 + 2] = (int32_t)from;
            blk[(size_t)b * 4 + 3] = (int32_t)to;
            chain_tiles += h_off[(size_t)b + 1] - h_off[(size_t)b];
        }
        chains.push_back(chain_lo);
        chains.push_back(wm.nblocks);
        wm.nchains = (int32_t)(chains.size() / 2);
    }
    ASX_TRY(hipMalloc((void **)&wm.blocks, sizeof(int32_t) * blk.size()));
    ASX_TRY(hipMalloc((void **)&wm.chains, sizeof(int32_t) * chains.size()));
    ASX_TRY(hipMemcpyAsync(wm.blocks, blk.data(), sizeof(int32_t) * blk.size(), hipMemcpyHostToDevice, s));
    ASX_TRY(hipMemcpyAsync(wm.chains, chains.data(), sizeof(int32_t) * chains.size(), hipMemcpyHostToDevice, s));
    ASX_TRY(hipStreamSynchronize(s));
    ASX_TRY(hipGetLastError());
    wm.has_carry = h_small[0] != 0;
#undef ASX_TRY
done:
    for (void *p : {(void *)cmin, (void *)cmax, (void *)row_start, (void *)bmin, (void *)bmax, (void *)btiles,
                    (void *)tile_off, (void *)d_small, tmp})
        if (p) (void)hipFree(p);
    if (st) {
        free_window(&wm);
        return st;
    }
    *out = wm;
    return ASX_STATUS_SUCCESS;
}

template <typename T>
int window_update_values(const WindowMatrix *wm, const T *val, hipStream_t s)
{
    const int64_t slots = (int64_t)wm->ntiles * kSlicedTile;
    if (slots == 0) return ASX_STATUS_SUCCESS;
    hipLaunchKernelGGL((k_window_regather<T>), dim3((unsigned)ceil_div64(slots, kBlock)), dim3(kBlock), 0, s, wm->perm,
                       slots, val, (T *)wm->val);
    return check_launch();
}

template <typename T>
int launch_spmv_window(int32_t m, int32_t n, T alpha, const WindowMatrix *wm, const T *x, T beta, T *y, hipStream_t s)
{
    if (m <= 0) return ASX_STATUS_SUCCESS;
    // x on a 16-byte boundary (every allocation is): 16-byte fetches; else element by element
    const auto kernel = ((uintptr_t)x % 16) == 0 ? k_spmv_window<T, kWindowWaves, true> : k_spmv_window<T, kWindowWaves, false>;
    hipLaunchKernelGGL(kernel, dim3((unsigned)wm->nchains), dim3(kWindowWaves * kWave), 0, s, n, alpha, beta,
                       reinterpret_cast<const int2 *>(wm->chains), reinterpret_cast<const int4 *>(wm->blocks), wm->cf,
                       (const T *)wm->val, reinterpret_cast<const int2 *>(wm->tile_info), x, y, (T *)wm->carry);
    if (wm->has_carry)
        hipLaunchKernelGGL((k_window_fixup<T>), dim3((unsigned)ceil_div64(wm->ntiles, kBlock)), dim3(kBlock), 0, s,
                           wm->ntiles, alpha, reinterpret_cast<const int2 *>(wm->tile_info), (const T *)wm->carry, y);
    return check_launch();
}

#define ASX_INST(T)                                                                                               \
    template int build_window<T>(int32_t, int32_t, int32_t, int32_t, const int32_t *, const int32_t *, const T *, \
                                 WindowMatrix *, hipStream_t);                                                    \
    template int window_update_values<T>(const WindowMatrix *, const T *, hipStream_t);                           \
    template int launch_spmv_window<T>(int32_t, int32_t, T, const WindowMatrix *, const T *, T, T *, hipStream_t);
ASX_INST(float)
ASX_INST(double)
#undef ASX_INST

}  // namespace asx
