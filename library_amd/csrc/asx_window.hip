// Row-block CSR SpMV with sliding windows of x in LDS, for matrices whose rows reach only
// nearby columns (stencils, banded and finite-element matrices) or a few bands of diagonals
// (stencils on three-dimensional grids).
//
// The row-ordered kernels read 4 bytes of column index per stored element, the row offsets, and
// gather x through the L2 (one request per stored element).  Here the rows are cut, once (plan
// build), into blocks of R consecutive rows whose columns all lie inside a window of fewer than
// kWindowCols columns, and consecutive blocks are chained: a workgroup walks its chain of blocks
// with LDS as a ring over the columns of x (column c lives at c mod kWindowCols), so that from
// one block to the next only the columns that are new are fetched - while the block before is
// still being multiplied - and x crosses the L2 once.  Where no such window exists but the
// stored elements lie on at most kWindowBands bands of diagonals (column minus row inside a few
// narrow intervals: the planes of a 7- or 27-point stencil), every band gets a ring of its own in
// LDS and a block fetches the new columns of every band (x then crosses the L2 once per band).
// The block's stored elements stream as tiles of 256 with a 16-bit LDS slot and a "first element
// of a row" flag per element (10 instead of 12.8 bytes per stored element in fp64; no row offsets
// are read).  Every row owns at least one slot (an empty row gets a zero that points at a zero in
// LDS), so the runs of a tile are consecutive rows and a run's sum goes straight to y.  Rows of up
// to 16 stored elements are never cut by a tile start (the tile is padded instead); a longer row
// that is cut leaves its later pieces in carry slots, which an ordered pass adds to y afterwards
// (no atomics; results are bit-reproducible).
//
// The reference has no counterpart (its CSR kernels read 32-bit columns and gather x from global
// memory: hip/kernel/level2/alphasparse_spmv_csr_vector.h:99-126).
#include <algorithm>
#include <vector>

#include "asx_internal.hpp"
#include "asx_scan.hpp"
#include "asx_tiles.hpp"

namespace asx {

namespace {

constexpr int32_t kNoCol = 0x7fffffff;
constexpr int kWindowCols = 16384;    // ring size in columns: 128 KiB of fp64, 64 KiB of fp32
constexpr int kWindowSlack = 8;       // a block's window is kept this much narrower (aligned fetches)
constexpr int kWindowWaves = 16;
constexpr int32_t kAlignRowLen = 16;  // rows up to this length are not cut by tile starts

constexpr int kSpanGroup = 128;  // rows per group of the column-span table; every block size is a multiple

// first and last column of every group of kSpanGroup consecutive rows (gmin = kNoCol, gmax = -1 for
// a group without stored elements); one wave per group, two rows per lane
__global__ __launch_bounds__(kBlock) void k_window_group_span(const int32_t *__restrict__ row_ptr,
                                                              const int32_t *__restrict__ col, int32_t m,
                                                              int32_t ngroups, int32_t *__restrict__ gmin,
                                                              int32_t *__restrict__ gmax)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t g = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    if (g >= ngroups) return;  // whole waves leave
    int32_t lo = kNoCol, hi = -1;
#pragma unroll
    for (int h = 0; h < kSpanGroup / kWave; ++h) {
        const int64_t r = g * kSpanGroup + h * kWave + lane;
        if (r < m)
            for (int32_t k = row_ptr[r]; k < row_ptr[r + 1]; ++k) {
                const int32_t c = col[k];
                lo = c < lo ? c : lo;
                hi = c > hi ? c : hi;
            }
    }
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        lo = min(lo, __shfl_xor(lo, d, kWave));
        hi = max(hi, __shfl_xor(hi, d, kWave));
    }
    if (lane == 0) {
        gmin[g] = lo;
        gmax[g] = hi;
    }
}
// Column span of every block of `per` groups; bmin / bmax are written when given; *widest receives
// (atomic max; preset to 0) the widest window a block needs once its start is rounded down to a
// multiple of 4 columns.
__global__ __launch_bounds__(kBlock) void k_window_block_span(const int32_t *__restrict__ gmin,
                                                              const int32_t *__restrict__ gmax, int32_t ngroups,
                                                              int32_t per, int32_t nblocks, int32_t *__restrict__ bmin,
                                                              int32_t *__restrict__ bmax, int32_t *__restrict__ widest)
{
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    int32_t lo = kNoCol, hi = -1;
    for (int64_t g = b * per; g < (b + 1) * per && g < ngroups; ++g) {
        lo = min(lo, gmin[g]);
        hi = max(hi, gmax[g]);
    }
    if (bmin) {
        bmin[b] = lo;
        bmax[b] = hi;
    }
    if (hi >= 0) atomicMax(widest, hi - (lo & ~3) + 1);
}
__global__ __launch_bounds__(kBlock) void k_window_fill_i32(int32_t *p, int64_t n, int32_t v)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// Slot (from the start of its block) at which every row starts, and the tiles of every block.  A
// row takes max(1, length) slots; a row of at most kAlignRowLen slots that would cross a tile
// start begins at that tile start instead.  One wave walks one block's rows in order, 64 at a time:
// starts from a scan of the lengths; at the first row of the 64 that has to move to the next tile
// the walk restarts behind that row (the rows after it shift).
__global__ __launch_bounds__(kBlock) void k_window_row_starts(const int32_t *__restrict__ row_ptr, int32_t m,
                                                              int32_t rows, int32_t nblocks,
                                                              int32_t *__restrict__ row_start,
                                                              int32_t *__restrict__ block_tiles)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t b = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    if (b >= nblocks) return;  // whole waves leave
    const int32_t r0 = (int32_t)(b * rows);
    const int32_t r1 = (int64_t)r0 + rows < m ? r0 + rows : m;
    int32_t pos = 0;
    int32_t r = r0;
    while (r < r1) {  // uniform over the wave
        const int32_t rr = r + lane;
        int32_t len = 0;
        if (rr < r1) {
            len = row_ptr[rr + 1] - row_ptr[rr];
            len = len > 0 ? len : 1;
        }
        int32_t incl = len;
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
            const int32_t t = __shfl_up(incl, d, kWave);
            if (lane >= d) incl += t;
        }
        const int32_t start = pos + incl - len;
        const bool moves = rr < r1 && len <= kAlignRowLen && start % kSlicedTile + len > kSlicedTile;
        const unsigned long long mask = __ballot(moves);
        if (mask == 0) {
            if (rr < r1) row_start[rr] = start;
            const int32_t cnt = r1 - r < kWave ? r1 - r : kWave;
            pos += __builtin_amdgcn_readlane(incl, cnt - 1);
            r += cnt;
        } else {
            const int f = __builtin_ctzll(mask);
            const int32_t moved = (__builtin_amdgcn_readlane(start, f) / kSlicedTile + 1) * kSlicedTile;
            if (lane < f) row_start[rr] = start;
            if (lane == f) row_start[rr] = moved;
            pos = moved + __builtin_amdgcn_readlane(len, f);
            r += f + 1;
        }
    }
    if (lane == 0) block_tiles[b] = (pos + kSlicedTile - 1) / kSlicedTile;
}

// The slots that hold no stored element: the slot of an empty row, the slots between a row's end
// and the start of the next one where that row was moved to a tile start, and the tail of a
// block's last tile.  Each is a zero that points at the zero behind the rings and opens a run of
// its own.  One thread per row fills what follows its own stored elements.
template <typename T>
__global__ __launch_bounds__(kBlock) void k_window_pads(const int32_t *__restrict__ row_ptr, int32_t m, int32_t rows,
                                                        const int32_t *__restrict__ row_start,
                                                        const int32_t *__restrict__ tile_off, uint16_t pad,
                                                        uint16_t *__restrict__ cf, T *__restrict__ val,
                                                        int32_t *__restrict__ perm)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= m) return;
    const int64_t b = r / rows;
    const int64_t last = (b + 1) * rows < m ? (b + 1) * rows : m;  // one past the block's last row
    const int32_t from = row_start[r] + (row_ptr[r + 1] - row_ptr[r]);
    const int32_t to = r + 1 < last ? row_start[r + 1] : (tile_off[b + 1] - tile_off[b]) * kSlicedTile;
    const int64_t base = (int64_t)tile_off[b] * kSlicedTile;
    for (int32_t o = from; o < to; ++o) {
        const int64_t d = base + o;
        const int64_t phys = d / kSlicedTile * kSlicedTile + tile_val_pos<T>((int)(d % kSlicedTile));
        cf[d] = pad;
        val[phys] = T(0);
        perm[phys] = -1;
    }
}

// Where the columns of x live in LDS.  One band (nbands = 1): column c at c mod kWindowCols.
// Several: the stored elements whose offset from the diagonal, c - floor(r n / m), lies in
// [dlo[k], dhi[k]] use ring k: column c at base[k] + c mod width[k].
struct BandTable {
    int32_t nbands;
    int32_t dlo[kWindowBands], dhi[kWindowBands], base[kWindowBands], width[kWindowBands];
};
__host__ __device__ __forceinline__ int64_t band_centre(int64_t r, int64_t m, int64_t n) { return r * n / m; }

// bit b of `bits` set = some stored element has (c - centre(r) + n) / 64 == b
__global__ __launch_bounds__(kBlock) void k_window_offset_bins(const int32_t *__restrict__ row_ptr,
                                                               const int32_t *__restrict__ col, int32_t m, int32_t n,
                                                               uint32_t *__restrict__ bits)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= m) return;
    const int64_t shift = (int64_t)n - band_centre(r, m, n);
    int64_t last = -1;
    for (int32_t k = row_ptr[r]; k < row_ptr[r + 1]; ++k) {
        const int64_t bin = ((int64_t)col[k] + shift) >> 6;
        if (bin == last) continue;
        last = bin;
        const uint32_t mask = 1u << (bin & 31);
        if (!(bits[bin >> 5] & mask)) atomicOr(bits + (bin >> 5), mask);  // mostly set already: few atomics
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_window_place(const int32_t *__restrict__ row_ptr,
                                                         const int32_t *__restrict__ col, const T *__restrict__ val,
                                                         int32_t m, int32_t n, int32_t nnz, int32_t rows, BandTable bands,
                                                         const int32_t *__restrict__ seg_row,
                                                         const int32_t *__restrict__ row_start,
                                                         const int32_t *__restrict__ tile_off, uint16_t *__restrict__ cf,
                                                         T *__restrict__ val_out, int32_t *__restrict__ perm)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    // row holding stored element i: largest r with row_ptr[r] <= i; the workgroup's kBlock elements
    // lie in rows seg_row[blockIdx.x] .. seg_row[blockIdx.x + 1]
    int32_t lo = seg_row[blockIdx.x], hi = seg_row[blockIdx.x + 1];
    hi = hi > m - 1 ? m - 1 : hi;
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
    const int32_t c = col[i];
    int k = 0;
    if (bands.nbands > 1) {
        const int64_t off = (int64_t)c - band_centre(r, m, n);
        for (int j = 1; j < kWindowBands; ++j)
            if (j < bands.nbands && off >= bands.dlo[j]) k = j;  // bands ascend and cover every offset
    }
    const int32_t slot = bands.base[k] + c % bands.width[k];
    cf[d] = (uint16_t)(slot | (head ? 0x8000 : 0));
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

// The pieces of x a block needs before it is multiplied (at most kWindowBands ranges of columns
// [from, to), from a multiple of 4, together at most kWindowCols columns; ring of piece q: slots
// base .. base + width) into registers, one 16-byte unit per thread and step, and later from the
// registers into the rings.  Columns at or past n read as 0.  Every register is written by one
// load instruction only (predicated, after a zero fill), never by two alternative ones: with
// alternatives the compiler orders them with a full s_waitcnt between the steps and the fetch
// takes one memory round trip per step.  VEC (x on a 16-byte boundary, n at least one unit): one
// 16-byte load per unit; the unit that straddles the end of x is read from the last whole unit
// inside x (an unaligned address) and shifted into place when it is stored.  Otherwise element by
// element.  NB = 1: one piece, ring of kWindowCols slots from slot 0 (no piece search, constant modulus).
template <typename T, int THREADS, bool VEC, int NB>
struct XFetch {
    static constexpr int V = 16 / sizeof(T);
    static constexpr int PER = kWindowCols / (THREADS * V);
    typedef T vec_t __attribute__((ext_vector_type(V)));
    typedef vec_t vec_u __attribute__((aligned(sizeof(T))));
    vec_t buf[PER];
    // the pending fetch (uniform values): its pieces, the first unit of each and the ring slot of
    // its first column
    int32_t from[NB], to[NB], base[NB], width[NB], ustart[NB], fslot[NB];

    __device__ __forceinline__ void set(const int4 *__restrict__ pieces, int32_t lo, int32_t hi)
    {
        int32_t u = 0;
#pragma unroll
        for (int q = 0; q < NB; ++q) {
            int4 pc = make_int4(0, 0, 0, 4);
            if (lo + q < hi) pc = pieces[lo + q];  // uniform
            from[q] = __builtin_amdgcn_readfirstlane(pc.x);
            to[q] = __builtin_amdgcn_readfirstlane(pc.y);
            base[q] = NB == 1 ? 0 : __builtin_amdgcn_readfirstlane(pc.z);
            width[q] = NB == 1 ? kWindowCols : __builtin_amdgcn_readfirstlane(pc.w);
            fslot[q] = (int32_t)((uint32_t)from[q] % (uint32_t)width[q]);
            ustart[q] = u;
            u += (to[q] - from[q] + V - 1) / V;
        }
    }
    // unit u: first column, end of its piece, LDS slot (a unit past the last piece lands at or past
    // `to` of the last one).  A piece is no longer than its ring, so one wrap suffices.
    __device__ __forceinline__ void locate(int32_t u, int32_t &c, int32_t &c_to, int32_t &slot) const
    {
        int32_t f = from[0], s = 0, fs = fslot[0], b = base[0], w = width[0];
        c_to = to[0];
#pragma unroll
        for (int q = 1; q < NB; ++q) {
            const bool in = u >= ustart[q];
            f = in ? from[q] : f;
            s = in ? ustart[q] : s;
            fs = in ? fslot[q] : fs;
            b = in ? base[q] : b;
            w = in ? width[q] : w;
            c_to = in ? to[q] : c_to;
        }
        const int32_t off = (u - s) * V;
        c = f + off;
        const int32_t sl = fs + off;
        slot = b + (sl >= w ? sl - w : sl);
    }
    __device__ __forceinline__ void load(const T *__restrict__ x, int32_t n)
    {
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            int32_t c, c_to, slot;
            locate(k * THREADS + (int)threadIdx.x, c, c_to, slot);
            buf[k] = vec_t(T(0));
            if (VEC) {
                if (c < c_to && c < n) buf[k] = *reinterpret_cast<const vec_u *>(x + (n - c >= V ? (int64_t)c : (int64_t)n - V));
            } else {
#pragma unroll
                for (int e = 0; e < V; ++e)
                    if (c_to - c > e && n - c > e) buf[k][e] = x[(int64_t)c + e];
            }
        }
    }
    __device__ __forceinline__ void store(T *xs, int32_t n) const
    {
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            int32_t c, c_to, slot;
            locate(k * THREADS + (int)threadIdx.x, c, c_to, slot);
            if (c < c_to) {
                vec_t v = buf[k];
                if (VEC && c < n && n - c < V) {
                    // holds x[n - V .. n): the columns c .. n - 1 move to the front, zeros behind them
                    const int cnt = n - c;
                    vec_t w = vec_t(T(0));
#pragma unroll
                    for (int e = 0; e < V - 1; ++e)
#pragma unroll
                        for (int j = 1; j < V; ++j)
                            if (e < cnt && j == V - cnt + e) w[e] = v[j];
                    v = w;
                }
                *reinterpret_cast<vec_t *>(xs + slot) = v;
            }
        }
    }
};

template <typename T, int NW, bool VEC, int NB, int D>
__global__ __launch_bounds__(NW *kWave) void k_spmv_window(int32_t n, T alpha, T beta, const int2 *__restrict__ chains,
                                                           const int4 *__restrict__ blocks,
                                                           const int4 *__restrict__ pieces,
                                                           const uint16_t *__restrict__ cf, const T *__restrict__ val,
                                                           const int2 *__restrict__ tile_info,
                                                           const T *__restrict__ x, T *__restrict__ y,
                                                           T *__restrict__ carry)
{
    // the rings over the columns of x, then the zero the pads point at
    __shared__ __align__(16) T xs[kWindowCols + 16 / sizeof(T)];
    __shared__ T stage_all[NW * kStageRows];
    const int2 chain = chains[blockIdx.x];  // first block, end block
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    T *stage = stage_all + wave * kStageRows;
    const int32_t chain_last = blocks[chain.y - 1].y - 1;  // last tile of the chain
    // this wave's tiles are those congruent to its number, across the blocks of the chain; D are
    // in flight (loaded D steps ahead; past the end of the chain the last tile is re-read)
    WindowTile<T> tl[D];
    int32_t t = blocks[chain.x].x + wave;
#pragma unroll
    for (int d = 0; d < D; ++d)
        window_tile_load<T>(tl[d], t + d * NW < chain_last ? t + d * NW : chain_last, lane, cf, val, tile_info);
    if (threadIdx.x == 0) xs[kWindowCols] = T(0);
    XFetch<T, NW * kWave, VEC, NB> xf;
    int4 blk = blocks[chain.x];  // first tile, end tile, pieces of x to fetch before the block: first, end
    xf.set(pieces, blk.z, blk.w);
    xf.load(x, n);
    int32_t b = chain.x, tile_hi;
    // Start of block b: the columns fetched for it go into the ring once every wave is done with
    // the block before; the next block's new columns are fetched while this one is multiplied.
#define ASX_BLOCK_BEGIN()                      \
    {                                          \
        __syncthreads();                       \
        xf.store(xs, n);                       \
        __syncthreads();                       \
        tile_hi = blk.y;                       \
        if (b + 1 < chain.y) {                 \
            blk = blocks[b + 1];               \
            xf.set(pieces, blk.z, blk.w);      \
            xf.load(x, n);                     \
        }                                      \
    }
#define ASX_NEXT(TL, TT) window_tile_load<T>(TL, (TT) < chain_last ? (TT) : chain_last, lane, cf, val, tile_info)
    // one tile: its rows' sums into the staging area, the loads of the tile D steps ahead (into
    // the registers this one has just left), then the staged sums to y
#define ASX_STEP(TL, TT)                                                                                          \
    {                                                                                                             \
        const StoreRows<T> out{y, carry + (TT), stage, TL.base & 0x7fffffff, TL.limit, TL.base < 0, alpha, beta}; \
        tile_reduce<T>(TL, lane, xs, out);                                                                        \
        ASX_NEXT(TL, (TT) + D * NW);                                                                              \
        out.flush(lane);                                                                                          \
    }
    // Every wave passes the start of every block of the chain (the barriers count all waves),
    // whether it has tiles in the block or not.  The D tile buffers take turns without changing
    // places (the loop over them is unrolled).
    ASX_BLOCK_BEGIN()
    for (;;) {  // all conditions are uniform over the wave
#pragma unroll
        for (int d = 0; d < D; ++d) {
            while (t >= tile_hi) {
                if (++b >= chain.y) return;
                ASX_BLOCK_BEGIN()
            }
            ASX_STEP(tl[d], t);
            t += NW;
        }
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
    for (void *q : {p->store, p->tables, p->carry})
        if (q) (void)hipFree(q);
    p->store = p->tables = p->val = p->carry = nullptr;
    p->cf = nullptr;
    p->perm = p->tile_info = p->blocks = p->pieces = p->chains = nullptr;
}

template <typename T>
int build_window(int32_t m, int32_t n, int32_t nnz, int32_t target_wgs, const int32_t *row_ptr, const int32_t *col,
                 const T *val, WindowMatrix *out, hipStream_t s)
{
    WindowMatrix wm{};
    if (m <= 0 || nnz <= 0 || n <= 0) return ASX_STATUS_INVALID_SIZE;
    if (target_wgs < 1) return ASX_STATUS_INVALID_VALUE;
    int st = ASX_STATUS_SUCCESS;
    int32_t *arena = nullptr;
    int32_t *gmin = nullptr, *gmax = nullptr, *row_start = nullptr, *seg_row = nullptr;
    int32_t *bmin = nullptr, *bmax = nullptr, *btiles = nullptr, *tile_off = nullptr, *d_small = nullptr;
    int32_t *tmp = nullptr;
    std::vector<int32_t> h_bmin, h_bmax, h_off, blk, pcs, chains;
    std::vector<uint32_t> h_bits;
    uint32_t *d_bits = nullptr;
    BandTable bands{};
    int64_t slots = 0;
    constexpr int kCandidates = 11;
    static const int32_t kBlockRows[kCandidates] = {8192, 6144, 4096, 3072, 2048, 1536, 1024, 768, 512, 384, 256};
    int32_t h_small[16] = {0};
    const unsigned mgrid = (unsigned)ceil_div64(m, kBlock);
    const int32_t min_blocks = 4 * target_wgs;  // larger blocks only while at least this many blocks remain
    const int32_t max_nb = (int32_t)ceil_div64(m, 256);
    const int32_t ngroups = (int32_t)ceil_div64(m, kSpanGroup);
    const int32_t nseg = (int32_t)ceil_div64(nnz, kBlock);
#define ASX_TRY(expr)         \
    do {                      \
        st = status_of(expr); \
        if (st) goto done;    \
    } while (0)
    // the scratch of the build in one allocation: the span of every group of rows (two arrays), where
    // every row starts, the row holding every 256th stored element, four arrays of max_nb + 1, a
    // few counters, the scan's block sums
    {
        const auto pad64 = [](size_t v) { return (v + 63) & ~(size_t)63; };
        const size_t per_group = pad64((size_t)ngroups), per_row = pad64((size_t)m), per_seg = pad64((size_t)nseg + 1);
        const size_t per_block = pad64((size_t)max_nb + 1);
        ASX_TRY(hipMalloc((void **)&arena, sizeof(int32_t) * (2 * per_group + per_row + per_seg + 4 * per_block + 64 +
                                                              scan_scratch_ints((int64_t)max_nb + 1))));
        gmin = arena, gmax = gmin + per_group, row_start = gmax + per_group, seg_row = row_start + per_row;
        bmin = seg_row + per_seg, bmax = bmin + per_block, btiles = bmax + per_block, tile_off = btiles + per_block;
        d_small = tile_off + per_block;
        tmp = d_small + 64;
    }

    // 1. column span of every group of rows
    hipLaunchKernelGGL(k_window_group_span, dim3((unsigned)ceil_div64((int64_t)ngroups * kWave, kBlock)), dim3(kBlock), 0, s,
                       row_ptr, col, m, ngroups, gmin, gmax);
    // 2. the largest block of rows whose widest window fits the ring: the widest window of every
    //    candidate size, all read back at once
    hipLaunchKernelGGL(k_window_fill_i32, dim3(1), dim3(kBlock), 0, s, d_small, (int64_t)16, 0);
    for (int k = 0; k < kCandidates; ++k) {
        const int32_t rows = kBlockRows[k];
        if (rows > 256 && ceil_div64(m, rows) < min_blocks) continue;  // too few blocks to share out
        const int32_t nb = (int32_t)ceil_div64(m, rows);
        hipLaunchKernelGGL(k_window_block_span, dim3((unsigned)ceil_div64(nb, kBlock)), dim3(kBlock), 0, s, gmin, gmax, ngroups,
                           rows / kSpanGroup, nb, (int32_t *)nullptr, (int32_t *)nullptr, d_small + k);
    }
    st = launch_nnz_split_rows(row_ptr, m, nnz, kBlock, seg_row, s);  // for step 4; runs while the host waits
    if (st) goto done;
    ASX_TRY(hipMemcpyAsync(h_small, d_small, sizeof(int32_t) * kCandidates, hipMemcpyDeviceToHost, s));
    ASX_TRY(hipStreamSynchronize(s));
    wm.rows_per_block = 0;
    for (int k = 0; k < kCandidates; ++k) {
        const int32_t rows = kBlockRows[k];
        if (rows > 256 && ceil_div64(m, rows) < min_blocks) continue;
        if (h_small[k] <= kWindowCols - kWindowSlack) {
            wm.rows_per_block = rows;
            wm.nblocks = (int32_t)ceil_div64(m, rows);
            hipLaunchKernelGGL(k_window_block_span, dim3((unsigned)ceil_div64(wm.nblocks, kBlock)), dim3(kBlock), 0, s, gmin,
                               gmax, ngroups, rows / kSpanGroup, wm.nblocks, bmin, bmax, d_small + 15);
            break;
        }
    }
    bands.nbands = 1;
    bands.base[0] = 0;
    bands.width[0] = kWindowCols;
    if (wm.rows_per_block == 0) {
        // 2b. some 256 rows reach further than the ring.  Bands of diagonals instead: which offsets
        //     c - centre(r) occur (a bit per 64 of them), the runs of occupied offsets, and the
        //     largest block whose bands (block's advance along the diagonal + width of the run) fit
        //     the LDS together.  More runs than rings: the closest runs are joined.
        const int64_t nbins = (2 * (int64_t)n >> 6) + 2;
        const size_t words = (size_t)(nbins + 31) / 32;
        ASX_TRY(hipMalloc((void **)&d_bits, sizeof(uint32_t) * words));
        ASX_TRY(hipMemsetAsync(d_bits, 0, sizeof(uint32_t) * words, s));
        hipLaunchKernelGGL(k_window_offset_bins, dim3(mgrid), dim3(kBlock), 0, s, row_ptr, col, m, n, d_bits);
        h_bits.resize(words);
        ASX_TRY(hipMemcpyAsync(h_bits.data(), d_bits, sizeof(uint32_t) * words, hipMemcpyDeviceToHost, s));
        ASX_TRY(hipStreamSynchronize(s));
        std::vector<std::pair<int64_t, int64_t>> runs;  // first and last occupied bin
        for (int64_t b = 0; b < nbins; ++b) {
            if (!(h_bits[(size_t)(b >> 5)] >> (b & 31) & 1u)) continue;
            if (!runs.empty() && runs.back().second + 1 >= b)
                runs.back().second = b;
            else
                runs.emplace_back(b, b);
        }
        while ((int)runs.size() > kWindowBands) {  // join the two runs with the smallest gap
            size_t best = 0;
            for (size_t i = 1; i + 1 < runs.size(); ++i)
                if (runs[i + 1].first - runs[i].second < runs[best + 1].first - runs[best].second) best = i;
            runs[best].second = runs[best + 1].second;
            runs.erase(runs.begin() + (long)best + 1);
        }
        // one run of offsets: the rows fill a band too wide for the single window tried above
        // (the one-ring kernel places column c at c mod kWindowCols; it is not built from here)
        if (runs.size() < 2) {
            st = ASX_STATUS_NOT_SUPPORTED;
            goto done;
        }
        bands.nbands = (int32_t)runs.size();
        for (int k = 0; k < bands.nbands; ++k) {
            bands.dlo[k] = (int32_t)std::max<int64_t>((runs[(size_t)k].first << 6) - n, -(int64_t)n);
            bands.dhi[k] = (int32_t)std::min<int64_t>(((runs[(size_t)k].second + 1) << 6) - 1 - n, n);
        }
        for (int32_t rows : {8192, 7168, 6144, 5120, 4608, 4096, 3584, 3072, 2560, 2048, 1792, 1536, 1280, 1024, 768, 512, 384, 256}) {
            if (rows > 256 && ceil_div64(m, rows) < min_blocks) continue;
            const int64_t advance = ceil_div64((int64_t)rows * n, m) + 1;  // of the centre over a block
            int64_t total = 0;
            for (int k = 0; k < bands.nbands; ++k)
                total += (advance + ((int64_t)bands.dhi[k] - bands.dlo[k]) + 1 + kWindowSlack + 3 + 3) & ~(int64_t)3;
            if (total > kWindowCols) continue;
            wm.rows_per_block = rows;
            wm.nblocks = (int32_t)ceil_div64(m, rows);
            int32_t at = 0;
            for (int k = 0; k < bands.nbands; ++k) {
                bands.base[k] = at;
                bands.width[k] = (int32_t)((advance + ((int64_t)bands.dhi[k] - bands.dlo[k]) + 1 + kWindowSlack + 3 + 3) & ~(int64_t)3);
                at += bands.width[k];
            }
            break;
        }
        if (wm.rows_per_block == 0) {
            st = ASX_STATUS_NOT_SUPPORTED;  // the bands of 256 rows do not fit the LDS: not this kernel's matrix
            goto done;
        }
    }
    wm.nbands = bands.nbands;
    // 3. where every row starts inside its block; tiles of every block
    hipLaunchKernelGGL(k_window_row_starts, dim3((unsigned)ceil_div64((int64_t)wm.nblocks * kWave, kBlock)), dim3(kBlock), 0, s, row_ptr, m,
                       wm.rows_per_block, wm.nblocks, row_start, btiles);
    ASX_TRY(hipMemsetAsync(btiles + wm.nblocks, 0, sizeof(int32_t), s));
    st = launch_exclusive_scan_i32(btiles, tile_off, (int64_t)wm.nblocks + 1, tmp, s);
    if (st) goto done;
    h_bmin.resize((size_t)wm.nblocks);
    h_bmax.resize((size_t)wm.nblocks);
    h_off.resize((size_t)wm.nblocks + 1);
    if (bands.nbands == 1) {
        ASX_TRY(hipMemcpyAsync(h_bmin.data(), bmin, sizeof(int32_t) * h_bmin.size(), hipMemcpyDeviceToHost, s));
        ASX_TRY(hipMemcpyAsync(h_bmax.data(), bmax, sizeof(int32_t) * h_bmax.size(), hipMemcpyDeviceToHost, s));
    }
    ASX_TRY(hipMemcpyAsync(h_off.data(), tile_off, sizeof(int32_t) * h_off.size(), hipMemcpyDeviceToHost, s));
    ASX_TRY(hipStreamSynchronize(s));
    wm.ntiles = h_off[(size_t)wm.nblocks];
    slots = (int64_t)wm.ntiles * kSlicedTile;
    if (slots > 0x7fffffff) {
        st = ASX_STATUS_INVALID_SIZE;
        goto done;
    }
    {   // the regrouped copy in one allocation
        const size_t o_val = 0, o_perm = align_up(sizeof(T) * (size_t)slots, 256);
        const size_t o_cf = o_perm + align_up(sizeof(int32_t) * (size_t)slots, 256);
        const size_t o_info = o_cf + align_up(sizeof(uint16_t) * (size_t)slots, 256);
        ASX_TRY(hipMalloc(&wm.store, o_info + sizeof(int2) * (size_t)wm.ntiles));
        char *base = static_cast<char *>(wm.store);
        wm.val = base + o_val, wm.perm = (int32_t *)(base + o_perm), wm.cf = (uint16_t *)(base + o_cf);
        wm.tile_info = (int32_t *)(base + o_info);
    }
    ASX_TRY(hipMalloc(&wm.carry, sizeof(T) * (size_t)wm.ntiles));
    // 4. every stored element to its slot; every other slot becomes a zero that points at the zero
    //    behind the rings and opens a run of its own
    hipLaunchKernelGGL((k_window_place<T>), dim3((unsigned)ceil_div64(nnz, kBlock)), dim3(kBlock), 0, s, row_ptr, col, val,
                       m, n, nnz, wm.rows_per_block, bands, seg_row, row_start, tile_off, wm.cf, (T *)wm.val, wm.perm);
    hipLaunchKernelGGL((k_window_pads<T>), dim3(mgrid), dim3(kBlock), 0, s, row_ptr, m, wm.rows_per_block, row_start, tile_off,
                       (uint16_t)(0x8000 | kWindowCols), wm.cf, (T *)wm.val, wm.perm);
    // 5. first row and number of rows of every tile
    hipLaunchKernelGGL(k_window_fill_i32, dim3(1), dim3(kBlock), 0, s, d_small, (int64_t)2, 0);
    hipLaunchKernelGGL(k_window_tile_info, dim3((unsigned)ceil_div64(wm.ntiles, kBlock)), dim3(kBlock), 0, s, row_start, m,
                       wm.rows_per_block, wm.nblocks, tile_off, wm.ntiles, (int2 *)wm.tile_info, d_small);
    ASX_TRY(hipMemcpyAsync(h_small, d_small, sizeof(int32_t), hipMemcpyDeviceToHost, s));
    // 6. chains of blocks, one per workgroup, of about equal numbers of tiles.  Inside a chain a
    //    block fetches, per band, only the columns behind those already in the band's ring; a block
    //    whose columns start before what a ring still holds begins a new chain (and fetches its
    //    whole windows).
    {
        const int64_t per_chain = std::max<int64_t>(1, ceil_div64(wm.ntiles, target_wgs));
        blk.resize((size_t)wm.nblocks * 4);
        int64_t have[kWindowBands];  // columns [low, have) were fetched in this chain (have = -1: nothing yet)
        int64_t low[kWindowBands];
        for (int k = 0; k < kWindowBands; ++k) have[k] = -1, low[k] = 0;
        int32_t chain_lo = 0;
        int64_t chain_tiles = 0;
        for (int32_t b = 0; b < wm.nblocks; ++b) {
            // columns the block needs in every band, rounded to multiples of 4: [lo, hi)
            int64_t lo[kWindowBands], hi[kWindowBands];
            const int64_t r0 = (int64_t)b * wm.rows_per_block, r1 = std::min<int64_t>(r0 + wm.rows_per_block, m);
            for (int k = 0; k < bands.nbands; ++k) {
                if (bands.nbands == 1) {
                    const bool empty = h_bmax[(size_t)b] < 0;
                    lo[k] = empty ? 0 : (h_bmin[(size_t)b] & ~3);
                    hi[k] = empty ? 0 : ((int64_t)h_bmax[(size_t)b] + 4) & ~(int64_t)3;  // past the last, rounded up
                } else {
                    const int64_t a = std::min<int64_t>(std::max<int64_t>(band_centre(r0, m, n) + bands.dlo[k], 0), n);
                    const int64_t z = std::min<int64_t>(std::max<int64_t>(band_centre(r1 - 1, m, n) + bands.dhi[k] + 1, 0), n);
                    lo[k] = a & ~(int64_t)3;
                    hi[k] = z > a ? (z + 3) & ~(int64_t)3 : lo[k];
                }
            }
            bool fresh = false;
            if (b != chain_lo) {
                for (int k = 0; k < bands.nbands; ++k)  // columns never fetched in this chain, or already overwritten
                    if (hi[k] > lo[k] && have[k] >= 0 &&
                        (lo[k] < low[k] || lo[k] < std::max(have[k], hi[k]) - bands.width[k] + kWindowSlack))
                        fresh = true;
                if (chain_tiles >= per_chain) fresh = true;
            }
            if (fresh) {
                chains.push_back(chain_lo);
                chains.push_back(b);
                chain_lo = b;
                chain_tiles = 0;
                for (int k = 0; k < kWindowBands; ++k) have[k] = -1, low[k] = 0;
            }
            blk[(size_t)b * 4 + 0] = h_off[(size_t)b];
            blk[(size_t)b * 4 + 1] = h_off[(size_t)b + 1];
            blk[(size_t)b * 4 + 2] = (int32_t)(pcs.size() / 4);
            for (int k = 0; k < bands.nbands; ++k) {
                int64_t from = lo[k], to = lo[k];
                if (hi[k] > lo[k]) {
                    if (have[k] < 0 || lo[k] >= have[k]) {  // nothing useful in the ring: the whole window
                        from = lo[k];
                        to = hi[k];
                        low[k] = lo[k];
                    } else {
                        from = have[k];
                        to = std::max(have[k], hi[k]);
                    }
                    have[k] = to;
                }
                pcs.push_back((int32_t)from);
                pcs.push_back((int32_t)to);
                pcs.push_back(bands.base[k]);
                pcs.push_back(bands.width[k]);
            }
            blk[(size_t)b * 4 + 3] = (int32_t)(pcs.size() / 4);
            chain_tiles += h_off[(size_t)b + 1] - h_off[(size_t)b];
        }
        chains.push_back(chain_lo);
        chains.push_back(wm.nblocks);
        wm.nchains = (int32_t)(chains.size() / 2);
        wm.npieces = (int32_t)(pcs.size() / 4);
    }
    {   // the tables of the blocks in one allocation (16-byte entries first)
        const size_t o_pieces = align_up(sizeof(int32_t) * blk.size(), 256);
        const size_t o_chains = o_pieces + align_up(sizeof(int32_t) * pcs.size(), 256);
        ASX_TRY(hipMalloc(&wm.tables, o_chains + sizeof(int32_t) * chains.size()));
        char *base = static_cast<char *>(wm.tables);
        wm.blocks = (int32_t *)base, wm.pieces = (int32_t *)(base + o_pieces), wm.chains = (int32_t *)(base + o_chains);
    }
    ASX_TRY(hipMemcpyAsync(wm.pieces, pcs.data(), sizeof(int32_t) * pcs.size(), hipMemcpyHostToDevice, s));
    ASX_TRY(hipMemcpyAsync(wm.blocks, blk.data(), sizeof(int32_t) * blk.size(), hipMemcpyHostToDevice, s));
    ASX_TRY(hipMemcpyAsync(wm.chains, chains.data(), sizeof(int32_t) * chains.size(), hipMemcpyHostToDevice, s));
    ASX_TRY(hipStreamSynchronize(s));
    ASX_TRY(hipGetLastError());
    wm.has_carry = h_small[0] != 0;
#undef ASX_TRY
done:
    for (void *p : {(void *)arena, (void *)d_bits})
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
int launch_spmv_window(int32_t m, int32_t n, T alpha, const WindowMatrix *wm, const T *x, T beta, T *y, T *carry,
                       hipStream_t s)
{
    if (m <= 0) return ASX_STATUS_SUCCESS;
    if (wm->has_carry && !carry) return ASX_STATUS_INVALID_POINTER;
    // x on a 16-byte boundary (every allocation is) and at least one 16-byte unit long: 16-byte
    // fetches; else element by element
    const bool vec = ((uintptr_t)x % 16) == 0 && (size_t)n * sizeof(T) >= 16;
    // tiles in flight per wave: three with one window (measured 1-2 % ahead of two); two with bands,
    // where three no longer fit the 128 registers a lane of a 1024-thread workgroup may use
    const auto kernel = wm->nbands == 1
                            ? (vec ? k_spmv_window<T, kWindowWaves, true, 1, 3> : k_spmv_window<T, kWindowWaves, false, 1, 3>)
                            : (vec ? k_spmv_window<T, kWindowWaves, true, kWindowBands, 2>
                                   : k_spmv_window<T, kWindowWaves, false, kWindowBands, 2>);
    hipLaunchKernelGGL(kernel, dim3((unsigned)wm->nchains), dim3(kWindowWaves * kWave), 0, s, n, alpha, beta,
                       reinterpret_cast<const int2 *>(wm->chains), reinterpret_cast<const int4 *>(wm->blocks),
                       reinterpret_cast<const int4 *>(wm->pieces), wm->cf, (const T *)wm->val,
                       reinterpret_cast<const int2 *>(wm->tile_info), x, y, carry);
    if (wm->has_carry)
        hipLaunchKernelGGL((k_window_fixup<T>), dim3((unsigned)ceil_div64(wm->ntiles, kBlock)), dim3(kBlock), 0, s,
                           wm->ntiles, alpha, reinterpret_cast<const int2 *>(wm->tile_info), (const T *)carry, y);
    return check_launch();
}

#define ASX_INST(T)                                                                                               \
    template int build_window<T>(int32_t, int32_t, int32_t, int32_t, const int32_t *, const int32_t *, const T *, \
                                 WindowMatrix *, hipStream_t);                                                    \
    template int window_update_values<T>(const WindowMatrix *, const T *, hipStream_t);                           \
    template int launch_spmv_window<T>(int32_t, int32_t, T, const WindowMatrix *, const T *, T, T *, T *, hipStream_t);
ASX_INST(float)
ASX_INST(double)
#undef ASX_INST

}  // namespace asx
