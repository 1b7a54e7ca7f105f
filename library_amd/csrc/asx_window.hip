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
// LDS and a block fetches the new columns of every band (x then crosses the L2 once per band);
// three bands a whole number of planes apart share three regions of LDS that take turns, the
// blocks of a chain climb the planes, and x crosses the L2 about once (see BandTable).
// The block's stored elements stream as tiles of 256 with a 16-bit LDS slot and a "first element
// of a row" flag per element (10 instead of 12.8 bytes per stored element in fp64; no row offsets
// are read).  Every row owns at least two slots (what its stored elements leave free holds zeros
// that point at a zero in LDS), so the runs of a tile are consecutive rows, at most 128 of them,
// and a run's sum goes straight to y.  Rows of up
// to 16 stored elements are never cut by a tile start (the tile is padded instead); a longer row
// that is cut leaves its later pieces in carry slots, which an ordered pass adds to y afterwards
// (no atomics; results are bit-reproducible).
//
// The reference has no counterpart (its CSR kernels read 32-bit columns and gather x from global
// memory: hip/kernel/level2/alphasparse_spmv_csr_vector.h:99-126).
#include <algorithm>
#include <vector>

#include "asx_internal.hpp"
#include "asx_tiles.hpp"

namespace asx {

namespace {

constexpr int32_t kNoCol = 0x7fffffff;
constexpr int kWindowCols = 16384;    // ring size in columns: 128 KiB of fp64, 64 KiB of fp32
constexpr int kWindowSlack = 8;       // a block's window is kept this much narrower (aligned fetches)
constexpr int kFetchCols = 8192;     // columns of x a block past the first of its chain may fetch
constexpr int kWindowWaves = 16;
constexpr int32_t kAlignRowLen = 16;  // rows up to this length are not cut by tile starts
constexpr int32_t kMinRowSlots = 2;   // slots a row takes at least

// Tiles in flight per wave: as many as the 128 registers a lane of a 1024-thread workgroup may use
// hold beside the columns of x on their way to LDS (the compiler spills those first)
template <typename T>
constexpr int window_depth(int rings, bool beta)
{
    return rings > 1 ? 2 : sizeof(T) == 8 ? 2 : 3;
}
constexpr int kSpanGroup = 128;  // rows per group of the column-span table; every block size is a multiple

// first and last column of every group of kSpanGroup consecutive rows (gmin = kNoCol, gmax = -1 for
// a group without stored elements); one wave per group reads the group's columns in order.
// *any_short (preset to 0) becomes 1 when a row holds fewer than kMinRowSlots stored elements.
__global__ __launch_bounds__(kBlock) void k_window_group_span(const int32_t *__restrict__ row_ptr,
                                                              const int32_t *__restrict__ col, int32_t m,
                                                              int32_t ngroups, int32_t *__restrict__ gmin,
                                                              int32_t *__restrict__ gmax, int32_t *__restrict__ any_short)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t g = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    if (g >= ngroups) return;  // whole waves leave
    int32_t lo = kNoCol, hi = -1;
    const int64_t r1 = (g + 1) * kSpanGroup < m ? (g + 1) * kSpanGroup : m;
    bool is_short = false;  // a row of fewer than kMinRowSlots stored elements: it will be padded
    for (int64_t r = g * kSpanGroup + lane; r < r1; r += kWave) is_short |= row_ptr[r + 1] - row_ptr[r] < kMinRowSlots;
    if (is_short) *any_short = 1;
    for (int32_t k = row_ptr[g * kSpanGroup] + lane, end = row_ptr[r1]; k < end; k += kWave) {
        const int32_t c = col[k];
        lo = c < lo ? c : lo;
        hi = c > hi ? c : hi;
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
// row takes max(kMinRowSlots, length) slots (a tile of 256 slots then holds at most 128 rows, which
// is what a wave stages and stores per tile); a row of at most kAlignRowLen slots that would cross
// a tile start begins at that tile start instead.  One wave walks one block's rows in order, 64 at a time:
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
            len = len > kMinRowSlots ? len : kMinRowSlots;
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

// The slots that hold no stored element: the slots of an empty row, the second slot of a row with
// one stored element, the slots between a row's end and the start of the next one where that row
// was moved to a tile start, and the tail of a block's last tile.  Each is a zero that points at the
// zero behind the rings; the first slot of an empty row opens the row's run, a slot that makes a row
// up to kMinRowSlots belongs to that run, every other one opens a run of its own.  One thread per
// row fills what follows its own stored elements.
template <typename T>
__global__ __launch_bounds__(kBlock) void k_window_pads(const int32_t *__restrict__ row_ptr, int32_t m, int32_t rows,
                                                        const int32_t *__restrict__ row_start,
                                                        const int32_t *__restrict__ tile_off,
                                                        const int32_t *__restrict__ block_tiles, uint16_t pad,
                                                        uint16_t *__restrict__ cf, T *__restrict__ val,
                                                        int32_t *__restrict__ perm, bool halves)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= m) return;
    const int64_t b = r / rows;
    const int64_t last = (b + 1) * rows < m ? (b + 1) * rows : m;  // one past the block's last row
    const int32_t len = row_ptr[r + 1] - row_ptr[r];
    const int32_t from = row_start[r] + len;
    const int32_t own = row_start[r] + (len > kMinRowSlots ? len : kMinRowSlots);  // end of the row's own slots
    const int32_t to = r + 1 < last ? row_start[r + 1] : block_tiles[b] * kSlicedTile;
    const int64_t base = (int64_t)tile_off[b] * kSlicedTile;
    for (int32_t o = from; o < to; ++o) {
        const int64_t d = base + o;
        const int64_t phys = d / kSlicedTile * kSlicedTile + tile_val_pos<T>((int)(d % kSlicedTile));
        cf[halves ? d / kSlicedTile * kSlicedTile + tile_halves_pos((int)(d % kSlicedTile)) : d] =
            o < own && o > row_start[r] ? (uint16_t)(pad & 0x7fff) : pad;
        if (val) {  // uniform: no copy of the values when the kernel reads A's in place
            val[phys] = T(0);
            perm[phys] = -1;
        }
    }
}

// Where the columns of x live in LDS.  One band (nbands = 1): column c at c mod kWindowCols.
// Several: the stored elements whose offset from the diagonal, c - floor(r n / m), lies in
// [dlo[k], dhi[k]] use ring k: column c at base[k] + c mod width[k].
// Stacked planes (stack_rows = P > 0; three bands whose centres lie -P, 0 and +P from the diagonal, as
// in a stencil on a three-dimensional grid whose planes hold P points): the blocks of a chain are P
// rows apart, and what block (plane p) fetched as its +P band is what the chain's next block
// (plane p + 1) needs as its centre band and the one after as its -P band.  The three bands
// therefore share three regions of stack_size slots that take turns: the columns around row r + d P,
// d = -1, 0, 1, live in region (r / P + d) mod 3, column c at c mod stack_size inside it.
struct BandTable {
    int32_t nbands;
    int32_t dlo[kWindowBands], dhi[kWindowBands], base[kWindowBands], width[kWindowBands];
    int32_t stack_rows, stack_size;
};
__host__ __device__ __forceinline__ int64_t band_centre(int64_t r, int64_t m, int64_t n) { return r * n / m; }

// The row that holds stored element i: the largest r with row_ptr[r] <= i.  The kBlock elements of
// a workgroup lie in rows seg_row[blockIdx.x] .. seg_row[blockIdx.x + 1]; their offsets are staged
// in LDS (when they are at most kBlock + 1: no long run of empty rows) and searched there.  Every
// thread of the workgroup calls this; *first_of_row receives row_ptr[r].
__device__ __forceinline__ int32_t row_of_element(const int32_t *__restrict__ row_ptr, int32_t m,
                                                  const int32_t *__restrict__ seg_row, int64_t i, int32_t *s_rp /* kBlock + 1 */,
                                                  int32_t *first_of_row)
{
    const int32_t r_lo = seg_row[blockIdx.x];
    int32_t r_hi = seg_row[blockIdx.x + 1];
    r_hi = r_hi > m - 1 ? m - 1 : r_hi;
    const int32_t cnt = r_hi - r_lo + 1;
    const bool staged = cnt <= kBlock + 1;  // uniform
    if (staged)
        for (int32_t j = threadIdx.x; j < cnt; j += kBlock) s_rp[j] = row_ptr[r_lo + j];
    __syncthreads();
    int32_t lo = 0, hi = cnt - 1;
    if (staged) {
        while (lo < hi) {
            const int32_t mid = lo + (hi - lo + 1) / 2;
            if (s_rp[mid] <= i)
                lo = mid;
            else
                hi = mid - 1;
        }
        *first_of_row = s_rp[lo];
    } else {
        while (lo < hi) {
            const int32_t mid = lo + (hi - lo + 1) / 2;
            if (row_ptr[r_lo + mid] <= i)
                lo = mid;
            else
                hi = mid - 1;
        }
        *first_of_row = row_ptr[r_lo + lo];
    }
    return r_lo + lo;
}

// bit b of `bits` set = some stored element has (c - centre(r) + n) / 64 == b.  One thread per
// stored element (the columns are read in order).  The workgroup collects its bits in LDS first (a
// few words: its elements lie on a few bands) and ors into memory only the words that still miss
// some of them: a hundred million atomics on the same fifty words would take milliseconds.
__global__ __launch_bounds__(kBlock) void k_window_offset_bins(const int32_t *__restrict__ row_ptr,
                                                               const int32_t *__restrict__ col, int32_t m, int32_t n,
                                                               int32_t nnz, const int32_t *__restrict__ seg_row,
                                                               uint32_t *bits)
{
    constexpr int kSlots = 64;  // words collected per workgroup, by word index modulo kSlots
    __shared__ uint32_t s_word[kSlots], s_mask[kSlots];
    __shared__ int32_t s_rp[kBlock + 1];
    if (threadIdx.x < kSlots) s_word[threadIdx.x] = 0xffffffffu, s_mask[threadIdx.x] = 0;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int32_t first;
    const int32_t r = row_of_element(row_ptr, m, seg_row, i < nnz ? i : nnz - 1, s_rp, &first);  // syncs
    if (i < nnz) {
        const int64_t bin = ((int64_t)col[i] + (int64_t)n - band_centre(r, m, n)) >> 6;
        const uint32_t word = (uint32_t)(bin >> 5), mask = 1u << (bin & 31);
        const uint32_t owner = atomicCAS(&s_word[word % kSlots], 0xffffffffu, word);
        if (owner == 0xffffffffu || owner == word)
            atomicOr(&s_mask[word % kSlots], mask);
        else if (!(__atomic_load_n(bits + word, __ATOMIC_RELAXED) & mask))  // the slot serves another word
            atomicOr(bits + word, mask);
    }
    __syncthreads();
    if (threadIdx.x < kSlots && s_mask[threadIdx.x]) {
        uint32_t *w = bits + s_word[threadIdx.x];
        if ((__atomic_load_n(w, __ATOMIC_RELAXED) & s_mask[threadIdx.x]) != s_mask[threadIdx.x]) atomicOr(w, s_mask[threadIdx.x]);
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_window_place(const int32_t *__restrict__ row_ptr,
                                                         const int32_t *__restrict__ col, const T *__restrict__ val,
                                                         int32_t m, int32_t n, int32_t nnz, int32_t rows, BandTable bands,
                                                         const int32_t *__restrict__ seg_row,
                                                         const int32_t *__restrict__ row_start,
                                                         const int32_t *__restrict__ tile_off, uint16_t *__restrict__ cf,
                                                         T *__restrict__ val_out, int32_t *__restrict__ perm, bool halves)
{
    __shared__ int32_t s_rp[kBlock + 1];
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int32_t first;
    const int32_t r = row_of_element(row_ptr, m, seg_row, i < nnz ? i : nnz - 1, s_rp, &first);  // syncs
    if (i >= nnz) return;
    const int32_t b = r / rows;
    const int32_t o = row_start[r] + (int32_t)(i - first);
    const int64_t d = (int64_t)tile_off[b] * kSlicedTile + o;
    const bool head = i == first || o % kSlicedTile == 0;
    const int32_t c = col[i];
    int k = 0;
    if (bands.nbands > 1) {
        const int64_t off = (int64_t)c - band_centre(r, m, n);
        for (int j = 1; j < kWindowBands; ++j)
            if (j < bands.nbands && off >= bands.dlo[j]) k = j;  // bands ascend and cover every offset
    }
    int32_t slot;
    if (bands.stack_rows > 0) {
        const int32_t q = r / bands.stack_rows + (k - 1);  // -1 .. number of planes
        slot = ((q % 3 + 3) % 3) * bands.stack_size + c % bands.stack_size;
    } else {
        slot = bands.base[k] + c % bands.width[k];
    }
    cf[halves ? d / kSlicedTile * kSlicedTile + tile_halves_pos((int)(d % kSlicedTile)) : d] = (uint16_t)(slot | (head ? 0x8000 : 0));
    if (val_out) {  // uniform
        const int64_t phys = d / kSlicedTile * kSlicedTile + tile_val_pos<T>((int)(d % kSlicedTile));
        val_out[phys] = val[i];
        perm[phys] = (int32_t)i;
    }
}

// per tile: x = the row its first slot belongs to, bit 31 set when the tile starts inside that
// row; y = the number of runs of the tile that are rows (the slots behind them are padding); where
// no row is padded (every row holds kMinRowSlots stored elements or more) the stored elements of a
// tile are consecutive in A: z = the index of the first, w = how many (the tile's other slots,
// behind them, are padding).
// The blocks are stored in the order the chains walk them: stored_off[i] = first tile of the i-th
// stored block, which holds the rows of block order[i] (of block i without an order).
__global__ __launch_bounds__(kBlock) void k_window_tile_info(const int32_t *__restrict__ row_start, int32_t m,
                                                             int32_t rows, int32_t nblocks,
                                                             const int32_t *__restrict__ stored_off,
                                                             const int32_t *__restrict__ order, int32_t ntiles,
                                                             const int32_t *__restrict__ row_ptr,
                                                             int4 *__restrict__ tile_info, int32_t *__restrict__ any_cont)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= ntiles) return;
    int32_t lo = 0, hi = nblocks - 1;  // stored block of tile t: largest i with stored_off[i] <= t
    while (lo < hi) {
        const int32_t mid = lo + (hi - lo + 1) / 2;
        if (stored_off[mid] <= t)
            lo = mid;
        else
            hi = mid - 1;
    }
    const int32_t b = order ? order[lo] : lo;
    const int64_t r0 = (int64_t)b * rows;
    const int32_t r1 = r0 + rows < m ? (int32_t)(r0 + rows) : m;
    const int32_t o = (int32_t)(t - stored_off[lo]) * kSlicedTile;
    int32_t a = (int32_t)r0, z = r1 - 1;  // largest row whose start is <= o
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
    const int32_t first = row_ptr[a] + (o - row_start[a]);
    const int32_t end = row_start[u - 1] + (row_ptr[u] - row_ptr[u - 1]) - o;  // end of the last row's stored elements
    tile_info[t] = make_int4(a | (cont ? (int32_t)0x80000000 : 0), u - a, first, end < kSlicedTile ? end : kSlicedTile);
    if (cont) *any_cont = 1;
}

// Copies the values again from where they came from.  `unless_equal` (may be null): four words, two
// checksums of the values now and two of the values the copy holds; where they agree nothing is done.
template <typename T>
__global__ __launch_bounds__(kBlock) void k_window_regather(const int32_t *__restrict__ perm, int64_t slots,
                                                            const T *__restrict__ val, T *__restrict__ val_out,
                                                            const unsigned long long *unless_equal)
{
    if (unless_equal && unless_equal[0] == unless_equal[2] && unless_equal[1] == unless_equal[3]) return;  // uniform
    for (int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; d < slots; d += (int64_t)gridDim.x * blockDim.x) {
        const int32_t src = perm[d];
        val_out[d] = src >= 0 ? val[src] : T(0);
    }
}

// ---- the kernel ----------------------------------------------------------------------------
// Run k of a tile is row (first row of the tile) + k, for the `limit` runs that are rows (at most
// kStageRows: a row takes at least two slots); the first sum of a tile that starts inside a row
// goes to the tile's carry slot.  The sums pass through a staging area of the wave in LDS and
// leave as stores of consecutive lanes to consecutive rows: stored straight from the lanes that
// close the runs (4 or 5 masked stores a tile, 8 bytes every 32 to 40), the same 134 MB of y cost
// 66 us of the 5-point stencil's 220; staged, a third of that.
//
// Memory operations of a wave complete in the order they were issued, and a wait for one of them
// names how many younger ones may still be in flight.  A tile's loads are issued D steps before
// the tile is multiplied; for them to stay in flight that long, every wait of the steady state
// must be for something at least as old, and the compiler must be able to count, on every path
// through the loop, what was issued in between.  Hence:
//  * with beta != 0 (BETA) what y holds in a tile's rows is loaded together with the tile, D steps
//    ahead, not when the rows are written: a wait for a load issued then would also wait for every
//    tile on its way;
//  * nothing inside a step branches on the lane: sums nobody wants go to a spare place in LDS,
//    rows a lane does not own are cut off by the range check of a buffer store.  Branches that
//    depend on the lane make the compiler rebuild the loops around them with flags, and across
//    those it assumes the worst: that a tile is multiplied right after it was requested;
//  * the loop over a wave's tiles of one block is a loop of its own, unrolled D times, once for
//    every buffer the block can start with; the start of a block, which waits for the columns of
//    x it stores, separates them.
constexpr int kStageRows = 128;
constexpr int kStageSlots = kStageRows + kWave;  // + one place per lane for the sums nobody wants
constexpr uint32_t kOutOfRange = 0xfffffff0u;     // a byte offset past any range of rows

// y in rows row0 .. row0 + rows - 1 as a buffer: loads past the range return 0, stores are dropped
template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t rows_of_y(T *y, int32_t row0, int32_t rows)
{
    return __builtin_amdgcn_make_buffer_rsrc(y + row0, 0, rows * (int32_t)sizeof(T), 0x00020000);
}
template <typename T>
struct RowIO;
template <>
struct RowIO<double> {
    typedef int bits_t __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ double load(__amdgpu_buffer_rsrc_t r, uint32_t off)
    {
        return __builtin_bit_cast(double, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0));
    }
    static __device__ __forceinline__ void store(double v, __amdgpu_buffer_rsrc_t r, uint32_t off)
    {
        __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(bits_t, v), r, off, 0, 0);
    }
};
template <>
struct RowIO<float> {
    static __device__ __forceinline__ float load(__amdgpu_buffer_rsrc_t r, uint32_t off)
    {
        return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
    }
    static __device__ __forceinline__ void store(float v, __amdgpu_buffer_rsrc_t r, uint32_t off)
    {
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), r, off, 0, 0);
    }
};

template <typename T, bool BETA>
struct WindowTile : Tile<T> {
    int32_t limit;             // base, limit: the tile's two words, uniform
    T yv[kStageRows / kWave];  // BETA: y in rows (first row) + lane + 64 k
};
// A tile's four values per lane, read in place from A's val: the tile's stored elements are
// `count` consecutive ones from `first` on (no row of the plan is padded), and what lies past them
// is padding, which the buffer's range check reads as 0.  fp32: lane l holds the 4l-th to the
// (4l+3)-th; fp64: the 2l-th, the next, the (128+2l)-th and the next (tile_reduce_halves).
template <typename T>
struct ValuesInPlace;
template <>
struct ValuesInPlace<double> {
    static __device__ __forceinline__ void load(const double *val, int32_t first, int32_t count, int lane, double v[4])
    {
        typedef double f64x2 __attribute__((ext_vector_type(2)));
        const __amdgpu_buffer_rsrc_t r =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<double *>(val) + first, 0, count * (int32_t)sizeof(double), 0x00020000);
        // slots 2 lane, 2 lane + 1 and 128 + 2 lane, 128 + 2 lane + 1: each load reads 1 KiB of consecutive values
        const f64x2 a = __builtin_bit_cast(f64x2, __builtin_amdgcn_raw_buffer_load_b128(r, (uint32_t)lane * 16u, 0, 2));
        const f64x2 b = __builtin_bit_cast(f64x2, __builtin_amdgcn_raw_buffer_load_b128(r, 1024u + (uint32_t)lane * 16u, 0, 2));
        v[0] = a.x, v[1] = a.y, v[2] = b.x, v[3] = b.y;
    }
};
template <>
struct ValuesInPlace<float> {
    static __device__ __forceinline__ void load(const float *val, int32_t first, int32_t count, int lane, float v[4])
    {
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        const __amdgpu_buffer_rsrc_t r =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(val) + first, 0, count * (int32_t)sizeof(float), 0x00020000);
        const f32x4 a = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (uint32_t)lane * 16u, 0, 2));
        v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w;
    }
};

// the loads of tile t, whose words are `info`; INPLACE: the values from A's val, else from the plan's copy
template <typename T, bool BETA, bool INPLACE>
__device__ __forceinline__ void window_tile_load(WindowTile<T, BETA> &tl, int32_t t, int4 info, int lane,
                                                 const uint16_t *__restrict__ cf, const T *__restrict__ val, T *y)
{
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 cw = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(cf + (int64_t)t * kSlicedTile) + lane);
    tl.c01 = cw.x;
    tl.c23 = cw.y;
    if (INPLACE)  // the buffer's words as scalars by name: left to itself the compiler keeps the count in a vector
                  // register and wraps every load into a loop over the distinct values of the lanes
        ValuesInPlace<T>::load(val, __builtin_amdgcn_readfirstlane(info.z), __builtin_amdgcn_readfirstlane(info.w), lane, tl.v);
    else
        TileValues<T>::load(val + (int64_t)t * kSlicedTile, lane, tl.v);
    tl.base = info.x;
    tl.limit = info.y;
    if (BETA) {
        const __amdgpu_buffer_rsrc_t rows = rows_of_y<T>(y, info.x & 0x7fffffff, info.y);
#pragma unroll
        for (int k = 0; k < kStageRows / kWave; ++k) tl.yv[k] = RowIO<T>::load(rows, (uint32_t)((k * kWave + lane) * sizeof(T)));
    }
}

template <typename T>
struct StageRows {
    T *stage;
    int lane;
    __device__ __forceinline__ void operator()(bool wanted, int rank, T v) const
    {
        stage[wanted && rank < kStageRows ? rank : kStageRows + lane] = v;  // runs past the rows are padding
    }
};

// Everything a step needs beside its tile.
template <typename T>
struct WindowStep {
    const uint16_t *__restrict__ cf;
    const T *__restrict__ val;
    const int4 *__restrict__ tile_info;
    T *y, *carry;
    const T *xs;
    T *stage;
    T alpha, beta;
    int32_t chain_last;
    int lane;
    int4 info_next;  // the words of the tile the next step will request
};
// One tile: its rows' sums into the staging area and from there to y, then the loads of the tile
// `ahead` tiles further on (past the end of the chain: the last tile again) into the registers this
// one has just left, and the words of the tile after that.
template <typename T, bool BETA, bool INPLACE>
__device__ __forceinline__ void window_step(WindowTile<T, BETA> &tl, int32_t t, int32_t ahead, int32_t stride, WindowStep<T> &w)
{
    if (INPLACE && sizeof(T) == 8)
        tile_reduce_halves<T>(tl, w.lane, w.xs, StageRows<T>{w.stage, w.lane});
    else
        tile_reduce<T>(tl, w.lane, w.xs, StageRows<T>{w.stage, w.lane});
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // the wave's LDS writes and reads execute in order
    __builtin_amdgcn_wave_barrier();
    const int32_t row0 = tl.base & 0x7fffffff, limit = tl.limit;
    const bool cont = tl.base < 0;
    const __amdgpu_buffer_rsrc_t rows = rows_of_y<T>(w.y, row0, limit);
#pragma unroll
    for (int k = 0; k < kStageRows / kWave; ++k) {
        if (k * kWave < limit) {  // uniform
            const int32_t i = k * kWave + w.lane;
            const T v = w.stage[i];
            const T out = BETA ? fma_t<T>(w.alpha, v, w.beta * tl.yv[k]) : w.alpha * v;
            // the first sum of a tile that starts inside a row is no row's
            RowIO<T>::store(out, rows, k == 0 && cont && i == 0 ? kOutOfRange : (uint32_t)(i * sizeof(T)));
        }
    }
    if (cont) w.carry[t] = w.stage[0];  // uniform; every lane stores the same value
    __builtin_amdgcn_wave_barrier();
    const int32_t t1 = t + ahead < w.chain_last ? t + ahead : w.chain_last;
    window_tile_load<T, BETA, INPLACE>(tl, t1, w.info_next, w.lane, w.cf, w.val, w.y);
    const int32_t t2 = t + ahead + stride < w.chain_last ? t + ahead + stride : w.chain_last;
    w.info_next = w.tile_info[t2];
}
// `cnt` tiles of one wave in turn, the first in buffer P; a loop of its own for every P, with one
// way out (a loop left from the middle is rebuilt with flags too), so that on every path through
// it a buffer is used D - 1 steps after it was requested
template <typename T, bool BETA, bool INPLACE, int D, int NW, int P>
__device__ __forceinline__ void window_steps(WindowTile<T, BETA> (&tl)[D], int32_t &t, int32_t cnt, WindowStep<T> &w)
{
    for (int32_t i = cnt / D; i > 0; --i) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            window_step<T, BETA, INPLACE>(tl[(P + j) % D], t, D * NW, NW, w);
            t += NW;
        }
    }
    const int32_t rest = cnt % D;
#pragma unroll
    for (int j = 0; j + 1 < D; ++j) {
        if (j < rest) {
            window_step<T, BETA, INPLACE>(tl[(P + j) % D], t, D * NW, NW, w);
            t += NW;
        }
    }
}

// The pieces of x a block needs before it is multiplied (at most kWindowBands ranges of columns
// [from, to), from and to multiples of 4; ring of piece q: slots base .. base + width) into
// registers, one 16-byte unit per thread and step, and later from the registers into the rings.
// x is read as a buffer whose range ends with x: what lies past the last column reads as 0, word
// by word, so a unit may straddle the end, and x needs no more than the alignment of its elements.
// With several pieces (NB > 1) every piece starts at a multiple of 64 units: the 64 lanes of a wave
// then work on one piece, and which one is found with scalar compares; the builder keeps the
// pieces of a block, each rounded up to 64 units, within what the registers hold: kFetchCols
// columns a round.  The first block of a chain, which fetches whole windows, takes as many rounds as
// it needs; every other block's pieces fit one (the builder starts a new chain otherwise), so the
// registers that carry x through a block are half of what a whole window would take.
// NB = 1: one piece, ring of kWindowCols slots from slot 0 (constant modulus).
template <typename T, int THREADS, int NB>
struct XFetch {
    static constexpr int V = 16 / sizeof(T);
    static constexpr int PER = kFetchCols / (THREADS * V);
    static constexpr int kRound = PER * THREADS;  // units a round moves
    typedef T vec_t __attribute__((ext_vector_type(V)));
    typedef uint32_t bits_t __attribute__((ext_vector_type(4)));
    vec_t buf[PER];
    // the pending fetch (uniform values): its pieces, the first unit of each, the ring slot of its
    // first column and how many of its columns lie inside x
    int32_t from[NB], len[NB], inside[NB], base[NB], width[NB], ustart[NB], fslot[NB];
    int32_t units;  // of the pending fetch, the padding between its pieces included

    __device__ __forceinline__ void set(const int4 *__restrict__ pieces, int32_t lo, int32_t hi, int32_t n)
    {
        int32_t u = 0;
#pragma unroll
        for (int q = 0; q < NB; ++q) {
            int4 pc = make_int4(0, 0, 0, 4);
            if (lo + q < hi) pc = pieces[lo + q];  // uniform
            from[q] = __builtin_amdgcn_readfirstlane(pc.x);
            len[q] = __builtin_amdgcn_readfirstlane(pc.y) - from[q];
            const int32_t left = n - from[q];
            inside[q] = left < 0 ? 0 : left < len[q] ? left : len[q];
            base[q] = NB == 1 ? 0 : __builtin_amdgcn_readfirstlane(pc.z);
            width[q] = NB == 1 ? kWindowCols : __builtin_amdgcn_readfirstlane(pc.w);
            fslot[q] = (int32_t)((uint32_t)from[q] % (uint32_t)width[q]);
            ustart[q] = u;
            u += (len[q] + V - 1) / V;
            if (NB > 1) u = (u + kWave - 1) & ~(kWave - 1);
        }
        units = u;
    }
    // the piece the 64 units from `first_unit` on belong to (all values uniform)
    struct Piece {
        int32_t from, len, inside, base, width, ustart, fslot;
    };
    __device__ __forceinline__ Piece piece_of(int32_t first_unit) const
    {
        Piece p{from[0], len[0], inside[0], base[0], width[0], ustart[0], fslot[0]};
#pragma unroll
        for (int j = 1; j < NB; ++j) {
            const bool in = first_unit >= ustart[j];
            p.from = in ? from[j] : p.from;
            p.len = in ? len[j] : p.len;
            p.inside = in ? inside[j] : p.inside;
            p.base = in ? base[j] : p.base;
            p.width = in ? width[j] : p.width;
            p.ustart = in ? ustart[j] : p.ustart;
            p.fslot = in ? fslot[j] : p.fslot;
        }
        return p;
    }
    // round `u0 / kRound` of the pending fetch: units u0 .. u0 + kRound - 1
    __device__ __forceinline__ void load(const T *__restrict__ x, int wave, int32_t u0 = 0)
    {
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const Piece p = piece_of(u0 + k * THREADS + wave * kWave);
            const int32_t u = u0 + k * THREADS + (int)threadIdx.x - p.ustart;  // unit inside the piece
            const __amdgpu_buffer_rsrc_t cols =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(x) + p.from, 0, p.inside * (int32_t)sizeof(T), 0x00020000);
            buf[k] = __builtin_bit_cast(vec_t, __builtin_amdgcn_raw_buffer_load_b128(cols, (uint32_t)u * 16u, 0, 0));
        }
    }
    __device__ __forceinline__ void store(T *xs, int wave, int32_t u0 = 0) const
    {
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const Piece p = piece_of(u0 + k * THREADS + wave * kWave);
            const int32_t e = (u0 + k * THREADS + (int)threadIdx.x - p.ustart) * V;  // column inside the piece
            if (e < p.len) {
                const int32_t sl = p.fslot + e;  // a piece is no longer than its ring: one wrap at most
                *reinterpret_cast<vec_t *>(xs + p.base + (sl >= p.width ? sl - p.width : sl)) = buf[k];
            }
        }
    }
};

template <typename T, int NW, int NB, int D, bool BETA, bool INPLACE>
__global__ __launch_bounds__(NW *kWave) void k_spmv_window(int32_t n, T alpha, T beta, const int2 *__restrict__ chains,
                                                           const int4 *__restrict__ blocks,
                                                           const int4 *__restrict__ pieces,
                                                           const uint16_t *__restrict__ cf, const T *__restrict__ val,
                                                           const int4 *__restrict__ tile_info,
                                                           const T *__restrict__ x, T *y, T *__restrict__ carry)
{
    static_assert(D >= 1 && D <= 3, "one loop per starting buffer is written out for up to three buffers");
    // the rings over the columns of x, then the zero the pads point at
    __shared__ __align__(16) T xs[kWindowCols + 16 / sizeof(T)];
    __shared__ T stage_all[NW * kStageSlots];
    const int2 chain = chains[blockIdx.x];  // first block, end block
    // the wave's number as a scalar: the tile counters and every loop condition below are uniform
    const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    WindowStep<T> w{cf, val, tile_info, y, carry, xs, stage_all + wave * kStageSlots, alpha, beta,
                    blocks[chain.y - 1].y - 1, lane, make_int4(0, 0, 0, 0)};
    // this wave's tiles are those congruent to its number, across the blocks of the chain; D are
    // in flight (requested D steps ahead; past the end of the chain the last tile is re-read)
    WindowTile<T, BETA> tl[D];
    int32_t t = blocks[chain.x].x + wave;
#pragma unroll
    for (int d = 0; d < D; ++d) {
        const int32_t td = t + d * NW < w.chain_last ? t + d * NW : w.chain_last;
        window_tile_load<T, BETA, INPLACE>(tl[d], td, tile_info[td], lane, cf, val, y);
    }
    w.info_next = tile_info[t + D * NW < w.chain_last ? t + D * NW : w.chain_last];
    if (threadIdx.x == 0) xs[kWindowCols] = T(0);
    XFetch<T, NW * kWave, NB> xf;
    int4 blk = blocks[chain.x];  // first tile, end tile, pieces of x to fetch before the block: first, end
    // the first block's columns (whole windows), a round of registers at a time
    xf.set(pieces, blk.z, blk.w, n);
    for (int32_t u0 = 0; u0 < xf.units; u0 += xf.kRound) {
        xf.load(x, wave, u0);
        xf.store(xs, wave, u0);
    }
    int32_t first = 0;  // the buffer that holds the wave's next tile
    // Every wave passes the start and the end of every block of the chain (the barriers count all
    // waves), whether it has tiles in the block or not.  All conditions are uniform over the wave.
    for (int32_t b = chain.x; b < chain.y; ++b) {
        __syncthreads();  // the block's columns are in the rings
        const int32_t tile_hi = blk.y;
        const bool more = b + 1 < chain.y;
        if (more) {  // the next block's new columns are fetched while this one is multiplied
            blk = blocks[b + 1];
            xf.set(pieces, blk.z, blk.w, n);
            xf.load(x, wave);
        }
        const int32_t cnt = t < tile_hi ? (tile_hi - t + NW - 1) / NW : 0;  // this wave's tiles in the block
        // the D tile buffers take turns without changing places
        if (D == 1 || first == 0)
            window_steps<T, BETA, INPLACE, D, NW, 0>(tl, t, cnt, w);
        else if (D == 2 || first == 1)
            window_steps<T, BETA, INPLACE, D, NW, 1 % D>(tl, t, cnt, w);
        else
            window_steps<T, BETA, INPLACE, D, NW, 2 % D>(tl, t, cnt, w);
        first = (first + cnt) % D;
        __syncthreads();  // every wave is done with the block: its columns may go
        if (more) xf.store(xs, wave);
    }
}

// Adds the carries to their rows: the thread of the first tile of a run of tiles that start inside
// the same row sums the run's carries and adds the total once.  Up to kSerialCarries of them it
// sums itself, in tile order; what a longer run holds beyond those (a row of several thousand
// stored elements) the 64 lanes of its wave sum together, 64 tiles a round, combined in a fixed
// order: the same bits in every call.
constexpr int32_t kSerialCarries = 8;
template <typename T>
__global__ __launch_bounds__(kBlock) void k_window_fixup(int32_t ntiles, T alpha, const int4 *__restrict__ tile_info,
                                                         const T *__restrict__ carry, T *__restrict__ y)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int32_t w = t < ntiles ? tile_info[t].x : 0;
    // a tile that starts inside a row and is the first of its run
    const bool head = w < 0 && !(t > 0 && tile_info[t - 1].x == w);
    T s = T(0);
    int32_t taken = 0;
    if (head) {
        for (int64_t j = t; taken < kSerialCarries && j < ntiles && tile_info[j].x == w; ++j, ++taken) s += carry[j];
    }
    const bool more = head && taken == kSerialCarries && t + taken < ntiles && tile_info[t + taken].x == w;
    unsigned long long todo = __ballot(more);
    while (todo) {  // uniform over the wave
        const int f = __builtin_ctzll(todo);
        todo &= todo - 1;
        const int32_t wf = __builtin_amdgcn_readlane(w, f);
        const int64_t tf = ((int64_t)blockIdx.x * blockDim.x + (threadIdx.x & ~(kWave - 1)) + f) + kSerialCarries;
        T part = T(0);
        for (int64_t j0 = tf;; j0 += kWave) {
            const int64_t j = j0 + lane;
            const bool in = j < ntiles && tile_info[j].x == wf;
            if (in) part += carry[j];
            if (__ballot(in) != ~0ull) break;  // the run ended inside these 64 tiles
        }
#pragma unroll
        for (int d = kWave / 2; d > 0; d >>= 1) part += __shfl_xor(part, d, kWave);
        if (lane == f) s += part;
    }
    if (head) {
        const int32_t r = w & 0x7fffffff;
        y[r] = fma_t<T>(alpha, s, y[r]);
    }
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
int build_window(int32_t m, int32_t n, int32_t nnz, int32_t target_wgs, bool in_place, const int32_t *row_ptr,
                 const int32_t *col, const T *val, WindowMatrix *out, hipStream_t s)
{
    WindowMatrix wm{};
    if (m <= 0 || nnz <= 0 || n <= 0) return ASX_STATUS_INVALID_SIZE;
    if (target_wgs < 1) return ASX_STATUS_INVALID_VALUE;
    int st = ASX_STATUS_SUCCESS;
    int32_t *arena = nullptr;
    int32_t *gmin = nullptr, *gmax = nullptr, *row_start = nullptr, *seg_row = nullptr;
    int32_t *bmin = nullptr, *bmax = nullptr, *btiles = nullptr, *tile_off = nullptr, *d_small = nullptr;
    std::vector<int32_t> h_bmin, h_bmax, h_bt, h_off, h_soff, h_order, blk, pcs, chains;
    int64_t stack_ulo = 0, stack_uhi = 0;
    bool stacked = false, halves = false;
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
    // few counters
    {
        const auto pad64 = [](size_t v) { return (v + 63) & ~(size_t)63; };
        const size_t per_group = pad64((size_t)ngroups), per_row = pad64((size_t)m), per_seg = pad64((size_t)nseg + 1);
        const size_t per_block = pad64((size_t)max_nb + 1);
        ASX_TRY(hipMalloc((void **)&arena, sizeof(int32_t) * (2 * per_group + per_row + per_seg + 4 * per_block + 64)));
        gmin = arena, gmax = gmin + per_group, row_start = gmax + per_group, seg_row = row_start + per_row;
        bmin = seg_row + per_seg, bmax = bmin + per_block, btiles = bmax + per_block, tile_off = btiles + per_block;
        d_small = tile_off + per_block;
    }

    // 1. column span of every group of rows
    hipLaunchKernelGGL(k_window_fill_i32, dim3(1), dim3(kBlock), 0, s, d_small, (int64_t)16, 0);
    hipLaunchKernelGGL(k_window_group_span, dim3((unsigned)ceil_div64((int64_t)ngroups * kWave, kBlock)), dim3(kBlock), 0, s,
                       row_ptr, col, m, ngroups, gmin, gmax, d_small + 13);
    // 2. the largest block of rows whose widest window fits the ring: the widest window of every
    //    candidate size, all read back at once
    for (int k = 0; k < kCandidates; ++k) {
        const int32_t rows = kBlockRows[k];
        if (rows > 256 && ceil_div64(m, rows) < min_blocks) continue;  // too few blocks to share out
        const int32_t nb = (int32_t)ceil_div64(m, rows);
        hipLaunchKernelGGL(k_window_block_span, dim3((unsigned)ceil_div64(nb, kBlock)), dim3(kBlock), 0, s, gmin, gmax, ngroups,
                           rows / kSpanGroup, nb, (int32_t *)nullptr, (int32_t *)nullptr, d_small + k);
    }
    st = launch_nnz_split_rows(row_ptr, m, nnz, kBlock, seg_row, s);  // for step 4; runs while the host waits
    if (st) goto done;
    ASX_TRY(hipMemcpyAsync(h_small, d_small, sizeof(int32_t) * 14, hipMemcpyDeviceToHost, s));
    ASX_TRY(hipStreamSynchronize(s));
    // no row shorter than kMinRowSlots: no slot between the stored elements of a tile is padding, and
    // the kernel can read A's values in place; fp64 ones two 16-byte loads a lane, a pair of slots
    // from either half of the tile (tile_reduce_halves; the lane's four column words lie together)
    wm.by_reference = in_place && h_small[13] == 0;
    halves = wm.by_reference && sizeof(T) == 8;
    wm.rows_per_block = 0;
    {
        // Of the sizes whose windows fit, the one with the shortest longest chain: a workgroup walks
        // ceil(blocks / workgroups) blocks, each of which costs its rows (at a workgroup's share of
        // 5.6 TB/s) and about 1.1 us to start.  4.5 M rows of a 5-point stencil on 256 workgroups:
        // 1099 blocks of 4096 rows make chains of 5 (20480 rows), 1465 blocks of 3072 chains of 6
        // (18432 rows).  A block past the first of a chain may fetch kFetchCols columns at most, so
        // sizes that advance further than that along the columns are left out.
        const double row_bytes = (double)nnz / (double)m * (double)(sizeof(T) + 2) + 3.0 * (double)sizeof(T);
        const double row_time = row_bytes / (5.6e12 / (double)target_wgs), start_time = 1.1e-6;
        double best = 0.0;
        int best_k = -1;
        for (int k = 0; k < kCandidates; ++k) {
            const int32_t rows = kBlockRows[k];
            if (rows > 256 && ceil_div64(m, rows) < min_blocks) continue;
            if (h_small[k] > kWindowCols - kWindowSlack) continue;
            if (rows > 256 && (double)rows * (double)n / (double)m > (double)kFetchCols) continue;
            const double chain = (double)ceil_div64(ceil_div64(m, rows), target_wgs) * ((double)rows * row_time + start_time);
            if (best_k < 0 || chain < best * 0.98) best = chain, best_k = k;  // a larger size unless a smaller one is clearly ahead
        }
        if (best_k >= 0) {
            const int32_t rows = kBlockRows[best_k];
            wm.rows_per_block = rows;
            wm.nblocks = (int32_t)ceil_div64(m, rows);
            hipLaunchKernelGGL(k_window_block_span, dim3((unsigned)ceil_div64(wm.nblocks, kBlock)), dim3(kBlock), 0, s, gmin,
                               gmax, ngroups, rows / kSpanGroup, wm.nblocks, bmin, bmax, d_small + 15);
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
        // a ring holds a multiple of 64 16-byte units: a block's pieces, each rounded up to 64 units
        // (one wave's worth) as the kernel fetches them, then fit the registers the fetch passes through
        const auto ring_size = [](int64_t columns) {
            constexpr int64_t unit = kWave * (16 / (int64_t)sizeof(T));
            return (columns + unit - 1) / unit * unit;
        };
        const int64_t nbins = (2 * (int64_t)n >> 6) + 2;
        const size_t words = (size_t)(nbins + 31) / 32;
        ASX_TRY(hipMalloc((void **)&d_bits, sizeof(uint32_t) * words));
        ASX_TRY(hipMemsetAsync(d_bits, 0, sizeof(uint32_t) * words, s));
        hipLaunchKernelGGL(k_window_offset_bins, dim3((unsigned)nseg), dim3(kBlock), 0, s, row_ptr, col, m, n, nnz, seg_row, d_bits);
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
        const auto join_runs = [&runs](size_t keep) {  // join the two runs with the smallest gap until `keep` are left
            while (runs.size() > keep) {
                size_t best = 0;
                for (size_t i = 1; i + 1 < runs.size(); ++i)
                    if (runs[i + 1].first - runs[i].second < runs[best + 1].first - runs[best].second) best = i;
                runs[best].second = runs[best + 1].second;
                runs.erase(runs.begin() + (long)best + 1);
            }
        };
        const auto set_bands = [&runs, &bands, n]() {
            bands.nbands = (int32_t)runs.size();
            for (int k = 0; k < bands.nbands; ++k) {
                bands.dlo[k] = (int32_t)std::max<int64_t>((runs[(size_t)k].first << 6) - n, -(int64_t)n);
                bands.dhi[k] = (int32_t)std::min<int64_t>(((runs[(size_t)k].second + 1) << 6) - 1 - n, n);
            }
        };
        // Stacked planes first (see BandTable): a square matrix whose runs, joined into three bands,
        // lie a whole number of planes apart.  P = the divisor of m nearest to half the distance
        // between the outer bands (any P is correct; one off the true distance only widens what the
        // regions must hold); U = the offsets all three bands span once band k is shifted back by
        // (k - 1) P; R = P / d rows per block: the largest that leaves enough blocks, else the
        // smallest whose three regions fit.
        if (runs.size() >= 3 && m == n) {
            const std::vector<std::pair<int64_t, int64_t>> all_runs = runs;
            join_runs(3);
            set_bands();
            const int64_t p0 = (((int64_t)bands.dlo[2] + bands.dhi[2]) - ((int64_t)bands.dlo[0] + bands.dhi[0])) / 4;
            int64_t P = 0;
            for (int64_t e = 0; e <= 64 && !P; ++e)
                for (int64_t cand : {p0 - e, p0 + e})
                    if (cand >= 256 && cand < m && m % cand == 0) {
                        P = cand;
                        break;
                    }
            if (P) {
                int64_t ulo = INT64_MAX, uhi = INT64_MIN;
                for (int k = 0; k < 3; ++k) {
                    ulo = std::min<int64_t>(ulo, bands.dlo[k] - (k - 1) * P);
                    uhi = std::max<int64_t>(uhi, bands.dhi[k] - (k - 1) * P);
                }
                int64_t pick = 0, size = 0;
                for (int64_t d = 1; P / d >= 256; ++d) {
                    if (P % d) continue;
                    const int64_t rows = P / d;
                    const int64_t sz = ring_size(rows + (uhi - ulo) + kWindowSlack + 3 + 3);
                    if (rows > 8192 || 3 * sz > kWindowCols) continue;
                    pick = rows, size = sz;
                    if (m / rows >= min_blocks) break;
                }
                if (pick) {
                    wm.rows_per_block = (int32_t)pick;
                    wm.nblocks = (int32_t)(m / pick);
                    bands.stack_rows = (int32_t)P;
                    bands.stack_size = (int32_t)size;
                    stack_ulo = ulo, stack_uhi = uhi;
                    for (int k = 0; k < 3; ++k) bands.base[k] = 0, bands.width[k] = (int32_t)size;  // not used to place
                }
            }
            if (!wm.rows_per_block) runs = all_runs;
        }
        if (!wm.rows_per_block) {
            // a ring per band; more runs than rings: the closest runs are joined
            join_runs(kWindowBands);
            // one run of offsets: the rows fill a band too wide for the single window tried above
            // (the one-ring kernel places column c at c mod kWindowCols; it is not built from here)
            if (runs.size() < 2) {
                st = ASX_STATUS_NOT_SUPPORTED;
                goto done;
            }
            set_bands();
        }
        for (int32_t rows : {8192, 7168, 6144, 5120, 4608, 4096, 3584, 3072, 2560, 2048, 1792, 1536, 1280, 1024, 768, 512, 384, 256}) {
            if (wm.rows_per_block) break;  // stacked planes
            if (rows > 256 && ceil_div64(m, rows) < min_blocks) continue;
            const int64_t advance = ceil_div64((int64_t)rows * n, m) + 1;  // of the centre over a block
            int64_t total = 0;
            for (int k = 0; k < bands.nbands; ++k)
                total += ring_size(advance + ((int64_t)bands.dhi[k] - bands.dlo[k]) + 1 + kWindowSlack + 3 + 3);
            if (total > kWindowCols) continue;
            wm.rows_per_block = rows;
            wm.nblocks = (int32_t)ceil_div64(m, rows);
            int32_t at = 0;
            for (int k = 0; k < bands.nbands; ++k) {
                bands.base[k] = at;
                bands.width[k] = (int32_t)ring_size(advance + ((int64_t)bands.dhi[k] - bands.dlo[k]) + 1 + kWindowSlack + 3 + 3);
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
    stacked = bands.stack_rows > 0;
    wm.stack_rows = bands.stack_rows;
    // 3. where every row starts inside its block; tiles of every block; the order the blocks are
    //    stored in (the order the chains walk them) and the first tile of each
    hipLaunchKernelGGL(k_window_row_starts, dim3((unsigned)ceil_div64((int64_t)wm.nblocks * kWave, kBlock)), dim3(kBlock), 0, s, row_ptr, m,
                       wm.rows_per_block, wm.nblocks, row_start, btiles);
    h_bmin.resize((size_t)wm.nblocks);
    h_bmax.resize((size_t)wm.nblocks);
    h_bt.resize((size_t)wm.nblocks);
    h_off.resize((size_t)wm.nblocks + 1);
    if (bands.nbands == 1) {
        ASX_TRY(hipMemcpyAsync(h_bmin.data(), bmin, sizeof(int32_t) * h_bmin.size(), hipMemcpyDeviceToHost, s));
        ASX_TRY(hipMemcpyAsync(h_bmax.data(), bmax, sizeof(int32_t) * h_bmax.size(), hipMemcpyDeviceToHost, s));
    }
    ASX_TRY(hipMemcpyAsync(h_bt.data(), btiles, sizeof(int32_t) * h_bt.size(), hipMemcpyDeviceToHost, s));
    ASX_TRY(hipStreamSynchronize(s));
    if (stacked) {
        // column j of blocks (the j-th R rows of every plane), plane after plane, then column j + 1
        const int32_t per_plane = bands.stack_rows / wm.rows_per_block, nplanes = m / bands.stack_rows;
        h_order.resize((size_t)wm.nblocks);
        h_soff.resize((size_t)wm.nblocks + 1);
        int64_t at = 0;
        for (int32_t i = 0; i < wm.nblocks; ++i) {
            const int32_t b = (i % nplanes) * per_plane + i / nplanes;
            h_order[(size_t)i] = b;
            h_soff[(size_t)i] = (int32_t)at;
            h_off[(size_t)b] = (int32_t)at;
            at += h_bt[(size_t)b];
        }
        slots = at * kSlicedTile;
        h_soff[(size_t)wm.nblocks] = h_off[(size_t)wm.nblocks] = (int32_t)std::min<int64_t>(at, 0x7fffffff);
    } else {
        int64_t at = 0;
        for (int32_t b = 0; b < wm.nblocks; ++b) {
            h_off[(size_t)b] = (int32_t)at;
            at += h_bt[(size_t)b];
        }
        slots = at * kSlicedTile;
        h_off[(size_t)wm.nblocks] = (int32_t)std::min<int64_t>(at, 0x7fffffff);
    }
    if (slots > 0x7fffffff) {
        st = ASX_STATUS_INVALID_SIZE;
        goto done;
    }
    wm.ntiles = (int32_t)(slots / kSlicedTile);
    ASX_TRY(hipMemcpyAsync(tile_off, h_off.data(), sizeof(int32_t) * h_off.size(), hipMemcpyHostToDevice, s));
    if (stacked) {  // bmin and bmax are free: they serve single windows only
        ASX_TRY(hipMemcpyAsync(bmin, h_soff.data(), sizeof(int32_t) * h_soff.size(), hipMemcpyHostToDevice, s));
        ASX_TRY(hipMemcpyAsync(bmax, h_order.data(), sizeof(int32_t) * h_order.size(), hipMemcpyHostToDevice, s));
    }
    {   // the regrouped copy in one allocation (values and their source indices only when they are copied)
        const size_t o_val = 0, o_perm = wm.by_reference ? 0 : align_up(sizeof(T) * (size_t)slots, 256);
        const size_t o_cf = o_perm + (wm.by_reference ? 0 : align_up(sizeof(int32_t) * (size_t)slots, 256));
        const size_t o_info = o_cf + align_up(sizeof(uint16_t) * (size_t)slots, 256);
        ASX_TRY(hipMalloc(&wm.store, o_info + sizeof(int4) * (size_t)wm.ntiles));
        char *base = static_cast<char *>(wm.store);
        wm.val = wm.by_reference ? nullptr : base + o_val;
        wm.perm = wm.by_reference ? nullptr : (int32_t *)(base + o_perm);
        wm.cf = (uint16_t *)(base + o_cf);
        wm.tile_info = (int32_t *)(base + o_info);
    }
    ASX_TRY(hipMalloc(&wm.carry, sizeof(T) * (size_t)wm.ntiles));
    // 4. every stored element to its slot; every other slot becomes a zero that points at the zero
    //    behind the rings and opens a run of its own
    hipLaunchKernelGGL((k_window_place<T>), dim3((unsigned)ceil_div64(nnz, kBlock)), dim3(kBlock), 0, s, row_ptr, col, val,
                       m, n, nnz, wm.rows_per_block, bands, seg_row, row_start, tile_off, wm.cf, (T *)wm.val, wm.perm, halves);
    hipLaunchKernelGGL((k_window_pads<T>), dim3(mgrid), dim3(kBlock), 0, s, row_ptr, m, wm.rows_per_block, row_start, tile_off,
                       btiles, (uint16_t)(0x8000 | kWindowCols), wm.cf, (T *)wm.val, wm.perm, halves);
    // 5. first row and number of rows of every tile
    hipLaunchKernelGGL(k_window_fill_i32, dim3(1), dim3(kBlock), 0, s, d_small, (int64_t)2, 0);
    hipLaunchKernelGGL(k_window_tile_info, dim3((unsigned)ceil_div64(wm.ntiles, kBlock)), dim3(kBlock), 0, s, row_start, m,
                       wm.rows_per_block, wm.nblocks, stacked ? bmin : tile_off, stacked ? bmax : (int32_t *)nullptr,
                       wm.ntiles, row_ptr, (int4 *)wm.tile_info, d_small);
    ASX_TRY(hipMemcpyAsync(h_small, d_small, sizeof(int32_t), hipMemcpyDeviceToHost, s));
    // 6. chains of blocks, one per workgroup, of about equal numbers of tiles.  Inside a chain a
    //    block fetches, per band, only the columns behind those already in the band's ring; a block
    //    whose columns start before what a ring still holds begins a new chain (and fetches its
    //    whole windows).
    {
    const int64_t per_chain = std::max<int64_t>(1, ceil_div64(wm.ntiles, target_wgs));
    const auto fetch_unit = [](int64_t columns) {  // several pieces: each takes whole waves of 64 16-byte units
        constexpr int64_t unit = kWave * (16 / (int64_t)sizeof(T));
        return (columns + unit - 1) / unit * unit;
    };
    blk.resize((size_t)wm.nblocks * 4);
    if (stacked) {
        // A chain stays inside one column of blocks and climbs the planes.  Region g holds, for one
        // q at a time, the columns around the rows of plane q of this column: block (plane p) needs
        // q = p - 1, p, p + 1 and fetches those its chain has not left in place.
        const int64_t P = bands.stack_rows, R = wm.rows_per_block, nplanes = m / P;
        int64_t held[3] = {INT64_MIN, INT64_MIN, INT64_MIN};
        int32_t chain_lo = 0;
        int64_t chain_tiles = 0;
        for (int32_t i = 0; i < wm.nblocks; ++i) {
            const int64_t j = i / nplanes, p = i % nplanes;
            if (i != chain_lo && (p == 0 || chain_tiles >= per_chain)) {
                chains.push_back(chain_lo);
                chains.push_back(i);
                chain_lo = i;
                chain_tiles = 0;
                held[0] = held[1] = held[2] = INT64_MIN;
            }
            blk[(size_t)i * 4 + 0] = h_soff[(size_t)i];
            blk[(size_t)i * 4 + 1] = h_soff[(size_t)i + 1];
            blk[(size_t)i * 4 + 2] = (int32_t)(pcs.size() / 4);
            for (int64_t q = p - 1; q <= p + 1; ++q) {
                const int g = (int)(((q % 3) + 3) % 3);
                int64_t from = 0, to = 0;
                if (held[g] != q) {
                    const int64_t a = std::min<int64_t>(std::max<int64_t>(q * P + j * R + stack_ulo, 0), n);
                    const int64_t z = std::min<int64_t>(std::max<int64_t>(q * P + (j + 1) * R + stack_uhi, 0), n);
                    from = a & ~(int64_t)3;
                    to = z > a ? (z + 3) & ~(int64_t)3 : from;
                    held[g] = q;
                }
                pcs.push_back((int32_t)from);
                pcs.push_back((int32_t)to);
                pcs.push_back(g * bands.stack_size);
                pcs.push_back(bands.stack_size);
            }
            blk[(size_t)i * 4 + 3] = (int32_t)(pcs.size() / 4);
            chain_tiles += h_soff[(size_t)i + 1] - h_soff[(size_t)i];
        }
        chains.push_back(chain_lo);
        chains.push_back(wm.nblocks);
    } else {
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
                int64_t fetch = 0;  // what the block would fetch as the chain's next one, as the kernel counts it
                for (int k = 0; k < bands.nbands; ++k) {  // columns never fetched in this chain, or already overwritten
                    if (hi[k] > lo[k] && have[k] >= 0 &&
                        (lo[k] < low[k] || lo[k] < std::max(have[k], hi[k]) - bands.width[k] + kWindowSlack))
                        fresh = true;
                    const int64_t piece = hi[k] <= lo[k] ? 0 : have[k] < 0 || lo[k] >= have[k] ? hi[k] - lo[k] : std::max(have[k], hi[k]) - have[k];
                    fetch += bands.nbands > 1 ? fetch_unit(piece) : piece;
                }
                if (fetch > kFetchCols) fresh = true;  // more than one round of the fetch registers: only a chain's first block may
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
    }
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
int window_update_values(const WindowMatrix *wm, const T *val, hipStream_t s, const unsigned long long *unless_equal)
{
    const int64_t slots = (int64_t)wm->ntiles * kSlicedTile;
    if (slots == 0 || wm->by_reference) return ASX_STATUS_SUCCESS;  // nothing copied: nothing to bring up to date
    // a bounded grid: where the checksums agree the kernel has nothing to do but to end
    const unsigned grid = (unsigned)std::min<int64_t>(ceil_div64(slots, kBlock), 8192);
    hipLaunchKernelGGL((k_window_regather<T>), dim3(grid), dim3(kBlock), 0, s, wm->perm, slots, val, (T *)wm->val, unless_equal);
    return check_launch();
}

template <typename T>
int launch_spmv_window(int32_t m, int32_t n, T alpha, const WindowMatrix *wm, const T *val, const T *x, T beta, T *y, T *carry,
                       hipStream_t s)
{
    if (m <= 0) return ASX_STATUS_SUCCESS;
    if (wm->has_carry && !carry) return ASX_STATUS_INVALID_POINTER;
    if (wm->by_reference && !val) return ASX_STATUS_INVALID_POINTER;
    // kernels of their own for beta != 0 (y is loaded ahead with the tiles) and for values read in
    // place from A's val (else from the plan's copy)
    const bool bands = wm->nbands != 1, b0 = beta == T(0), in_place = wm->by_reference != 0;
#define ASX_PICK2(NB, BETA) \
    (in_place ? k_spmv_window<T, kWindowWaves, NB, window_depth<T>(NB, BETA), BETA, true> \
              : k_spmv_window<T, kWindowWaves, NB, window_depth<T>(NB, BETA), BETA, false>)
#define ASX_PICK(NB) (b0 ? ASX_PICK2(NB, false) : ASX_PICK2(NB, true))
    const auto kernel = bands ? ASX_PICK(kWindowBands) : ASX_PICK(1);
#undef ASX_PICK
#undef ASX_PICK2
    hipLaunchKernelGGL(kernel, dim3((unsigned)wm->nchains), dim3(kWindowWaves * kWave), 0, s, n, alpha, beta,
                       reinterpret_cast<const int2 *>(wm->chains), reinterpret_cast<const int4 *>(wm->blocks),
                       reinterpret_cast<const int4 *>(wm->pieces), wm->cf, in_place ? val : (const T *)wm->val,
                       reinterpret_cast<const int4 *>(wm->tile_info), x, y, carry);
    if (wm->has_carry)
        hipLaunchKernelGGL((k_window_fixup<T>), dim3((unsigned)ceil_div64(wm->ntiles, kBlock)), dim3(kBlock), 0, s,
                           wm->ntiles, alpha, reinterpret_cast<const int4 *>(wm->tile_info), (const T *)carry, y);
    return check_launch();
}

#define ASX_INST(T)                                                                                               \
    template int build_window<T>(int32_t, int32_t, int32_t, int32_t, bool, const int32_t *, const int32_t *, const T *, \
                                 WindowMatrix *, hipStream_t);                                                    \
    template int window_update_values<T>(const WindowMatrix *, const T *, hipStream_t, const unsigned long long *);                           \
    template int launch_spmv_window<T>(int32_t, int32_t, T, const WindowMatrix *, const T *, const T *, T, T *, T *, hipStream_t);
ASX_INST(float)
ASX_INST(double)
#undef ASX_INST

}  // namespace asx
