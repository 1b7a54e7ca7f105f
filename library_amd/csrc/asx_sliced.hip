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
#include <algorithm>
#include <vector>

#include "asx_internal.hpp"
#include "asx_scan.hpp"
#include "asx_tiles.hpp"

namespace asx {

namespace {

constexpr int32_t kPadRow = 0x7fffffff;

// ---- plan build ---------------------------------------------------------------------------
// The regrouping is a stable counting sort by slice, written for this purpose: the stored
// elements are cut into blocks of kSortElems consecutive ones; a first kernel counts each block's
// elements per slice; an exclusive scan over (slice, block) gives every block its place inside
// every slice; a second kernel ranks the elements of a block inside their slices (stable: row
// order, then column order, survives inside a slice), orders them by slice in LDS and writes
// column, value, source index and row of each straight to its slot, in runs of consecutive slots.
constexpr int kSortThreads = 512;
constexpr int kSortWaves = kSortThreads / kWave;
constexpr int kSortElems = 4096;  // per block
constexpr int kSortPerLane = kSortElems / kSortThreads;
constexpr int kSortWaveElems = kSortElems / kSortWaves;

__global__ __launch_bounds__(kSortThreads) void k_sliced_count(const int32_t *__restrict__ col, int32_t nnz,
                                                                int32_t width, int32_t nslices, int32_t nblocks,
                                                                int32_t *__restrict__ counts)
{
    __shared__ int32_t hist[kSlicedMaxSlices];
    for (int s = threadIdx.x; s < nslices; s += kSortThreads) hist[s] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kSortElems;
#pragma unroll
    for (int k = 0; k < kSortPerLane; ++k) {
        const int64_t i = base + k * kSortThreads + threadIdx.x;
        if (i < nnz) atomicAdd(&hist[col[i] / width], 1);  // integer counts: the order does not matter
    }
    __syncthreads();
    for (int s = threadIdx.x; s < nslices; s += kSortThreads) counts[(int64_t)s * nblocks + blockIdx.x] = hist[s];
    if (blockIdx.x == 0 && threadIdx.x == 0) counts[(int64_t)nslices * nblocks] = 0;
}

// pstart[s] = stored elements in slices before s (s = nslices: all of them)
__global__ __launch_bounds__(kBlock) void k_sliced_slice_starts(const int32_t *__restrict__ offs, int32_t nslices,
                                                                 int32_t nblocks, int32_t *__restrict__ pstart)
{
    const int32_t s = (int32_t)(blockIdx.x * blockDim.x + threadIdx.x);
    if (s <= nslices) pstart[s] = offs[(int64_t)s * nblocks];
}

// largest r in [lo, hi] with row_ptr[r] <= i
__device__ __forceinline__ int32_t row_holding(const int32_t *__restrict__ row_ptr, int32_t lo, int32_t hi, int32_t i)
{
    while (lo < hi) {
        const int32_t mid = lo + (hi - lo + 1) / 2;
        if (row_ptr[mid] <= i)
            lo = mid;
        else
            hi = mid - 1;
    }
    return lo;
}

// in-place exclusive sum of a[0 .. n), n <= 2 * kSortThreads, by the whole workgroup (barriers inside)
__device__ __forceinline__ void block_exclusive_sum(int32_t *a, int n, int32_t *wave_tot)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int32_t v0 = 2 * tid < n ? a[2 * tid] : 0, v1 = 2 * tid + 1 < n ? a[2 * tid + 1] : 0;
    int32_t incl = v0 + v1;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int32_t t = __shfl_up(incl, d, kWave);
        if (lane >= d) incl += t;
    }
    if (lane == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    int32_t before = 0;
    for (int w = 0; w < wave; ++w) before += wave_tot[w];
    const int32_t excl = before + incl - (v0 + v1);
    if (2 * tid < n) a[2 * tid] = excl;
    if (2 * tid + 1 < n) a[2 * tid + 1] = excl + v0;
    __syncthreads();
}

template <typename T>
__device__ __forceinline__ int64_t slot_val_pos(int64_t d)
{
    return d / kSlicedTile * kSlicedTile + tile_val_pos<T>((int)(d % kSlicedTile));
}

// Run-start flags are not known here (they need the neighbours in slice order): cf gets the column
// inside the slice, k_sliced_emit adds bit 15.
template <typename T, int MAXS>
__global__ __launch_bounds__(kSortThreads) void k_sliced_scatter(
    const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col, const T *__restrict__ val,
    const int32_t *__restrict__ seg_row, int32_t m, int32_t nnz, int32_t width, int32_t nslices, int32_t nbits,
    int32_t nblocks, const int32_t *__restrict__ offs, const int32_t *__restrict__ tile_off, int32_t *__restrict__ lrow,
    uint16_t *__restrict__ cf, T *__restrict__ val_out, int32_t *__restrict__ perm, uint16_t *__restrict__ pos,
    int32_t *__restrict__ block_base)
{
    __shared__ int32_t cnt[kSortWaves * MAXS];  // per wave and slice: count, then first rank of the wave's elements
    __shared__ int32_t lofs[MAXS];              // per slice: the block's count, then its first position in slice order
    __shared__ int32_t gbase[MAXS];             // per slice: slot of the block's first element of the slice
    __shared__ int32_t wave_tot[kSortWaves];
    __shared__ int32_t dest[kSortElems];        // slot of the element at each position of the block in slice order
    __shared__ __align__(16) unsigned char stage_raw[kSortElems * 10];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    // consecutive blocks write neighbouring slots of every slice: keep them on one XCD, whose L2
    // then merges their pieces of a cache line (the grid is a multiple of kXcds workgroups)
    const int32_t per_xcd = (int32_t)gridDim.x / kXcds;
    const int32_t b = ((int32_t)blockIdx.x % kXcds) * per_xcd + (int32_t)blockIdx.x / kXcds;
    if (b >= nblocks) return;  // the whole workgroup leaves
    for (int i = tid; i < kSortWaves * nslices; i += kSortThreads) cnt[i] = 0;
    __syncthreads();
    int32_t *mycnt = cnt + wave * nslices;
    const int64_t wbase = (int64_t)b * kSortElems + (int64_t)wave * kSortWaveElems;
    int32_t c[kSortPerLane], rk[kSortPerLane];
#pragma unroll
    for (int k = 0; k < kSortPerLane; ++k) {
        const int64_t i = wbase + k * kWave + lane;
        c[k] = i < nnz ? col[i] : 0;
    }
    // rank of every element among the wave's elements of its slice, in element order: the wave
    // takes its elements 64 at a time; inside a step the lanes of one slice find each other by
    // ballots over the bits of the slice number
#pragma unroll
    for (int k = 0; k < kSortPerLane; ++k) {
        const bool valid = wbase + k * kWave + lane < nnz;
        const int32_t key = c[k] / width;
        unsigned long long same = __ballot(valid);
        for (int bit = 0; bit < nbits; ++bit) {
            const bool one = (key >> bit) & 1;
            const unsigned long long bal = __ballot(one);
            same &= one ? bal : ~bal;
        }
        const int below = lanes_below(same);  // lanes of this slice before this one
        const int32_t prev = valid ? mycnt[key] : 0;
        rk[k] = prev + below;
        if (valid && below == 0) mycnt[key] = prev + __popcll(same);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();
    for (int s = tid; s < nslices; s += kSortThreads) {
        int32_t run = 0;
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) {
            const int32_t t = cnt[w * nslices + s];
            cnt[w * nslices + s] = run;
            run += t;
        }
        lofs[s] = run;
        gbase[s] = tile_off[s] * kSlicedTile + offs[(int64_t)s * nblocks + b] - offs[(int64_t)s * nblocks];
        // for k_sliced_rescatter: where the block's elements of every slice start (row nblocks: where the slice's end)
        block_base[(int64_t)b * nslices + s] = gbase[s];
        if (b == nblocks - 1)
            block_base[(int64_t)nblocks * nslices + s] =
                tile_off[s] * kSlicedTile + offs[(int64_t)s * nblocks + nblocks] - offs[(int64_t)s * nblocks];
    }
    __syncthreads();
    block_exclusive_sum(lofs, nslices, wave_tot);
    // rows: the wave's 512 elements lie in rows seg_row[g] .. seg_row[g + 1]
    const int64_t g = wbase / kSortWaveElems;
    int32_t r_lo = 0, r_hi = m - 1;
    if (wbase < nnz) {
        r_lo = seg_row[g];
        r_hi = seg_row[g + 1];
        r_hi = r_hi > m - 1 ? m - 1 : r_hi;
    }
    int32_t *row_s = reinterpret_cast<int32_t *>(stage_raw), *src_s = row_s + kSortElems;
#pragma unroll
    for (int k = 0; k < kSortPerLane; ++k) {
        const int64_t i = wbase + k * kWave + lane;
        if (i < nnz) {
            const int32_t key = c[k] / width;
            const int32_t in_slice = mycnt[key] + rk[k];
            const int32_t p = lofs[key] + in_slice;
            rk[k] = p;
            pos[i] = (uint16_t)p;
            dest[p] = gbase[key] + in_slice;
            row_s[p] = row_holding(row_ptr, r_lo, r_hi, (int32_t)i);
            src_s[p] = (int32_t)i;
        }
    }
    __syncthreads();
    const int64_t left = (int64_t)nnz - (int64_t)b * kSortElems;
    const int32_t count = left < kSortElems ? (int32_t)left : kSortElems;
    for (int j = tid; j < count; j += kSortThreads) {
        const int64_t d = dest[j];
        lrow[d] = row_s[j];
        perm[slot_val_pos<T>(d)] = src_s[j];
    }
    __syncthreads();
    T *val_s = reinterpret_cast<T *>(stage_raw);
    uint16_t *cf_s = reinterpret_cast<uint16_t *>(stage_raw + (size_t)kSortElems * 8);
    T v[kSortPerLane];
#pragma unroll
    for (int k = 0; k < kSortPerLane; ++k) {
        const int64_t i = wbase + k * kWave + lane;
        v[k] = i < nnz ? val[i] : T(0);
    }
#pragma unroll
    for (int k = 0; k < kSortPerLane; ++k) {
        if (wbase + k * kWave + lane < nnz) {
            val_s[rk[k]] = v[k];
            cf_s[rk[k]] = (uint16_t)(c[k] % width);
        }
    }
    __syncthreads();
    for (int j = tid; j < count; j += kSortThreads) {
        const int64_t d = dest[j];
        val_out[slot_val_pos<T>(d)] = val_s[j];
        cf[d] = cf_s[j];
    }
}

// The slots behind a slice's last stored element, up to the end of its last tile, are pads: runs
// of their own with value 0 whose partial sums no row block reads.  One workgroup per slice.
template <typename T>
__global__ __launch_bounds__(kSlicedTile) void k_sliced_pads(const int32_t *__restrict__ pstart,
                                                              const int32_t *__restrict__ tile_off,
                                                              int32_t *__restrict__ lrow, uint16_t *__restrict__ cf,
                                                              T *__restrict__ val, int32_t *__restrict__ perm)
{
    const int32_t s = blockIdx.x;
    const int64_t d = (int64_t)tile_off[s] * kSlicedTile + (pstart[s + 1] - pstart[s]) + threadIdx.x;
    if (d >= (int64_t)tile_off[s + 1] * kSlicedTile) return;
    lrow[d] = kPadRow;
    cf[d] = 0x8000u;
    val[slot_val_pos<T>(d)] = T(0);
    perm[slot_val_pos<T>(d)] = -1;
}

// Run starts of a tile (one wave per tile, 4 consecutive slots per lane): a slot starts a run if
// it is the tile's first, if its row differs from the slot before it, or if it is a pad.
struct TileRuns {
    int32_t r[4];
    bool h[4];
    int before;  // run starts in the lanes below
    int total;
    __device__ __forceinline__ void load(const int32_t *__restrict__ lrow, int64_t t, int lane)
    {
        const int4 q = reinterpret_cast<const int4 *>(lrow + t * kSlicedTile)[lane];
        r[0] = q.x, r[1] = q.y, r[2] = q.z, r[3] = q.w;
        const int32_t prev = __shfl_up(q.w, 1, kWave);
        h[0] = lane == 0 || r[0] != prev || r[0] == kPadRow;
#pragma unroll
        for (int j = 1; j < 4; ++j) h[j] = r[j] != r[j - 1] || r[j] == kPadRow;
        const unsigned long long m0 = __ballot(h[0]), m1 = __ballot(h[1]), m2 = __ballot(h[2]), m3 = __ballot(h[3]);
        before = lanes_below(m0) + lanes_below(m1) + lanes_below(m2) + lanes_below(m3);
        total = __popcll(m0) + __popcll(m1) + __popcll(m2) + __popcll(m3);
    }
};

__global__ __launch_bounds__(kBlock) void k_sliced_tile_runs(const int32_t *__restrict__ lrow, int32_t ntiles,
                                                              int32_t *__restrict__ tile_cnt)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t t = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    if (t >= ntiles) return;  // whole waves leave
    TileRuns tr;
    tr.load(lrow, t, lane);
    if (lane == 0) tile_cnt[t] = tr.total;
    if (t == 0 && lane == 0) tile_cnt[ntiles] = 0;
}

// Per run: its row inside the row block (prow); per slot: the run-start bit of cf; per (row
// block, slice): the first partial sum of the block in the slice (chunk_lo), written by the run
// that is the first at or past the block's first row - and, behind a slice's last stored element,
// for all the blocks that follow.
__global__ __launch_bounds__(kBlock) void k_sliced_emit(const int32_t *__restrict__ lrow,
                                                         const int32_t *__restrict__ tile_base,
                                                         const int32_t *__restrict__ tile_off, int32_t ntiles,
                                                         int32_t nslices, int32_t rpw, int32_t nrb,
                                                         uint16_t *__restrict__ cf, uint16_t *__restrict__ prow,
                                                         int32_t *__restrict__ chunk_lo)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t t = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    if (t >= ntiles) return;  // whole waves leave
    int32_t lo = 0, hi = nslices - 1;  // slice of tile t: largest s with tile_off[s] <= t (uniform)
    while (lo < hi) {
        const int32_t mid = lo + (hi - lo + 1) / 2;
        if (tile_off[mid] <= t)
            lo = mid;
        else
            hi = mid - 1;
    }
    const int32_t s = lo;
    const bool first_tile = t == tile_off[s], last_tile = t + 1 == tile_off[s + 1];
    TileRuns tr;
    tr.load(lrow, t, lane);
    const int32_t base = tile_base[t];
    // row of the slot before the lane's first one (-1: none in this slice)
    int32_t prev = __shfl_up(tr.r[3], 1, kWave);
    if (lane == 0) prev = first_tile ? -1 : lrow[t * kSlicedTile - 1];
    // row of the slot behind the lane's last one (a pad, if the slice ends there)
    int32_t next = __shfl_down(tr.r[0], 1, kWave);
    if (lane == kWave - 1) next = last_tile ? kPadRow : lrow[(t + 1) * kSlicedTile];
    typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
    u16x4 *cfp = reinterpret_cast<u16x4 *>(cf + t * kSlicedTile) + lane;
    u16x4 w = *cfp;
    int id = base + tr.before - 1;  // run the slot before the lane's first one belongs to
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int32_t r = tr.r[j];
        const int32_t before = j == 0 ? prev : tr.r[j - 1];
        const int32_t after = j == 3 ? next : tr.r[j + 1];
        if (tr.h[j]) {
            ++id;
            w[j] |= 0x8000u;
            // bit 15: may continue the row of the partial sum before it (a run cut at a tile start)
            const bool cont = lane == 0 && j == 0 && before == r && r != kPadRow;
            prow[id] = (uint16_t)((r % rpw) | (cont ? 0x8000 : 0));
            if (r != kPadRow) {
                const int32_t rb = r / rpw;
                for (int32_t q = before < 0 ? 0 : before / rpw + 1; q <= rb; ++q) chunk_lo[(int64_t)q * nslices + s] = id;
            }
        }
        if (r != kPadRow && after == kPadRow)  // the slice's last stored element
            for (int32_t q = r / rpw + 1; q <= nrb; ++q) chunk_lo[(int64_t)q * nslices + s] = id + 1;
    }
    *cfp = w;
}

// slices without stored elements: every row block's range is empty
__global__ __launch_bounds__(kBlock) void k_sliced_empty_slices(const int32_t *__restrict__ tile_base,
                                                                 const int32_t *__restrict__ tile_off, int32_t nslices,
                                                                 int32_t nrb, int32_t *__restrict__ chunk_lo)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= ((int64_t)nrb + 1) * nslices) return;
    const int32_t s = (int32_t)(i % nslices);
    if (tile_off[s] == tile_off[s + 1]) chunk_lo[i] = tile_base[tile_off[s]];
}


// The values of A once more into a plan's slots (asx_plan_update_values), from the side of A: a
// workgroup reads kSortElems consecutive values and, for each, its position among the block's
// elements in slice order (kept from the build: 2 bytes), orders them so in LDS, and writes them
// out as the build did, a run of consecutive slots per slice (where each run starts: block_base,
// also kept).  Reading through the slots' source indices instead (one thread per slot) takes a
// 32-byte sector of A's values for every value: 371 us on the power-law matrix, three multiplies.
// `unless_equal` (may be null): four words, two checksums of the values now and two of the values
// the copy holds; where they agree nothing is done.
template <typename T, int MAXS>
__global__ __launch_bounds__(kSortThreads) void k_sliced_rescatter(const T *__restrict__ val, int32_t nnz, int32_t nslices,
                                                                   int32_t nblocks, const uint16_t *__restrict__ pos,
                                                                   const int32_t *__restrict__ block_base,
                                                                   T *__restrict__ val_out,
                                                                   const unsigned long long *unless_equal)
{
    __shared__ int32_t lofs[MAXS];      // per slice: the block's count, then its first position in slice order
    __shared__ int32_t gbase[MAXS];     // per slice: slot of the block's first element of the slice
    __shared__ int32_t wave_tot[kSortWaves];
    __shared__ T val_s[kSortElems];
    if (unless_equal && unless_equal[0] == unless_equal[2] && unless_equal[1] == unless_equal[3]) return;  // uniform
    const int tid = threadIdx.x;
    const int32_t per_xcd = (int32_t)gridDim.x / kXcds;  // as in k_sliced_scatter: neighbouring blocks on one XCD
    const int32_t b = ((int32_t)blockIdx.x % kXcds) * per_xcd + (int32_t)blockIdx.x / kXcds;
    if (b >= nblocks) return;  // the whole workgroup leaves
    const int64_t base = (int64_t)b * kSortElems;
    const int64_t left = (int64_t)nnz - base;
    const int32_t count = left < kSortElems ? (int32_t)left : kSortElems;
    T v[kSortPerLane];
    uint16_t p[kSortPerLane];
#pragma unroll
    for (int k = 0; k < kSortPerLane; ++k) {
        const int32_t j = k * kSortThreads + tid;
        v[k] = j < count ? val[base + j] : T(0);
        p[k] = j < count ? pos[base + j] : (uint16_t)0;
    }
    for (int s = tid; s < nslices; s += kSortThreads) {
        const int32_t g = block_base[(int64_t)b * nslices + s];
        gbase[s] = g;
        lofs[s] = block_base[(int64_t)(b + 1) * nslices + s] - g;
    }
    __syncthreads();
    block_exclusive_sum(lofs, nslices, wave_tot);
#pragma unroll
    for (int k = 0; k < kSortPerLane; ++k)
        if (k * kSortThreads + tid < count) val_s[p[k]] = v[k];
    __syncthreads();
    for (int j = tid; j < count; j += kSortThreads) {
        int lo = 0, hi = nslices - 1;  // the slice of position j: the last one that starts at or before j
        while (lo < hi) {
            const int mid = lo + (hi - lo + 1) / 2;
            if (lofs[mid] <= j)
                lo = mid;
            else
                hi = mid - 1;
        }
        val_out[slot_val_pos<T>((int64_t)gbase[lo] + (j - lofs[lo]))] = val_s[j];
    }
}

// ---- pass 1 ------------------------------------------------------------------------------
// A run's sum goes, at the run's rank, into the wave's staging area in LDS; the tile's sums then
// leave as stores of consecutive lanes to consecutive partial sums.
constexpr int kStageRuns = kSlicedTile;  // every run of a tile
template <typename T>
struct StageRun {
    T *stage;
    __device__ __forceinline__ void operator()(bool wanted, int rank, T v) const
    {
        if (wanted) stage[rank] = v;
    }
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

// A workgroup takes the pieces wg_pieces[2 blockIdx.x].x .. .y - 1 of `pieces` in turn: tiles .y .. .z - 1
// of slice .x each (nearly always one piece; two where the workgroup's share of the tiles reaches
// over the end of a slice).  wg_pieces[2 blockIdx.x + 1] repeats the first of them, so that the
// kernel's first loads wait for one read of a table, not two.
template <typename T, int WIDTH, int NW, int D>
__global__ __launch_bounds__(NW *kWave) void k_sliced_products(int32_t n, const int4 *__restrict__ wg_pieces,
                                                               const int4 *__restrict__ pieces,
                                                               const uint16_t *__restrict__ cf,
                                                               const T *__restrict__ val,
                                                               const int32_t *__restrict__ tile_base,
                                                               const T *__restrict__ x, T *__restrict__ partial)
{
    __shared__ T xs[WIDTH];
    __shared__ T stage_all[NW * kStageRuns];
    const int4 mine = wg_pieces[2 * blockIdx.x];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    T *stage = stage_all + wave * kStageRuns;
    for (int32_t pc = mine.x; pc < mine.y; ++pc) {  // uniform over the workgroup
        const int4 wg = pc == mine.x ? wg_pieces[2 * blockIdx.x + 1] : pieces[pc];
        const int64_t c0 = (int64_t)wg.x * WIDTH;
        const int32_t cnt = n - c0 < WIDTH ? (int32_t)(n - c0) : WIDTH;
        // the first tiles' loads go out before the slice of x is fetched (they do not need it)
        const int32_t last = wg.z - 1;
        Tile<T> tl[D];
        int32_t t = wg.y + wave;
#pragma unroll
        for (int d = 0; d < D; ++d) tile_load<T>(tl[d], t + d * NW < last ? t + d * NW : last, lane, cf, val, tile_base);
        if (pc != mine.x) __syncthreads();  // every wave is done with the slice before
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
}

// ---- pass 2 ------------------------------------------------------------------------------
// The partial sums of a row block, range after range in slice order, are cut (when the plan is
// built) into steps of up to 64 entries.  A step takes its entries from up to kPieces consecutive
// pieces of ranges (a range may be split between steps); lane l reads entry base[p] + l of the
// piece p it falls in.  Descriptor of a step: base[0..2], then
// first lane of piece 1 | first lane of piece 2 << 8 | entries << 16.
constexpr int kPieces = 3;
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));

// One wave per row block walks the block's ranges (loaded 64 slices at a time, then read lane by
// lane: the walk itself is serial); `psteps == nullptr`: only count.
__global__ __launch_bounds__(kBlock) void k_sliced_pack(const int32_t *__restrict__ chunk_lo, int32_t nrb,
                                                         int32_t nslices, const int32_t *__restrict__ pstep_ptr,
                                                         int32_t *__restrict__ count, i32x4 *__restrict__ psteps)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t b = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    if (b >= nrb) return;  // whole waves leave
    const int32_t *lo_row = chunk_lo + b * nslices, *hi_row = lo_row + nslices;
    i32x4 *out = psteps ? psteps + pstep_ptr[b] : nullptr;
    int32_t nsteps = 0, fill = 0, pieces = 0;
    int32_t base0 = 0, base1 = 0, base2 = 0, first1 = kWave, first2 = kWave;
    for (int32_t s0 = 0; s0 < nslices; s0 += kWave) {
        const int32_t ns = nslices - s0 < kWave ? nslices - s0 : kWave;
        const int32_t lo_v = lane < ns ? lo_row[s0 + lane] : 0;
        const int32_t len_v = lane < ns ? hi_row[s0 + lane] - lo_v : 0;
        unsigned long long todo = __ballot(len_v > 0);
        while (todo) {  // uniform
            const int j = __builtin_ctzll(todo);
            todo &= todo - 1;
            int32_t lo = __builtin_amdgcn_readlane(lo_v, j), len = __builtin_amdgcn_readlane(len_v, j);
            while (len > 0) {
                if (pieces == kPieces || fill == kWave) {
                    if (out && lane == 0) out[nsteps] = i32x4{base0, base1, base2, first1 | first2 << 8 | fill << 16};
                    ++nsteps;
                    fill = pieces = 0;
                    first1 = first2 = kWave;
                }
                const int32_t take = len < kWave - fill ? len : kWave - fill;
                if (pieces == 0)
                    base0 = lo - fill;
                else if (pieces == 1)
                    base1 = lo - fill, first1 = fill;
                else
                    base2 = lo - fill, first2 = fill;
                ++pieces;
                fill += take;
                lo += take;
                len -= take;
            }
        }
    }
    if (fill > 0) {
        if (out && lane == 0) out[nsteps] = i32x4{base0, base1, base2, first1 | first2 << 8 | fill << 16};
        ++nsteps;
    }
    if (!psteps && lane == 0) count[b] = nsteps;
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
    for (void *q : {p->store, p->partial, (void *)p->prow, (void *)p->psteps})
        if (q) (void)hipFree(q);
    p->store = p->val = p->partial = nullptr;
    p->cf = p->prow = nullptr;
    p->perm = p->tile_base = p->wg_tab = p->wg_pieces = p->chunk_lo = p->pstep_ptr = p->psteps = p->block_base = nullptr;
    p->pos = nullptr;
}

template <typename T>
int build_sliced(int32_t m, int32_t n, int32_t nnz, int32_t width, int32_t rows_per_wave, int32_t target_wgs,
                 const int32_t *row_ptr, const int32_t *col, const T *val, SlicedMatrix *out, hipStream_t s)
{
    SlicedMatrix sm{};
    if (m <= 0 || nnz <= 0 || n <= 0) return ASX_STATUS_INVALID_SIZE;
    if (width < 1 || width > 32768 || rows_per_wave < 1 || rows_per_wave > 32767 || target_wgs < 1)
        return ASX_STATUS_INVALID_VALUE;
    sm.width = width;
    sm.nslices = (int32_t)ceil_div64(n, width);
    if (sm.nslices > kSlicedMaxSlices) return ASX_STATUS_NOT_SUPPORTED;
    sm.rows_per_wave = rows_per_wave;
    sm.nrb = (int32_t)ceil_div64(m, rows_per_wave);
    int nbits = 0;
    while ((1 << nbits) < sm.nslices) ++nbits;
    const int32_t nblocks = (int32_t)ceil_div64(nnz, kSortElems);
    const int32_t nseg = (int32_t)ceil_div64(nnz, kSortWaveElems);
    const int64_t ncount = (int64_t)sm.nslices * nblocks + 1;
    const int64_t cap64 = (int64_t)nnz + (int64_t)(kSlicedTile - 1) * sm.nslices;  // the most slots there can be
    const int64_t ncells = ((int64_t)sm.nrb + 1) * sm.nslices;
    if (cap64 > 0x7fffffff || ncount > 0x7fffffff || ncells > 0x7fffffff) return ASX_STATUS_INVALID_SIZE;

    int st = ASX_STATUS_SUCCESS;
    // Scratch of the build in one allocation: per-(slice, block) counts and their scan, the row
    // holding every 512th stored element, slice offsets (elements, tiles), the row of every slot,
    // per-tile and per-row-block counts, the scans' block sums.
    char *arena = nullptr;
    int32_t *counts = nullptr, *offs = nullptr, *seg_row = nullptr, *d_pstart = nullptr, *d_tile_off = nullptr;
    int32_t *lrow = nullptr, *tile_cnt = nullptr, *step_cnt = nullptr;
    int32_t *tmp = nullptr;
    std::vector<int32_t> pstart((size_t)sm.nslices + 1), tile_off((size_t)sm.nslices + 1, 0);
    std::vector<int32_t> tab, wgs;
    int64_t slots = 0;
    bool empty_slice = false;
    const size_t max_tiles = (size_t)ceil_div64(cap64, kSlicedTile);
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
    {
        size_t off = 0;
        const auto take = [&off](size_t count) {
            const size_t at = off;
            off += align_up(count * sizeof(int32_t), 256);
            return at;
        };
        const size_t o_counts = take((size_t)ncount), o_offs = take((size_t)ncount), o_seg = take((size_t)nseg + 1);
        const size_t o_pstart = take((size_t)sm.nslices + 1), o_toff = take((size_t)sm.nslices + 1);
        const size_t o_lrow = take((size_t)cap64), o_tcnt = take(max_tiles + 1), o_scnt = take((size_t)sm.nrb + 1);
        const size_t o_tmp = take(scan_scratch_ints(std::max<int64_t>(ncount, (int64_t)max_tiles + 1)));
        ASX_TRY(hipMalloc((void **)&arena, off));
        counts = (int32_t *)(arena + o_counts), offs = (int32_t *)(arena + o_offs), seg_row = (int32_t *)(arena + o_seg);
        d_pstart = (int32_t *)(arena + o_pstart), d_tile_off = (int32_t *)(arena + o_toff);
        lrow = (int32_t *)(arena + o_lrow), tile_cnt = (int32_t *)(arena + o_tcnt), step_cnt = (int32_t *)(arena + o_scnt);
        tmp = (int32_t *)(arena + o_tmp);
    }

    // 1. every block's stored elements per slice, and from their scan the block's place in each slice
    hipLaunchKernelGGL(k_sliced_count, dim3((unsigned)nblocks), dim3(kSortThreads), 0, s, col, nnz, width, sm.nslices,
                       nblocks, counts);
    ASX_TRY_ST(launch_exclusive_scan_i32(counts, offs, ncount, tmp, s));
    hipLaunchKernelGGL(k_sliced_slice_starts, dim3((unsigned)ceil_div64((int64_t)sm.nslices + 1, kBlock)), dim3(kBlock), 0, s,
                       offs, sm.nslices, nblocks, d_pstart);
    ASX_TRY(hipMemcpyAsync(pstart.data(), d_pstart, sizeof(int32_t) * pstart.size(), hipMemcpyDeviceToHost, s));
    ASX_TRY_ST(launch_nnz_split_rows(row_ptr, m, nnz, kSortWaveElems, seg_row, s));  // runs while the host waits
    ASX_TRY(hipStreamSynchronize(s));

    // 2. tiles: every slice starts a new tile
    for (int32_t sl = 0; sl < sm.nslices; ++sl) {
        tile_off[sl + 1] = tile_off[sl] + (int32_t)ceil_div64(pstart[sl + 1] - pstart[sl], kSlicedTile);
        empty_slice |= pstart[sl + 1] == pstart[sl];
    }
    sm.ntiles = tile_off[sm.nslices];
    slots = (int64_t)sm.ntiles * kSlicedTile;
    ASX_TRY(hipMemcpyAsync(d_tile_off, tile_off.data(), sizeof(int32_t) * tile_off.size(), hipMemcpyHostToDevice, s));
    //    workgroups of pass 1: about `target_wgs` equal shares of the tiles, whatever slices they lie
    //    in (a share per slice, rounded, left 270 workgroups for 256 compute units where 54 slices
    //    wanted 4.7 each: two rounds).  A cut that falls within 32 tiles of the start of a slice
    //    moves there; a share that still reaches over such a start is worked off as two pieces,
    //    one slice of x after the other.  No share smaller than 32 tiles unless there is only one.
    {
        const int64_t nt = sm.ntiles;
        const int32_t shares = (int32_t)std::max<int64_t>(1, std::min<int64_t>(target_wgs, nt / 32));
        std::vector<int32_t> cuts((size_t)shares + 1);
        for (int32_t k = 0; k <= shares; ++k) {
            int32_t c = (int32_t)(nt * k / shares);
            // the start of a slice nearest to c, when fewer than 32 tiles away
            const auto at = std::lower_bound(tile_off.begin(), tile_off.end(), c);
            const int32_t above = at != tile_off.end() ? *at - c : 32, below = at != tile_off.begin() ? c - *(at - 1) : 32;
            if (above < 32 && above <= below)
                c += above;
            else if (below < 32)
                c -= below;
            cuts[(size_t)k] = k == 0 ? 0 : k == shares ? (int32_t)nt : std::max(c, cuts[(size_t)k - 1]);
        }
        int32_t sl = 0;
        for (int32_t k = 0; k < shares; ++k) {
            const int32_t lo = cuts[(size_t)k], hi = cuts[(size_t)k + 1];
            if (hi <= lo) continue;
            const int32_t first_piece = (int32_t)(tab.size() / 4);
            while (tile_off[(size_t)sl + 1] <= lo) ++sl;  // the slice that holds tile lo
            for (int32_t a = lo; a < hi;) {
                while (tile_off[(size_t)sl + 1] <= a) ++sl;
                const int32_t z = std::min(hi, tile_off[(size_t)sl + 1]);
                tab.push_back(sl);
                tab.push_back(a);
                tab.push_back(z);
                tab.push_back(0);
                a = z;
            }
            wgs.push_back(first_piece);
            wgs.push_back((int32_t)(tab.size() / 4));
            wgs.push_back(0);
            wgs.push_back(0);
            for (int q = 0; q < 4; ++q) wgs.push_back(tab[(size_t)first_piece * 4 + q]);  // the first piece again
        }
        sm.npieces = (int32_t)(tab.size() / 4);
        sm.nwg = (int32_t)(wgs.size() / 8);
        // Workgroups next to each other in this list share slices of x: keep them on one XCD, whose
        // L2 then fetches a slice once (workgroup i runs on XCD i mod kXcds; entry j of the list goes
        // to position (j mod per_xcd) * kXcds + j / per_xcd, so consecutive entries share an XCD).
        if (sm.nwg % kXcds == 0 && sm.nwg > 0) {
            const int32_t per_xcd = sm.nwg / kXcds;
            std::vector<int32_t> placed(wgs.size());
            for (int32_t j = 0; j < sm.nwg; ++j) {
                const int32_t i = (j % per_xcd) * kXcds + j / per_xcd;
                for (int q = 0; q < 8; ++q) placed[(size_t)i * 8 + q] = wgs[(size_t)j * 8 + q];
            }
            wgs.swap(placed);
        }
    }
    {   // what the plan keeps and whose size is known by now, in one allocation
        size_t off = 0;
        const auto take = [&off](size_t bytes) {
            const size_t at = off;
            off += align_up(bytes, 256);
            return at;
        };
        const size_t o_val = take(sizeof(T) * (size_t)slots), o_perm = take(sizeof(int32_t) * (size_t)slots);
        const size_t o_cf = take(sizeof(uint16_t) * (size_t)slots), o_tb = take(sizeof(int32_t) * ((size_t)sm.ntiles + 1));
        const size_t o_wg = take(sizeof(int32_t) * std::max<size_t>(tab.size() + wgs.size(), 4));
        const size_t o_cl = take(sizeof(int32_t) * (size_t)ncells), o_sp = take(sizeof(int32_t) * ((size_t)sm.nrb + 1));
        const size_t o_pos = take(sizeof(uint16_t) * (size_t)nnz);
        const size_t o_bb = take(sizeof(int32_t) * ((size_t)nblocks + 1) * (size_t)sm.nslices);
        ASX_TRY(hipMalloc(&sm.store, off));
        char *base = static_cast<char *>(sm.store);
        sm.val = base + o_val, sm.perm = (int32_t *)(base + o_perm), sm.cf = (uint16_t *)(base + o_cf);
        sm.tile_base = (int32_t *)(base + o_tb), sm.wg_tab = (int32_t *)(base + o_wg);
        sm.chunk_lo = (int32_t *)(base + o_cl), sm.pstep_ptr = (int32_t *)(base + o_sp);
        sm.wg_pieces = sm.wg_tab + tab.size();
        sm.pos = (uint16_t *)(base + o_pos), sm.block_base = (int32_t *)(base + o_bb);
        sm.nnz = nnz, sm.nsort_blocks = nblocks;
        ASX_TRY(hipMemcpyAsync(sm.wg_tab, tab.data(), sizeof(int32_t) * tab.size(), hipMemcpyHostToDevice, s));
        ASX_TRY(hipMemcpyAsync(sm.wg_pieces, wgs.data(), sizeof(int32_t) * wgs.size(), hipMemcpyHostToDevice, s));
    }
    // 3. every stored element to its slot; the pads behind every slice
    {
        const unsigned sgrid = (unsigned)(ceil_div64(nblocks, kXcds) * kXcds);
#define ASX_SCATTER(MAXS)                                                                                              \
    hipLaunchKernelGGL((k_sliced_scatter<T, MAXS>), dim3(sgrid), dim3(kSortThreads), 0, s, row_ptr, col, val, seg_row, m, \
                       nnz, width, sm.nslices, nbits, nblocks, offs, d_tile_off, lrow, sm.cf, (T *)sm.val, sm.perm, sm.pos,     \
                       sm.block_base)
        if (sm.nslices <= 256)
            ASX_SCATTER(256);
        else
            ASX_SCATTER(kSlicedMaxSlices);
#undef ASX_SCATTER
        hipLaunchKernelGGL((k_sliced_pads<T>), dim3((unsigned)sm.nslices), dim3(kSlicedTile), 0, s, d_pstart, d_tile_off, lrow,
                           sm.cf, (T *)sm.val, sm.perm);
    }
    // 4. partial sums: one per run start; tile_base = the run starts before each tile
    {
        const unsigned wgrid = (unsigned)ceil_div64((int64_t)sm.ntiles * kWave, kBlock);
        hipLaunchKernelGGL(k_sliced_tile_runs, dim3(wgrid), dim3(kBlock), 0, s, lrow, sm.ntiles, tile_cnt);
        ASX_TRY_ST(launch_exclusive_scan_i32(tile_cnt, sm.tile_base, (int64_t)sm.ntiles + 1, tmp, s));
        ASX_TRY(hipMemcpyAsync(&sm.npartials, sm.tile_base + sm.ntiles, sizeof(int32_t), hipMemcpyDeviceToHost, s));
        ASX_TRY(hipStreamSynchronize(s));
        ASX_TRY(hipMalloc((void **)&sm.prow, sizeof(uint16_t) * ((size_t)sm.npartials + kSlicedReducePad)));
        ASX_TRY(hipMemsetAsync(sm.prow + sm.npartials, 0, sizeof(uint16_t) * kSlicedReducePad, s));
        // 5. rows of the partial sums, run-start bits, and where each row block starts inside each slice
        hipLaunchKernelGGL(k_sliced_emit, dim3(wgrid), dim3(kBlock), 0, s, lrow, sm.tile_base, d_tile_off, sm.ntiles,
                           sm.nslices, rows_per_wave, sm.nrb, sm.cf, sm.prow, sm.chunk_lo);
        if (empty_slice)
            hipLaunchKernelGGL(k_sliced_empty_slices, dim3((unsigned)ceil_div64(ncells, kBlock)), dim3(kBlock), 0, s,
                               sm.tile_base, d_tile_off, sm.nslices, sm.nrb, sm.chunk_lo);
    }
    // 6. the steps in which pass 2 reads each row block's ranges
    {
        const unsigned pgrid = (unsigned)ceil_div64((int64_t)sm.nrb * kWave, kBlock);
        ASX_TRY(hipMemsetAsync(step_cnt + sm.nrb, 0, sizeof(int32_t), s));
        hipLaunchKernelGGL(k_sliced_pack, dim3(pgrid), dim3(kBlock), 0, s, sm.chunk_lo, sm.nrb, sm.nslices, nullptr, step_cnt,
                           nullptr);
        ASX_TRY_ST(launch_exclusive_scan_i32(step_cnt, sm.pstep_ptr, (int64_t)sm.nrb + 1, tmp, s));
        ASX_TRY(hipMemcpyAsync(&sm.npsteps, sm.pstep_ptr + sm.nrb, sizeof(int32_t), hipMemcpyDeviceToHost, s));
        ASX_TRY(hipMalloc(&sm.partial, sizeof(T) * ((size_t)sm.npartials + kSlicedReducePad)));  // while the kernels run
        ASX_TRY(hipStreamSynchronize(s));
        ASX_TRY(hipMalloc((void **)&sm.psteps, sizeof(int32_t) * 4 * ((size_t)sm.npsteps + kSlicedStepPad)));
        ASX_TRY(hipMemsetAsync(sm.psteps + 4 * (size_t)sm.npsteps, 0, sizeof(int32_t) * 4 * kSlicedStepPad, s));
        hipLaunchKernelGGL(k_sliced_pack, dim3(pgrid), dim3(kBlock), 0, s, sm.chunk_lo, sm.nrb, sm.nslices, sm.pstep_ptr,
                           nullptr, reinterpret_cast<i32x4 *>(sm.psteps));
    }
    ASX_TRY(hipStreamSynchronize(s));
    ASX_TRY(hipGetLastError());
#undef ASX_TRY
#undef ASX_TRY_ST
done:
    if (arena) (void)hipFree(arena);
    if (st) {
        free_sliced(&sm);
        return st;
    }
    *out = sm;
    return ASX_STATUS_SUCCESS;
}


template <typename T>
int sliced_update_values(const SlicedMatrix *sm, const T *val, hipStream_t s, const unsigned long long *unless_equal)
{
    const int64_t slots = (int64_t)sm->ntiles * kSlicedTile;
    if (slots == 0) return ASX_STATUS_SUCCESS;
    // the pads keep the zeros the build gave them; where the checksums agree the kernel has nothing to do but to end
    const unsigned grid = (unsigned)(ceil_div64(sm->nsort_blocks, kXcds) * kXcds);
    if (sm->nslices <= 256)
        hipLaunchKernelGGL((k_sliced_rescatter<T, 256>), dim3(grid), dim3(kSortThreads), 0, s, val, sm->nnz, sm->nslices,
                           sm->nsort_blocks, sm->pos, sm->block_base, (T *)sm->val, unless_equal);
    else
        hipLaunchKernelGGL((k_sliced_rescatter<T, kSlicedMaxSlices>), dim3(grid), dim3(kSortThreads), 0, s, val, sm->nnz,
                           sm->nslices, sm->nsort_blocks, sm->pos, sm->block_base, (T *)sm->val, unless_equal);
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
    hipLaunchKernelGGL((k_sliced_products<T, W, 16, kDepth>), dim3((unsigned)sm->nwg), dim3(16 * kWave), 0, s, n,      \
                       reinterpret_cast<const int4 *>(sm->wg_pieces), tab, sm->cf, (const T *)sm->val, sm->tile_base, x, partial)
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
    template int sliced_update_values<T>(const SlicedMatrix *, const T *, hipStream_t, const unsigned long long *);                          \
    template int launch_spmv_sliced<T>(int32_t, int32_t, T, const SlicedMatrix *, const T *, T, T *, T *, hipStream_t);
ASX_INST(float)
ASX_INST(double)
#undef ASX_INST

}  // namespace asx
