// Internal declarations shared by the HIP translation units of libalphasparse_amd.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/alphasparse_amd.h"
#include "asx_device.hpp"

namespace asx {

// Tile geometry of the SpMV kernels (one workgroup of 256 threads per tile).
constexpr int kBlock = 256;
constexpr int kMergeItemsPerThread = 8;
constexpr int kMergeTile = kBlock * kMergeItemsPerThread;  // rows + stored elements per tile
constexpr int kStreamTile = 1024;                          // stored elements per row block
constexpr int kFlatTile = 1024;                            // stored elements per flat tile
constexpr int kLongRow = 8192;  // DEFAULT (with a plan) switches to the merge-path kernel above this row length
// SpMM: merge items (rows + stored elements) per wave
constexpr int kSpmmSegment = 128;

inline int status_of(hipError_t e)
{
    switch (e) {
    case hipSuccess: return ASX_STATUS_SUCCESS;
    case hipErrorOutOfMemory: return ASX_STATUS_ALLOC_FAILED;
    case hipErrorInvalidValue: return ASX_STATUS_INVALID_VALUE;
    case hipErrorInvalidDevicePointer: return ASX_STATUS_INVALID_POINTER;
    case hipErrorInvalidDevice:
    case hipErrorInvalidResourceHandle: return ASX_STATUS_INVALID_HANDLE;
    default: return ASX_STATUS_INTERNAL_ERROR;
    }
}
inline int check_launch() { return status_of(hipGetLastError()); }

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// ---- analysis launchers (asx_analysis.hip) ----
int launch_row_histogram(const int32_t *d_row_ptr, int32_t m, int64_t *d_hist, int64_t *d_stats,
                         hipStream_t s);
int launch_partition_rows_by_nnz(const int32_t *d_row_ptr, int32_t m, int32_t nparts, int32_t *d_out,
                                 hipStream_t s);
int launch_nnz_split_rows(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t items,
                          int32_t *d_out, hipStream_t s);
int launch_nnz_split_rows_n(const int32_t *d_row_ptr, int32_t m, int32_t nseg, int32_t items, int32_t *d_out,
                            hipStream_t s);
int launch_flat_seg_rows(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t *d_seg_row, hipStream_t s);
int launch_merge_path_search(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t items,
                             int32_t *d_xs, int32_t *d_ys, hipStream_t s);
int launch_loadbalance_partition(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t warp_size,
                                 int32_t nwarps, int32_t *d_out, hipStream_t s);
int launch_stream_row_blocks(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t *d_blocks,
                             hipStream_t s);
int launch_copy_bytes(const void *d_src, void *d_dst, size_t bytes, hipStream_t s);
int launch_fill_i32(int32_t *d_dst, int64_t n, int32_t value, hipStream_t s);
// d_now[0..1] = two 64-bit checksums of `bytes` bytes (a multiple of 4, from a 16-byte boundary);
// d_partials: 2 * checksum_parts() words of scratch
int checksum_parts();
int launch_checksum(const void *d_data, size_t bytes, unsigned long long *d_partials, unsigned long long *d_now, hipStream_t s);
// kept = now
int launch_checksum_commit(const unsigned long long *d_now, unsigned long long *d_kept, hipStream_t s);
int launch_sample_columns(const int32_t *d_col, int64_t stride, int shift, const int32_t *d_row_ptr, int32_t m,
                          int32_t width, int32_t samples, int32_t *d_out, hipStream_t s);
int launch_gather_lines(const void *d_buf, size_t bytes, int group_lanes, int per_lane, void *d_out, int *nthreads,
                        hipStream_t s);

// ---- SpMV launchers (asx_spmv.hip) ----
template <typename T>
int launch_spmv_vector(int32_t m, int32_t nnz, T alpha, const int32_t *row_ptr, const int32_t *col,
                       const T *val, const T *x, T beta, T *y, hipStream_t s);
template <typename T>
int launch_spmv_merge(int32_t m, int32_t nnz, T alpha, const int32_t *row_ptr, const int32_t *col,
                      const T *val, const T *x, T beta, T *y, const int32_t *xs, const int32_t *ys,
                      T *carry, hipStream_t s);
template <typename T>
int launch_spmv_stream(int32_t m, int32_t nnz, T alpha, const int32_t *row_ptr, const int32_t *col,
                       const T *val, const T *x, T beta, T *y, const int32_t *blocks, hipStream_t s);

template <typename T>
int launch_spmv_flat(int32_t m, int32_t nnz, T alpha, const int32_t *row_ptr, const int32_t *col,
                     const T *val, const T *x, T beta, T *y, const int32_t *seg_row, T *carry,
                     bool carry_pass, hipStream_t s);
int launch_flat_has_carry(const int32_t *d_row_ptr, int32_t m, int32_t nnz, const int32_t *d_seg_row,
                          int32_t *d_flag, hipStream_t s);

// ---- SpMM launchers (asx_spmm.hip) ----
template <typename T>
int launch_spmm_row(int32_t m, int32_t ncols, T alpha, const int32_t *row_ptr, const int32_t *col,
                    const T *val, const T *B, int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t s);
template <typename T>
int launch_spmm_merge(int32_t m, int32_t nnz, int32_t ncols, T alpha, const int32_t *row_ptr,
                      const int32_t *col, const T *val, const T *B, int64_t ldb, T beta, T *C,
                      int64_t ldc, const int32_t *xs, const int32_t *ys, T *carry, int32_t *carry_row,
                      hipStream_t s);

// merge-path split points of SpMM moved to the ends of the short rows they cut (out of place)
int launch_spmm_snap_splits(int32_t m, int32_t nnz, const int32_t *row_ptr, const int32_t *xs, const int32_t *ys,
                            int32_t *xs_out, int32_t *ys_out, hipStream_t s);

// ---- blocked (MFMA) SpMM (asx_blocked.hip) ----
struct BlockedMatrix {
    int32_t nbrows;     // ceil(m / 16)
    int32_t nblocks;    // non-empty 16x4 blocks
    int32_t *brow_ptr;  // nbrows + 1
    int32_t *bcol;      // column quad of each block
    void *bval;         // nblocks * 64 values, lane order of the MFMA A operand
    int32_t nnz;        // stored elements of A
    int32_t *upd_src;   // nnz: position in A's values of every stored element, in block order
    int64_t *upd_dst;   // nnz: its slot in bval; sign bit = repeats the (row, column) before it
};
template <typename T>
int build_blocked(int32_t m, int32_t k, int32_t nnz, const int32_t *row_ptr, const int32_t *col,
                  const T *val, BlockedMatrix *out, hipStream_t s);
void free_blocked(BlockedMatrix *b);
template <typename T>
int blocked_update_values(const BlockedMatrix *bm, const T *val, hipStream_t s);
template <typename T>
int launch_spmm_blocked(int32_t m, int32_t k, int32_t ncols, T alpha, const BlockedMatrix *bm, const T *B,
                        int64_t ldb, T beta, T *C, int64_t ldc, hipStream_t s);

constexpr int kXcds = 8;  // workgroups are dealt to the 8 XCDs round-robin (workgroup b runs on XCD b % 8)
// out[r] = first i with sorted[i] >= r, r in [0, n]
int launch_offsets_from_sorted(const int32_t *sorted, int32_t count, int32_t n, int32_t *out, hipStream_t s);

// ---- column-sliced SpMV (asx_sliced.hip) ----
// The stored elements regrouped by column slice (slice = col / width), a slice of x being small
// enough to sit in the LDS of one compute unit, so that the gathers of x never reach the L2.
// Pass 1: one workgroup per (slice, range of tiles) loads the slice of x into LDS and streams
// the slice's stored elements, kSlicedTile per wave and step, in row order; it writes one partial
// sum per run of elements of the same row (a run is also cut at every tile start, so tiles are
// independent).  Pass 2: one wave per block of `rows_per_wave` rows of A adds the partial sums of
// its rows, slice after slice, into LDS accumulators and writes y.  The partial sums of one row
// block inside one slice are a contiguous range (`chunk_lo`).
constexpr int kSlicedTile = 256;  // stored elements per wave and step: 4 per lane
constexpr int kSlicedMaxSlices = 1024;  // the plan build ranks stored elements by slice in LDS
struct SlicedMatrix {
    int32_t width;          // columns per slice
    int32_t nslices;
    int32_t ntiles;         // all slices; every slice starts a new tile and is padded to whole tiles
    int32_t npartials;      // partial sums written per call
    int32_t nwg;            // workgroups of pass 1
    int32_t npieces;        // what they work off: runs of tiles inside one slice
    int32_t rows_per_wave;  // pass 2
    int32_t nrb;            // ceil(m / rows_per_wave)
    void *store;            // one allocation: val, perm, cf, tile_base, wg_tab, chunk_lo, pstep_ptr
    void *val;              // ntiles * kSlicedTile values (a copy of A's, in slice order; pads are 0)
    void *partial;          // npartials + kSlicedReducePad values: the partial sums of one call, for callers
                            // that bring no buffer of their own (null once released)
    uint16_t *cf;           // ntiles * kSlicedTile: column inside the slice, bit 15 = first element of a run
    int32_t *perm;          // where each stored copy comes from in A's val (-1 for pads)
    int32_t *tile_base;     // ntiles + 1: index of the first partial sum of each tile
    int32_t *wg_tab;        // npieces x 4: slice, first tile, end tile, 0
    int32_t nnz, nsort_blocks;  // stored elements; blocks of 4096 of them, as the build sorted them
    uint16_t *pos;          // nnz: position of each stored element among its block's elements in slice order
    int32_t *block_base;    // (nsort_blocks + 1) x nslices: slot of a block's first element of each slice (last row: the slices' ends)
    int32_t *wg_pieces;     // nwg x 8: first piece, end piece of each workgroup, 0, 0, then the first piece's four
                            // words again (behind wg_tab in the store)
    uint16_t *prow;         // npartials + kSlicedReducePad: row of each partial sum inside its row block
    int32_t *chunk_lo;      // (nrb + 1) x nslices: first partial sum of row block b in slice s
    int32_t npsteps;        // steps of pass 2, all row blocks
    int32_t *pstep_ptr;     // nrb + 1: first step of each row block
    int32_t *psteps;        // npsteps (+ kSlicedStepPad) x 4: up to 64 partial sums from up to 3 pieces of ranges
};
constexpr int kSlicedStepPad = 64;     // readable step descriptors past the last one
constexpr int kSlicedReducePad = 256;  // entries of prow / partial that pass 2 may read past the last partial sum
template <typename T>
int build_sliced(int32_t m, int32_t n, int32_t nnz, int32_t width, int32_t rows_per_wave, int32_t target_wgs,
                 const int32_t *row_ptr, const int32_t *col, const T *val, SlicedMatrix *out, hipStream_t s);
void free_sliced(SlicedMatrix *p);
template <typename T>
int sliced_update_values(const SlicedMatrix *sm, const T *val, hipStream_t s, const unsigned long long *unless_equal = nullptr);
template <typename T>
int launch_spmv_sliced(int32_t m, int32_t n, T alpha, const SlicedMatrix *sm, const T *x, T beta, T *y, T *partial,
                       hipStream_t s);
inline size_t sliced_scratch_bytes(const SlicedMatrix *sm, size_t sv) { return ((size_t)sm->npartials + kSlicedReducePad) * sv; }

// ---- row blocks with sliding windows of x in LDS (asx_window.hip) ----
// Blocks of `rows_per_block` consecutive rows whose columns all lie inside at most kWindowBands
// bands that together span fewer than 16384 columns, chained: a workgroup walks a chain of blocks
// with a ring in LDS per band and fetches, per block, only the columns that are new.  The stored
// elements stream as tiles (16-bit LDS slot + row-start flag, as the sliced kernel's); every row
// owns at least one slot, so a tile's runs are consecutive rows and go straight to y.
constexpr int kWindowBands = 4;
struct WindowMatrix {
    int32_t rows_per_block;
    int32_t nblocks;
    int32_t nchains;         // workgroups
    int32_t npieces;         // entries of `pieces`
    int32_t ntiles;
    int32_t nbands;          // 1: one window per block; 2..kWindowBands: bands of diagonals
    int32_t stack_rows;      // > 0: three bands on stacked planes of this many rows, the blocks stored column by column
    int has_carry;           // some tile starts inside a row: the ordered carry pass is needed
    int by_reference;        // every row holds two stored elements or more: the stored elements of a tile are consecutive in
                             // A's val, which the kernel reads in place (no val, no perm)
    void *store;             // one allocation: val, perm (unless by_reference), cf, tile_info
    void *tables;            // one allocation: blocks, pieces, chains
    void *val;               // ntiles * kSlicedTile values (a copy of A's; pads are 0)
    void *carry;             // ntiles values: the carries of one call, for callers that bring no buffer (null once released)
    uint16_t *cf;            // ntiles * kSlicedTile: LDS slot of the column, bit 15 = first slot of a row (or tile)
    int32_t *perm;           // where each stored copy comes from in A's val (-1 for pads)
    int32_t *tile_info;      // ntiles x 4: row of the tile's first slot (bit 31: the tile starts inside it), rows in the tile,
                             // by_reference: index of the tile's first stored element in A's val, stored elements in the tile
    int32_t *blocks;         // nblocks x 4: first tile, end tile, first piece, end piece
    int32_t *pieces;         // x 4: columns of x to fetch before a block (from, to), first LDS slot and size of their ring
    int32_t *chains;         // nchains x 2: first block, end block
};
// in_place: where no row holds fewer than two stored elements, keep no copy of the values and read A's in every call
template <typename T>
int build_window(int32_t m, int32_t n, int32_t nnz, int32_t target_wgs, bool in_place, const int32_t *row_ptr,
                 const int32_t *col, const T *val, WindowMatrix *out, hipStream_t s);
void free_window(WindowMatrix *p);
template <typename T>
int window_update_values(const WindowMatrix *wm, const T *val, hipStream_t s, const unsigned long long *unless_equal = nullptr);
template <typename T>
int launch_spmv_window(int32_t m, int32_t n, T alpha, const WindowMatrix *wm, const T *val, const T *x, T beta, T *y, T *carry,
                       hipStream_t s);
inline size_t window_scratch_bytes(const WindowMatrix *wm, size_t sv) { return wm->has_carry ? (size_t)wm->ntiles * sv : 0; }

inline int32_t merge_tiles(int32_t m, int32_t nnz) { return (int32_t)ceil_div64((int64_t)m + nnz, kMergeTile); }
inline int32_t flat_tiles(int32_t nnz) { int32_t t = (int32_t)ceil_div64(nnz, kFlatTile); return t < 1 ? 1 : t; }
inline int32_t stream_blocks(int32_t nnz) { return (int32_t)ceil_div64(nnz, kStreamTile); }
inline int32_t spmm_segments(int32_t m, int32_t nnz) { return (int32_t)ceil_div64((int64_t)m + nnz, kSpmmSegment); }

}  // namespace asx

constexpr int kPlanCounters = 128;
// Plan: analysis results kept on the device across calls.
struct asx_plan {
    int is_spmm;
    int alg;  // resolved kernel
    int value_type;
    int32_t m, n, nnz, ncols;
    const int32_t *row_ptr;  // the device array the plan was built from (identity check only)
    int64_t *d_counters;     // kPlanCounters words on the device: histogram (33), stats (4), a flag (40), checksums of the values:
                             // of this call (44, 45) and of the copy the plan holds (46, 47), 64 sample counts (64..95)
    int checked;             // the plan holds a copy of A's values and a checksum of them (asx_spmv_plan_create_checked)
    unsigned long long *d_checksum_parts;  // checked plans: the workgroups' partial sums of one checksum run
    int32_t *d_meta;         // split points / row blocks (layout depends on alg)
    size_t meta_bytes;
    int32_t nunits;  // tiles / row blocks / segments
    int carry_pass;  // flat kernel: 0 when no row is cut by a tile boundary
    int64_t hist[33];
    int64_t stats[4];
    size_t workspace_bytes;
    asx::BlockedMatrix blocked;  // only for ASX_SPMM_BLOCKED plans
    asx::SlicedMatrix sliced;    // only for ASX_SPMV_SLICED plans
    asx::WindowMatrix window;    // only for ASX_SPMV_WINDOW plans
};
