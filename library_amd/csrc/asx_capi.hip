// extern "C" entry points of libalphasparse_amd.so: argument checks, workspace layout, plans,
// kernel selection.  No arithmetic lives here.  There is no CPU fallback: every compute entry
// point launches HIP kernels or returns an error status.
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "../../include/alphasparse_amd_bench.h"
#include "asx_internal.hpp"

using namespace asx;

namespace {

constexpr size_t kAlign = 256;

size_t vsize(int value_type) { return value_type == ASX_R_64F ? 8 : 4; }

struct MergeLayout {  // [xs | ys | carry] inside a workspace
    size_t xs_off, ys_off, carry_off, bytes;
};
MergeLayout spmv_merge_layout(int32_t m, int32_t nnz, size_t sv, bool with_split)
{
    MergeLayout L{};
    const size_t nt = (size_t)merge_tiles(m, nnz);
    size_t off = 0;
    if (with_split) {
        L.xs_off = off;
        off = align_up(off + (nt + 1) * 4, kAlign);
        L.ys_off = off;
        off = align_up(off + (nt + 1) * 4, kAlign);
    }
    L.carry_off = off;
    off = align_up(off + std::max<size_t>(nt, 1) * sv, kAlign);
    L.bytes = off;
    return L;
}

struct FlatLayout {  // [seg_row | carry]
    size_t seg_off, carry_off, bytes;
};
FlatLayout spmv_flat_layout(int32_t nnz, size_t sv, bool with_split)
{
    FlatLayout L{};
    const size_t nt = (size_t)flat_tiles(nnz);
    size_t off = 0;
    if (with_split) {
        L.seg_off = off;
        off = align_up(off + (nt + 1) * 4, kAlign);
    }
    L.carry_off = off;
    off = align_up(off + nt * sv, kAlign);
    L.bytes = off;
    return L;
}

struct SpmmLayout {  // [raw xs | raw ys | xs | ys | carry_row | carry]
    size_t raw_xs_off, raw_ys_off, xs_off, ys_off, crow_off, carry_off, bytes;
};
SpmmLayout spmm_merge_layout(int32_t m, int32_t nnz, int32_t ncols, size_t sv, bool with_split)
{
    SpmmLayout L{};
    const size_t ns = (size_t)spmm_segments(m, nnz);
    size_t off = 0;
    if (with_split) {
        for (size_t *o : {&L.raw_xs_off, &L.raw_ys_off, &L.xs_off, &L.ys_off}) {
            *o = off;
            off = align_up(off + (ns + 1) * 4, kAlign);
        }
    }
    L.crow_off = off;
    off = align_up(off + std::max<size_t>(ns, 1) * 4, kAlign);
    L.carry_off = off;
    off = align_up(off + std::max<size_t>(ns, 1) * (size_t)ncols * sv, kAlign);
    L.bytes = off;
    return L;
}

// What a sample of the columns says (up to 64 tiles of 1024 consecutive stored elements spread over
// the matrix, counted on the device):
//   spread  distinct 128-byte lines of x a tile's columns touch, per stored element.  Random
//           columns give about 1, a 5-point stencil 0.04, a band matrix 0.01.
//   pairs   (row, slice) pairs per stored element, for column slices of 128 KiB of x: the partial
//           sums the column-sliced kernel would carry through memory.  16 random columns per row
//           over 32 slices give 0.8, a band matrix about 1 / (row length).
struct ColumnSample {
    bool ok;
    double spread, pairs;
};
constexpr int32_t kSliceBytes = 131072;  // of x per slice: one workgroup of 16 waves per compute unit
ColumnSample sample_columns(const int32_t *d_row_ptr, int32_t m, const int32_t *d_col, int32_t nnz, size_t sv,
                            int32_t *d_scratch /* 128 ints */, hipStream_t s)
{
    ColumnSample cs{false, 0.0, 1.0};
    const int64_t tiles = nnz / kFlatTile;
    if (tiles < 1) return cs;
    const int samples = (int)std::min<int64_t>(64, tiles);
    const int64_t stride = tiles / samples;
    int32_t h[128];
    const int shift = sv == 8 ? 4 : 5;  // columns per 128-byte line of x
    if (launch_sample_columns(d_col, stride * kFlatTile, shift, d_row_ptr, m, (int32_t)(kSliceBytes / sv), samples, d_scratch,
                              s) != ASX_STATUS_SUCCESS ||
        hipMemcpyAsync(h, d_scratch, sizeof(h), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess)
        return cs;
    int64_t distinct = 0, pairs = 0;
    for (int t = 0; t < samples; ++t) distinct += h[t], pairs += h[64 + t];
    cs.ok = true;
    cs.spread = (double)distinct / ((double)samples * kFlatTile);
    cs.pairs = d_row_ptr ? (double)pairs / ((double)samples * kFlatTile) : 1.0;
    return cs;
}
constexpr double kScatteredMinSpread = 0.5;

constexpr int32_t kSmallNnz = 1 << 18;
constexpr int64_t kSmallMaxRow = 2048;

// DEFAULT with a plan: the flat kernel, except for matrices with very long rows, where the
// merge-path kernel measured about 1 % faster (power-law: 569 vs 576 us).  Elsewhere flat is the
// fastest of the four or within 1 % of it (5-point stencil 300 us vs stream 305; uniform 16/row
// 95 vs stream 96), and it has no bad case: work per tile is bounded whatever the row lengths.
// Matrices small enough to be bound by launch overhead take the vector kernel, the only one that
// is a single launch with no metadata (1280 x 1280 banded: 13.4 us against 16.2 us).
// Mostly-empty matrices (more than half of the rows hold nothing) take the merge-path kernel,
// which counts row ends as work: a flat tile next to a long run of empty rows has to write all
// of them itself.
int choose_spmv_from_stats(const int64_t hist[33], const int64_t stats[4], int32_t m, int32_t nnz)
{
    if (nnz <= kSmallNnz && stats[0] <= kSmallMaxRow && m <= kSmallNnz) return ASX_SPMV_VECTOR;
    if (stats[0] > kLongRow || hist[0] > (int64_t)m / 2) return ASX_SPMV_MERGE;
    return ASX_SPMV_FLAT;
}

template <typename T>
int spmv_impl(const asx_plan *plan, int alg, int32_t m, int32_t n, int32_t nnz, T alpha,
              const int32_t *row_ptr, const int32_t *col, const T *val, const T *x, T beta, T *y,
              void *ws, size_t ws_bytes, hipStream_t s)
{
    if (m < 0 || n < 0 || nnz < 0) return ASX_STATUS_INVALID_SIZE;
    if (m == 0) return ASX_STATUS_SUCCESS;
    if (!row_ptr || !y || (nnz > 0 && (!col || !val || !x))) return ASX_STATUS_INVALID_POINTER;
    const int vt = sizeof(T) == 8 ? ASX_R_64F : ASX_R_32F;
    int kernel;
    if (plan) {
        if (plan->is_spmm || plan->m != m || plan->nnz != nnz || plan->value_type != vt)
            return ASX_STATUS_INVALID_VALUE;
        kernel = plan->alg;
    } else {
        kernel = asx_spmv_resolve_alg(alg, m, nnz);
        if (kernel < 0) return ASX_STATUS_NOT_SUPPORTED;
    }
    char *w = (char *)ws;
    switch (kernel) {
    case ASX_SPMV_VECTOR:
        return launch_spmv_vector<T>(m, nnz, alpha, row_ptr, col, val, x, beta, y, s);
    case ASX_SPMV_STREAM: {
        const int32_t *blocks;
        if (plan) {
            blocks = plan->d_meta;
        } else {
            const size_t need = asx_spmv_workspace_bytes(kernel, vt, m, nnz);
            if (!ws) return ASX_STATUS_INVALID_POINTER;
            if (ws_bytes < need) return ASX_STATUS_INVALID_SIZE;
            int st = launch_stream_row_blocks(row_ptr, m, nnz, (int32_t *)w, s);
            if (st) return st;
            blocks = (const int32_t *)w;
        }
        return launch_spmv_stream<T>(m, nnz, alpha, row_ptr, col, val, x, beta, y, blocks, s);
    }
    case ASX_SPMV_MERGE: {
        const MergeLayout L = spmv_merge_layout(m, nnz, sizeof(T), plan == nullptr);
        if (!ws) return ASX_STATUS_INVALID_POINTER;
        if (ws_bytes < L.bytes) return ASX_STATUS_INVALID_SIZE;
        const int32_t *xs, *ys;
        if (plan) {
            const size_t nt = (size_t)merge_tiles(m, nnz);
            xs = plan->d_meta;
            ys = plan->d_meta + (nt + 1);
        } else {
            int st = launch_merge_path_search(row_ptr, m, nnz, kMergeTile, (int32_t *)(w + L.xs_off),
                                              (int32_t *)(w + L.ys_off), s);
            if (st) return st;
            xs = (const int32_t *)(w + L.xs_off);
            ys = (const int32_t *)(w + L.ys_off);
        }
        return launch_spmv_merge<T>(m, nnz, alpha, row_ptr, col, val, x, beta, y, xs, ys,
                                    (T *)(w + L.carry_off), s);
    }
    case ASX_SPMV_FLAT: {
        const FlatLayout L = spmv_flat_layout(nnz, sizeof(T), plan == nullptr);
        if (!ws) return ASX_STATUS_INVALID_POINTER;
        if (ws_bytes < L.bytes) return ASX_STATUS_INVALID_SIZE;
        const int32_t *seg;
        if (plan) {
            seg = plan->d_meta;
        } else {
            int st = launch_flat_seg_rows(row_ptr, m, nnz, (int32_t *)(w + L.seg_off), s);
            if (st) return st;
            seg = (const int32_t *)(w + L.seg_off);
        }
        return launch_spmv_flat<T>(m, nnz, alpha, row_ptr, col, val, x, beta, y, seg, (T *)(w + L.carry_off),
                                   plan ? plan->carry_pass != 0 : true, s);
    }
    case ASX_SPMV_SLICED: {
        // the slices hold a copy of A's columns and values and are built by asx_spmv_plan_create.
        // The partial sums of the call go into the caller's workspace when it is large enough, else
        // into the plan's own buffer (which calls that overlap would share)
        if (!plan || !plan->sliced.cf) return ASX_STATUS_NOT_INITIALIZED;
        if (plan->n != n) return ASX_STATUS_INVALID_VALUE;
        const size_t need = sliced_scratch_bytes(&plan->sliced, sizeof(T));
        T *scratch = ws && ws_bytes >= need ? (T *)ws : (T *)plan->sliced.partial;
        if (!scratch) return ws ? ASX_STATUS_INVALID_SIZE : ASX_STATUS_INVALID_POINTER;
        return launch_spmv_sliced<T>(m, n, alpha, &plan->sliced, x, beta, y, scratch, s);
    }
    case ASX_SPMV_WINDOW: {
        // the row blocks hold a copy of A's columns (and of its values, unless they can be read in
        // place) and are built by asx_spmv_plan_create; the carries of the call (plans with cut rows
        // only) go where the sliced kernel's partial sums go
        if (!plan || !plan->window.cf) return ASX_STATUS_NOT_INITIALIZED;
        if (plan->n != n) return ASX_STATUS_INVALID_VALUE;
        const size_t need = window_scratch_bytes(&plan->window, sizeof(T));
        T *scratch = ws && ws_bytes >= need ? (T *)ws : (T *)plan->window.carry;
        if (need && !scratch) return ws ? ASX_STATUS_INVALID_SIZE : ASX_STATUS_INVALID_POINTER;
        return launch_spmv_window<T>(m, n, alpha, &plan->window, val, x, beta, y, scratch, s);
    }
    default: return ASX_STATUS_NOT_SUPPORTED;
    }
}

template <typename T>
int spmm_impl(const asx_plan *plan, int alg, int32_t m, int32_t k, int32_t nnz, int32_t ncols, T alpha,
              const int32_t *row_ptr, const int32_t *col, const T *val, const T *B, int64_t ldb, T beta,
              T *C, int64_t ldc, void *ws, size_t ws_bytes, hipStream_t s)
{
    if (m < 0 || k < 0 || nnz < 0 || ncols < 0) return ASX_STATUS_INVALID_SIZE;
    if (m == 0 || ncols == 0) return ASX_STATUS_SUCCESS;
    if (ldb < ncols || ldc < ncols) return ASX_STATUS_INVALID_SIZE;
    if (!row_ptr || !C || (nnz > 0 && (!col || !val || !B))) return ASX_STATUS_INVALID_POINTER;
    const int vt = sizeof(T) == 8 ? ASX_R_64F : ASX_R_32F;
    int kernel;
    if (plan) {
        if (!plan->is_spmm || plan->m != m || plan->nnz != nnz || plan->value_type != vt ||
            plan->ncols != ncols)
            return ASX_STATUS_INVALID_VALUE;
        kernel = plan->alg;
    } else {
        kernel = asx_spmm_resolve_alg(alg, m, nnz, ncols);
        if (kernel < 0) return ASX_STATUS_NOT_SUPPORTED;
    }
    char *w = (char *)ws;
    switch (kernel) {
    case ASX_SPMM_ROW:
        return launch_spmm_row<T>(m, ncols, alpha, row_ptr, col, val, B, ldb, beta, C, ldc, s);
    case ASX_SPMM_MERGE: {
        const SpmmLayout L = spmm_merge_layout(m, nnz, ncols, sizeof(T), plan == nullptr);
        if (!ws) return ASX_STATUS_INVALID_POINTER;
        if (ws_bytes < L.bytes) return ASX_STATUS_INVALID_SIZE;
        const int32_t *xs, *ys;
        if (plan) {
            const size_t ns = (size_t)spmm_segments(m, nnz);
            xs = plan->d_meta;
            ys = plan->d_meta + (ns + 1);
        } else {
            int st = launch_merge_path_search(row_ptr, m, nnz, kSpmmSegment, (int32_t *)(w + L.raw_xs_off),
                                              (int32_t *)(w + L.raw_ys_off), s);
            if (!st)
                st = launch_spmm_snap_splits(m, nnz, row_ptr, (const int32_t *)(w + L.raw_xs_off),
                                             (const int32_t *)(w + L.raw_ys_off), (int32_t *)(w + L.xs_off),
                                             (int32_t *)(w + L.ys_off), s);
            if (st) return st;
            xs = (const int32_t *)(w + L.xs_off);
            ys = (const int32_t *)(w + L.ys_off);
        }
        return launch_spmm_merge<T>(m, nnz, ncols, alpha, row_ptr, col, val, B, ldb, beta, C, ldc, xs,
                                    ys, (T *)(w + L.carry_off), (int32_t *)(w + L.crow_off), s);
    }
    case ASX_SPMM_BLOCKED:
        // the blocks hold a copy of A's values and are built by asx_spmm_plan_create
        if (!plan || !plan->blocked.brow_ptr) return ASX_STATUS_NOT_INITIALIZED;
        return launch_spmm_blocked<T>(m, k, ncols, alpha, &plan->blocked, B, ldb, beta, C, ldc, s);
    default: return ASX_STATUS_NOT_SUPPORTED;
    }
}

}  // namespace

static int noalloc_scratch(void **out);

extern "C" {

const char *asx_version(void) { return "0.1"; }

int asx_device_info(int *compute_units, int *wavefront_size)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return status_of(e);
    int cu = 0, wf = 0;
    e = hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return status_of(e);
    e = hipDeviceGetAttribute(&wf, hipDeviceAttributeWarpSize, dev);
    if (e != hipSuccess) return status_of(e);
    if (compute_units) *compute_units = cu;
    if (wavefront_size) *wavefront_size = wf;
    // the address of this device's scratch array of asx_spmv_csr_f64_noalloc, so that its calls are
    // stream work only from the first one on (the lookup may load the library's code onto the device)
    void *unused = nullptr;
    (void)noalloc_scratch(&unused);
    return ASX_STATUS_SUCCESS;
}

// ---------------------------------------------------------------- analysis
int asx_row_length_histogram(const int32_t *d_row_ptr, int32_t m, int64_t *d_hist, int64_t *d_stats,
                             void *stream)
{
    if (m < 0) return ASX_STATUS_INVALID_SIZE;
    if (!d_hist || !d_stats || (m > 0 && !d_row_ptr)) return ASX_STATUS_INVALID_POINTER;
    return launch_row_histogram(d_row_ptr, m, d_hist, d_stats, (hipStream_t)stream);
}

int asx_partition_rows_by_nnz(const int32_t *d_row_ptr, int32_t m, int32_t nparts, int32_t *d_partition,
                              void *stream)
{
    if (m < 1 || nparts < 1) return ASX_STATUS_INVALID_SIZE;
    if (!d_row_ptr || !d_partition) return ASX_STATUS_INVALID_POINTER;
    return launch_partition_rows_by_nnz(d_row_ptr, m, nparts, d_partition, (hipStream_t)stream);
}

int asx_nnz_split_rows(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t items, int32_t *d_out,
                       void *stream)
{
    if (m < 0 || nnz < 0 || items < 1) return ASX_STATUS_INVALID_SIZE;
    if (!d_row_ptr || !d_out) return ASX_STATUS_INVALID_POINTER;
    return launch_nnz_split_rows(d_row_ptr, m, nnz, items, d_out, (hipStream_t)stream);
}

int asx_merge_path_search(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t items, int32_t *d_xs,
                          int32_t *d_ys, void *stream)
{
    if (m < 0 || nnz < 0 || items < 1) return ASX_STATUS_INVALID_SIZE;
    if (!d_row_ptr || !d_xs || !d_ys) return ASX_STATUS_INVALID_POINTER;
    return launch_merge_path_search(d_row_ptr, m, nnz, items, d_xs, d_ys, (hipStream_t)stream);
}

int64_t asx_loadbalance_nwarps(int64_t nnz, int64_t warp_size, int64_t nwarps_base)
{
    if (warp_size <= 0) return 0;
    int64_t mult = 8;
    if (nnz >= (int64_t)2e8)
        mult = 2048;
    else if (nnz >= (int64_t)2e7)
        mult = 512;
    else if (nnz >= (int64_t)2e6)
        mult = 128;
    else if (nnz >= (int64_t)2e5)
        mult = 32;
    return std::min(ceil_div64(nnz, warp_size), nwarps_base * mult);
}

int asx_loadbalance_partition(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t warp_size,
                              int32_t nwarps, int32_t *d_out, void *stream)
{
    if (m < 1 || nnz < 0 || warp_size < 1 || nwarps < 0) return ASX_STATUS_INVALID_SIZE;
    if (!d_row_ptr || (nwarps > 0 && !d_out)) return ASX_STATUS_INVALID_POINTER;
    return launch_loadbalance_partition(d_row_ptr, m, nnz, warp_size, nwarps, d_out,
                                        (hipStream_t)stream);
}

// ---------------------------------------------------------------- plans
}  // extern "C"

namespace {

// A plan with sizes and the row-length histogram, no kernel chosen yet.  The counters on the device
// stay with the plan (33 histogram bins, 4 stats, spare words for what else the build reads back):
// freeing them here would cost more than the build's kernels.
int plan_begin(asx_plan **out, int is_spmm, int value_type, int32_t m, int32_t n, int32_t nnz, const int32_t *d_row_ptr,
               int32_t ncols_dense, hipStream_t s)
{
    asx_plan *p = new (std::nothrow) asx_plan();
    if (!p) return ASX_STATUS_ALLOC_FAILED;
    std::memset(p, 0, sizeof(*p));
    p->is_spmm = is_spmm ? 1 : 0;
    p->alg = -1;
    p->value_type = value_type;
    p->m = m;
    p->n = n;
    p->nnz = nnz;
    p->ncols = is_spmm ? ncols_dense : 1;
    p->row_ptr = d_row_ptr;
    int st = status_of(hipMalloc((void **)&p->d_counters, kPlanCounters * sizeof(int64_t)));
    if (!st) st = launch_row_histogram(d_row_ptr, m, p->d_counters, p->d_counters + 33, s);
    if (!st) st = status_of(hipMemcpyAsync(p->hist, p->d_counters, 33 * sizeof(int64_t), hipMemcpyDeviceToHost, s));
    if (!st) st = status_of(hipMemcpyAsync(p->stats, p->d_counters + 33, 4 * sizeof(int64_t), hipMemcpyDeviceToHost, s));
    if (!st) st = status_of(hipStreamSynchronize(s));
    if (st) {
        asx_plan_destroy(p);
        return st;
    }
    *out = p;
    return ASX_STATUS_SUCCESS;
}

// Split points of a row-ordered kernel onto a plan from plan_begin.
int plan_row_ordered(asx_plan *p, int kernel, hipStream_t s)
{
    const int32_t m = p->m, nnz = p->nnz;
    const int32_t *d_row_ptr = p->row_ptr;
    const size_t sv = vsize(p->value_type);
    int st = ASX_STATUS_SUCCESS;
    p->alg = kernel;
    p->workspace_bytes = 0;
    if (m == 0) return ASX_STATUS_SUCCESS;  // nothing to analyse: calls with m == 0 return before any launch
    if (!p->is_spmm) {
        if (kernel == ASX_SPMV_STREAM) {
            int32_t nb = std::max(stream_blocks(nnz), 1);
            p->nunits = nb;
            p->meta_bytes = ((size_t)nb + 1) * 8;
            st = status_of(hipMalloc((void **)&p->d_meta, p->meta_bytes));
            if (!st) st = launch_stream_row_blocks(d_row_ptr, m, nnz, p->d_meta, s);
        } else if (kernel == ASX_SPMV_FLAT) {
            const size_t nt = (size_t)flat_tiles(nnz);
            p->nunits = (int32_t)nt;
            p->meta_bytes = (nt + 1) * 4;
            st = status_of(hipMalloc((void **)&p->d_meta, p->meta_bytes));
            if (!st) st = launch_flat_seg_rows(d_row_ptr, m, nnz, p->d_meta, s);
            p->workspace_bytes = spmv_flat_layout(nnz, sv, false).bytes;
            p->carry_pass = 1;
            if (!st) {  // is any row cut by a tile boundary?  (one int read back; creation syncs anyway)
                int32_t *d_flag = reinterpret_cast<int32_t *>(p->d_counters + 40), h_flag = 1;
                st = launch_fill_i32(d_flag, 1, 0, s);
                if (!st) st = launch_flat_has_carry(d_row_ptr, m, nnz, p->d_meta, d_flag, s);
                if (!st) st = status_of(hipMemcpyAsync(&h_flag, d_flag, sizeof(int32_t), hipMemcpyDeviceToHost, s));
                if (!st) st = status_of(hipStreamSynchronize(s));
                if (!st) p->carry_pass = h_flag != 0;
            }
        } else if (kernel == ASX_SPMV_MERGE) {
            const size_t nt = (size_t)merge_tiles(m, nnz);
            p->nunits = (int32_t)nt;
            p->meta_bytes = 2 * (nt + 1) * 4;
            st = status_of(hipMalloc((void **)&p->d_meta, p->meta_bytes));
            if (!st) st = launch_merge_path_search(d_row_ptr, m, nnz, kMergeTile, p->d_meta, p->d_meta + (nt + 1), s);
            p->workspace_bytes = spmv_merge_layout(m, nnz, sv, false).bytes;
        }
    } else if (kernel == ASX_SPMM_MERGE) {
        const size_t ns = (size_t)spmm_segments(m, nnz);
        p->nunits = (int32_t)ns;
        p->meta_bytes = 2 * (ns + 1) * 4;
        int32_t *raw = nullptr;  // the merge-path points, then snapped to short-row ends
        st = status_of(hipMalloc((void **)&p->d_meta, p->meta_bytes));
        if (!st) st = status_of(hipMalloc((void **)&raw, p->meta_bytes));
        if (!st) st = launch_merge_path_search(d_row_ptr, m, nnz, kSpmmSegment, raw, raw + (ns + 1), s);
        if (!st) st = launch_spmm_snap_splits(m, nnz, d_row_ptr, raw, raw + (ns + 1), p->d_meta, p->d_meta + (ns + 1), s);
        if (!st) st = status_of(hipStreamSynchronize(s));
        if (raw) (void)hipFree(raw);
        p->workspace_bytes = spmm_merge_layout(m, nnz, p->ncols, sv, false).bytes;
    }
    if (!st) st = status_of(hipStreamSynchronize(s));
    return st;
}

}  // namespace

extern "C" {

int asx_plan_create(asx_plan **out, int is_spmm, int alg, int value_type, int32_t m, int32_t n,
                    int32_t nnz, const int32_t *d_row_ptr, int32_t ncols_dense, void *stream)
{
    if (!out) return ASX_STATUS_INVALID_POINTER;
    *out = nullptr;
    if (m < 0 || n < 0 || nnz < 0 || ncols_dense < 1) return ASX_STATUS_INVALID_SIZE;
    if (value_type != ASX_R_32F && value_type != ASX_R_64F) return ASX_STATUS_NOT_SUPPORTED;
    if (m > 0 && !d_row_ptr) return ASX_STATUS_INVALID_POINTER;
    hipStream_t s = (hipStream_t)stream;
    asx_plan *p = nullptr;
    int st = plan_begin(&p, is_spmm, value_type, m, n, nnz, d_row_ptr, ncols_dense, s);
    if (st) return st;
    int kernel;
    if (!is_spmm)
        kernel = alg == ASX_SPMV_DEFAULT ? choose_spmv_from_stats(p->hist, p->stats, m, nnz) : asx_spmv_resolve_alg(alg, m, nnz);
    else
        kernel = asx_spmm_resolve_alg(alg, m, nnz, ncols_dense);
    if (kernel < 0 || (is_spmm && kernel == ASX_SPMM_BLOCKED)) {  // blocked plans need col and val too
        asx_plan_destroy(p);
        return ASX_STATUS_NOT_SUPPORTED;
    }
    st = plan_row_ordered(p, kernel, s);
    if (st) {
        asx_plan_destroy(p);
        return st;
    }
    *out = p;
    return ASX_STATUS_SUCCESS;
}

int asx_plan_destroy(asx_plan *plan)
{
    if (!plan) return ASX_STATUS_SUCCESS;
    int st = ASX_STATUS_SUCCESS;
    if (plan->d_meta) st = status_of(hipFree(plan->d_meta));
    if (plan->d_counters) (void)hipFree(plan->d_counters);
    if (plan->d_checksum_parts) (void)hipFree(plan->d_checksum_parts);
    free_blocked(&plan->blocked);
    free_sliced(&plan->sliced);
    free_window(&plan->window);
    delete plan;
    return st;
}

// Blocks are worth it when they are at least this full (bytes moved per stored element fall
// below the merge kernel's from about 1/8 upwards, see asx_blocked.hip).
static const double kBlockedMinFill = 0.125;
static const int32_t kBlockedProbeMaxNnz = 1 << 28;

int asx_spmm_plan_create(asx_plan **out, int alg, int value_type, int32_t m, int32_t k, int32_t nnz,
                         const int32_t *d_row_ptr, const int32_t *d_col, const void *d_val, int32_t ncols,
                         void *stream)
{
    if (!out) return ASX_STATUS_INVALID_POINTER;
    *out = nullptr;
    const int kernel = asx_spmm_resolve_alg(alg, m, nnz, ncols);
    if (kernel < 0) return ASX_STATUS_NOT_SUPPORTED;
    const bool want_blocked = kernel == ASX_SPMM_BLOCKED;
    // scattered columns (a sample of tiles of 1024 stored elements touches mostly distinct
    // 128-byte lines) cannot fill 16x4 blocks: the blocks are not even built then
    bool probe_blocked = alg == ASX_SPMM_DEFAULT && nnz > 0 && nnz <= kBlockedProbeMaxNnz && d_col &&
                         (value_type == ASX_R_32F || value_type == ASX_R_64F);
    if (probe_blocked) {
        int32_t *d_scratch = nullptr;
        if (hipMalloc((void **)&d_scratch, 128 * sizeof(int32_t)) != hipSuccess) return ASX_STATUS_ALLOC_FAILED;
        const ColumnSample cs = sample_columns(nullptr, m, d_col, nnz, vsize(value_type), d_scratch, (hipStream_t)stream);
        probe_blocked = cs.ok && cs.spread < kScatteredMinSpread;
        (void)hipFree(d_scratch);
    }
    if (!want_blocked && !probe_blocked)
        return asx_plan_create(out, 1, alg, value_type, m, k, nnz, d_row_ptr, ncols, stream);
    if (m < 0 || k < 0 || nnz < 0 || ncols < 1) return ASX_STATUS_INVALID_SIZE;
    if (value_type != ASX_R_32F && value_type != ASX_R_64F) return ASX_STATUS_NOT_SUPPORTED;
    if ((m > 0 && !d_row_ptr) || (nnz > 0 && (!d_col || !d_val))) return ASX_STATUS_INVALID_POINTER;
    hipStream_t s = (hipStream_t)stream;
    BlockedMatrix bm{};
    int st = value_type == ASX_R_64F
                 ? build_blocked<double>(m, k, nnz, d_row_ptr, d_col, (const double *)d_val, &bm, s)
                 : build_blocked<float>(m, k, nnz, d_row_ptr, d_col, (const float *)d_val, &bm, s);
    if (st) return st;
    const double fill = bm.nblocks > 0 ? (double)nnz / (64.0 * (double)bm.nblocks) : 0.0;
    if (!want_blocked && fill < kBlockedMinFill) {
        free_blocked(&bm);
        return asx_plan_create(out, 1, alg, value_type, m, k, nnz, d_row_ptr, ncols, stream);
    }
    asx_plan *p = new (std::nothrow) asx_plan();
    if (!p) {
        free_blocked(&bm);
        return ASX_STATUS_ALLOC_FAILED;
    }
    std::memset(p, 0, sizeof(*p));
    p->is_spmm = 1;
    p->alg = ASX_SPMM_BLOCKED;
    p->value_type = value_type;
    p->m = m;
    p->n = k;
    p->nnz = nnz;
    p->ncols = ncols;
    p->row_ptr = d_row_ptr;
    p->blocked = bm;
    p->nunits = bm.nblocks;
    p->workspace_bytes = 0;
    *out = p;
    return ASX_STATUS_SUCCESS;
}

}  // extern "C"

// ---- what DEFAULT picks when it may regroup A --------------------------------------------
// Decided from figures that do not change from one plan build to the next (the row-length
// histogram, the sizes, the column sample), never from timings: two analyses of one matrix keep the
// same kernel.  Estimated times (rates fitted to measurements on MI355X over families of matrices:
// uniform and power-law rows, bands, stencils, clustered columns):
//   row-ordered kernels   5 us + max(nnz spread' / g, bytes / 4.0 TB/s); g = gathers of x an L2
//                         serves per second: 180 G while x fits one (<= 3 MiB), 62 G once it does
//                         not (>= 6 MiB), linear in between; spread' = the sample's spread, at least
//                         0.05 (neighbouring columns share a line); bytes = nnz (sv + 4) + n sv + m (sv + 4)
//   column-sliced kernel  8 us + bytes / 6.0 TB/s, bytes = nnz (sv + 2) + P (2 sv + 2) + n sv + 2 m sv,
//                         P = nnz times the sample's pairs per stored element
//   row-block kernel      8 us + bytes / 5.0 TB/s (3.7 TB/s when rows longer than 16 are cut by
//                         tiles), bytes = (nnz + empty rows) (sv + 2) + n sv + 2 m sv; only for
//                         columns that are not scattered, and whether every block's columns fit a
//                         window is known once its build was tried
// A regrouped kernel is taken when its estimate is at least 3 % below the row-ordered one; of the
// two, the sliced one unless the row-block one is estimated more than 5 % faster.
constexpr int32_t kSlicedMinNnz = 1 << 21;
struct KernelEstimates {
    // seconds; infinity where the kernel does not apply.  window: with one ring of x per block;
    // window_bands: with rings per band of diagonals, window_stacked: with three bands on stacked
    // planes; which of the three it is only the build finds out
    double rows, sliced, window, window_bands, window_stacked;
};
static KernelEstimates estimate_kernels(const asx_plan *p, size_t sv, const ColumnSample &cs, bool window_ok, bool checked)
{
    const double inf = 1e30;
    const double nnz = (double)p->nnz, m = (double)p->m, n = (double)p->n, dsv = (double)sv;
    const double xbytes = n * dsv;
    const double lo = 3.0 * 1048576.0, hi = 6.0 * 1048576.0;
    const double f = xbytes <= lo ? 0.0 : xbytes >= hi ? 1.0 : (xbytes - lo) / (hi - lo);
    const double gather_rate = 180e9 + f * (62e9 - 180e9);
    KernelEstimates e;
    e.rows = 5e-6 + std::max(nnz * std::max(cs.spread, 0.05) / gather_rate, (nnz * (dsv + 4) + n * dsv + m * (dsv + 4)) / 4.0e12);
    const int64_t nslices = ceil_div64((int64_t)p->n * (int64_t)sv, kSliceBytes);
    e.sliced = nslices > kSlicedMaxSlices
                   ? inf
                   : 8e-6 + (nnz * (dsv + 2) + cs.pairs * nnz * (2 * dsv + 2) + n * dsv + 2 * m * dsv) / 6.0e12;
    // The row-block copy gives every row at least two slots.  Rates measured over the audit's
    // families (what the copy moves / (time - 8 us)): one ring 5.8e12 with rows the tiles do not cut
    // (5-point stencil, band of 9), 5.0 and 4.6e12 with rows of 19 and 65; rings per band, x fetched
    // about 1.5 times: 4.7e12 (7-point stencil) and 3.9e12 (27-point).
    const double wslots = nnz + 2.0 * (double)p->hist[0] + (double)p->hist[1];
    const bool uncut = p->stats[0] <= 16;
    e.window = !window_ok ? inf : 8e-6 + (wslots * (dsv + 2) + n * dsv + 2 * m * dsv) / (uncut ? 5.6e12 : 4.8e12);
    e.window_bands = !window_ok ? inf : 8e-6 + (wslots * (dsv + 2) + 1.5 * n * dsv + 2 * m * dsv) / (uncut ? 4.6e12 : 3.9e12);
    // three bands on stacked planes (x fetched about 1.3 times): 7-point stencil on 160^3 5.6e12 in
    // fp64 but 3.5e12 in fp32, where the time goes with the slots and not with the bytes; 27-point
    // on 96^3 (rows of 27, cut by tiles) 4.2e12
    e.window_stacked = !window_ok ? inf
                                  : 8e-6 + (wslots * (dsv + 2) + 1.3 * n * dsv + 2 * m * dsv) /
                                               (sv == 8 ? (uncut ? 5.6e12 : 4.2e12) : (uncut ? 3.5e12 : 3.0e12));
    if (checked) {
        // a checked plan reads the caller's values once more in every call (a stream of its own
        // kernel: 6.3 TB/s measured) and launches three small kernels
        const double check = 10e-6 + nnz * dsv / 6.0e12;
        e.sliced += check;
        if (p->hist[0] + p->hist[1] > 0)
            e.window += check, e.window_bands += check, e.window_stacked += check;
        else if (sv == 8)  // reads A's values in place: no check, but two scans a tile
            e.window *= 1.06, e.window_bands *= 1.06, e.window_stacked *= 1.06;
    }
    return e;
}

// Builds the sliced copy onto a plan that already holds the histogram (`p` takes the slices over;
// its own split points are dropped).
template <typename T>
int plan_add_slices(asx_plan *p, const int32_t *d_row_ptr, const int32_t *d_col, const T *d_val, double pairs_per_element,
                    hipStream_t s)
{
    int cus = 256;
    (void)asx_device_info(&cus, nullptr);
    // pass 2: one wave per block of rows, its accumulators (8 bytes a row) in LDS.  Blocks of 256
    // rows, doubled up to 1024 while that leaves more than 8 waves per compute unit and the block's
    // partial sums inside one slice (expected from the column sample) are fewer than 12: a
    // step of pass 2 takes its 64 entries from at most three ranges.  Small blocks mean many waves
    // in flight.  Measured: the power-law matrix (4 per range at 256 rows) 50 / 34.5 / 36.6 us with
    // 512 / 1024 / 2048 rows; 16 per row over 32 slices (100 per range at 256 rows) 17.5 / 20 us
    // with 256 / 512 rows; the same in fp64 over 64 slices 26.5 / 27.5 / 36.8 us with 256 / 512 / 1024.
    const int32_t nslices = (int32_t)ceil_div64((int64_t)p->n * (int64_t)sizeof(T), kSliceBytes);
    const double per_row_slice = pairs_per_element * (double)p->nnz / ((double)p->m * (double)nslices);
    int32_t rpw = 256;
    while (rpw < 1024 && (int64_t)rpw * cus * 8 < p->m && per_row_slice * rpw < 12.0) rpw *= 2;
    SlicedMatrix sm{};
    const int st = build_sliced<T>(p->m, p->n, p->nnz, (int32_t)(kSliceBytes / sizeof(T)), rpw, cus, d_row_ptr, d_col,
                                   d_val, &sm, s);
    if (st) return st;
    if (p->d_meta) (void)hipFree(p->d_meta);
    p->d_meta = nullptr;
    p->meta_bytes = 0;
    p->alg = ASX_SPMV_SLICED;
    p->sliced = sm;
    p->nunits = sm.ntiles;
    p->carry_pass = 0;
    p->workspace_bytes = sliced_scratch_bytes(&sm, sizeof(T));
    return ASX_STATUS_SUCCESS;
}

// Builds the row-block copy onto a plan that already holds the histogram.
template <typename T>
int plan_add_window(asx_plan *p, const int32_t *d_row_ptr, const int32_t *d_col, const T *d_val, bool follows_values, hipStream_t s)
{
    int cus = 256;
    (void)asx_device_info(&cus, nullptr);
    WindowMatrix wm{};
    // one chain of row blocks per compute unit for fp64 (128 KiB of LDS each), two for fp32
    // Reading A's values in place costs a multiply in fp32 nothing and in fp64 a twentieth to a
    // tenth (two scans a tile instead of one; 5-point stencil on 4096^2: 201 us from the copy, 210 to
    // 220 in place; a refresh of the copy takes more than a multiply): fp32 plans always do where
    // they can, fp64 plans when the caller wants values changed in place to be followed (a checked
    // plan), which then takes no check at all.
    const int st = build_window<T>(p->m, p->n, p->nnz, cus * (sizeof(T) == 4 ? 2 : 1), sizeof(T) == 4 || follows_values, d_row_ptr,
                                   d_col, d_val, &wm, s);
    if (st) return st;
    if (p->d_meta) (void)hipFree(p->d_meta);
    p->d_meta = nullptr;
    p->meta_bytes = 0;
    p->alg = ASX_SPMV_WINDOW;
    p->window = wm;
    p->nunits = wm.ntiles;
    p->carry_pass = wm.has_carry;
    p->workspace_bytes = window_scratch_bytes(&wm, sizeof(T));
    return ASX_STATUS_SUCCESS;
}

// DEFAULT tries the row-block copy for matrices the flat or merge-path kernel would take, without
// rows past the carry pass's limit, and with few rows of fewer than two stored elements: the copy
// gives every row at least two slots (a value, a column word and a source index each, read in every
// call), so a matrix where that padding exceeds a quarter of its stored elements stays with the
// other kernels.
// A regrouped copy roughly doubles what the matrix takes on the device (per stored element: the
// value, 2 bytes of column, 4 bytes of source index; the sliced kernel also 2 bytes for bringing
// the values up to date and a buffer for the partial sums of a call), and its build needs about 4
// bytes per stored element more for a while.
// DEFAULT only makes one while twice that is free: a caller who sized the device for one copy of A
// is not pushed to the edge by an analysis call.
static bool regrouped_copy_fits(const asx_plan *p, size_t sv)
{
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) return false;
    const double copy = (double)p->nnz * (double)(sv + 8) + (double)p->nnz * (double)(sv + 2) + (double)p->nnz * 4.0;
    return (double)free_b >= 2.0 * copy;
}

static bool window_may_pay(const asx_plan *p, int row_kernel)
{
    return (row_kernel == ASX_SPMV_FLAT || row_kernel == ASX_SPMV_MERGE) &&
           2 * p->hist[0] + p->hist[1] <= (int64_t)p->nnz / 4;
}

// the checksum words of a plan: of the values as they are now (2), of the values its copy holds (2)
static unsigned long long *checksum_words(const asx_plan *p) { return reinterpret_cast<unsigned long long *>(p->d_counters + 44); }

// Takes the checksum of d_val and keeps it as the checksum of the plan's copy (which was just made
// or refreshed from d_val).
static int keep_checksum(asx_plan *p, const void *d_val, hipStream_t s)
{
    unsigned long long *w = checksum_words(p);
    int st = ASX_STATUS_SUCCESS;
    if (!p->d_checksum_parts) st = status_of(hipMalloc((void **)&p->d_checksum_parts, sizeof(unsigned long long) * 2 * checksum_parts()));
    if (!st) st = launch_checksum(d_val, (size_t)p->nnz * vsize(p->value_type), p->d_checksum_parts, w, s);
    if (!st) st = launch_checksum_commit(w, w + 2, s);
    return st;
}

static int spmv_plan_create(asx_plan **out, int alg, int value_type, int32_t m, int32_t n, int32_t nnz,
                            const int32_t *d_row_ptr, const int32_t *d_col, const void *d_val, bool checked, void *stream)
{
    if (!out) return ASX_STATUS_INVALID_POINTER;
    *out = nullptr;
    if (m < 0 || n < 0 || nnz < 0) return ASX_STATUS_INVALID_SIZE;
    if (value_type != ASX_R_32F && value_type != ASX_R_64F) return ASX_STATUS_NOT_SUPPORTED;
    if (m > 0 && !d_row_ptr) return ASX_STATUS_INVALID_POINTER;
    const bool want = alg == ASX_SPMV_SLICED || alg == ASX_SPMV_WINDOW;
    if (want && (m == 0 || nnz == 0 || n == 0)) return ASX_STATUS_INVALID_SIZE;
    if (want && (!d_row_ptr || !d_col || !d_val)) return ASX_STATUS_INVALID_POINTER;
    int row_kernel = -1;  // the row-ordered kernel to fall back to
    if (alg != ASX_SPMV_DEFAULT && !want) {
        row_kernel = asx_spmv_resolve_alg(alg, m, nnz);
        if (row_kernel < 0) return ASX_STATUS_NOT_SUPPORTED;
    }
    hipStream_t s = (hipStream_t)stream;
    asx_plan *p = nullptr;
    int st = plan_begin(&p, 0, value_type, m, n, nnz, d_row_ptr, 1, s);
    if (st) return st;
    if (alg == ASX_SPMV_DEFAULT) row_kernel = choose_spmv_from_stats(p->hist, p->stats, m, nnz);
    const bool f64 = value_type == ASX_R_64F;
    const size_t sv = vsize(value_type);
    int32_t *d_sample = reinterpret_cast<int32_t *>(p->d_counters + 64);  // 128 ints
    const auto add_slices = [&](double pairs) {
        return f64 ? plan_add_slices<double>(p, d_row_ptr, d_col, (const double *)d_val, pairs, s)
                   : plan_add_slices<float>(p, d_row_ptr, d_col, (const float *)d_val, pairs, s);
    };
    const auto add_window = [&]() {
        return f64 ? plan_add_window<double>(p, d_row_ptr, d_col, (const double *)d_val, checked, s)
                   : plan_add_window<float>(p, d_row_ptr, d_col, (const float *)d_val, checked, s);
    };
    const bool can_regroup = alg == ASX_SPMV_DEFAULT && d_col && d_val && m > 0 && n > 0 && nnz >= kSlicedMinNnz &&
                             regrouped_copy_fits(p, sv);
    bool done = false;
    if (alg == ASX_SPMV_WINDOW) {
        st = add_window();
        done = true;
    } else if (alg == ASX_SPMV_SLICED) {
        const ColumnSample cs = sample_columns(d_row_ptr, m, d_col, nnz, sv, d_sample, s);  // sizes the row blocks of pass 2
        st = add_slices(cs.pairs);
        done = true;
    } else if (can_regroup) {
        // DEFAULT: a regrouped copy where it is estimated to pay; a build that fails (out of memory,
        // a matrix the kernel does not take) is not an error: the next choice stands
        const ColumnSample cs = sample_columns(d_row_ptr, m, d_col, nnz, sv, d_sample, s);
        if (cs.ok) {
            // the row-block kernel needs columns near each other; whether they fit its windows the
            // build finds out (NOT_SUPPORTED when some 256 rows reach further)
            const bool window_ok = window_may_pay(p, row_kernel) && cs.spread < kScatteredMinSpread;
            const KernelEstimates e = estimate_kernels(p, sv, cs, window_ok, checked);
            const bool sliced_pays = e.sliced < 0.97 * e.rows, window_pays = e.window < 0.97 * e.rows;
            if (window_pays && e.window < e.sliced / 1.05) done = add_window() == ASX_STATUS_SUCCESS;
            if (done && p->window.nbands > 1 && sliced_pays &&
                !((p->window.stack_rows > 0 ? e.window_stacked : e.window_bands) < e.sliced / 1.05)) {
                // the build needed a ring per band of diagonals; with those the slices are ahead
                WindowMatrix built = p->window;
                p->window = WindowMatrix{};
                if (add_slices(cs.pairs) == ASX_STATUS_SUCCESS)
                    free_window(&built);
                else
                    p->window = built, p->alg = ASX_SPMV_WINDOW;
            }
            if (!done && sliced_pays) done = add_slices(cs.pairs) == ASX_STATUS_SUCCESS;
            if (!done && window_pays && !(e.window < e.sliced / 1.05)) done = add_window() == ASX_STATUS_SUCCESS;
        }
    }
    if (!done) st = plan_row_ordered(p, row_kernel, s);
    if (!st && checked && asx_plan_holds_values(p)) {
        // the values must lie on a 16-byte boundary for the checksum's loads (every allocation does);
        // a view that does not keeps an unchecked plan out: row-ordered instead
        if (((uintptr_t)d_val % 16) == 0) {
            st = keep_checksum(p, d_val, s);
            p->checked = st == ASX_STATUS_SUCCESS;
        } else {
            asx_plan_destroy(p);
            if (want) return ASX_STATUS_INVALID_VALUE;  // the kernel was asked for by name
            return spmv_plan_create(out, alg, value_type, m, n, nnz, d_row_ptr, nullptr, nullptr, false, stream);
        }
    }
    if (st) {
        asx_plan_destroy(p);
        return st;
    }
    *out = p;
    return ASX_STATUS_SUCCESS;
}

extern "C" {

int asx_spmv_plan_create(asx_plan **out, int alg, int value_type, int32_t m, int32_t n, int32_t nnz,
                         const int32_t *d_row_ptr, const int32_t *d_col, const void *d_val, void *stream)
{
    return spmv_plan_create(out, alg, value_type, m, n, nnz, d_row_ptr, d_col, d_val, false, stream);
}

int asx_spmv_plan_create_checked(asx_plan **out, int alg, int value_type, int32_t m, int32_t n, int32_t nnz,
                                 const int32_t *d_row_ptr, const int32_t *d_col, const void *d_val, void *stream)
{
    return spmv_plan_create(out, alg, value_type, m, n, nnz, d_row_ptr, d_col, d_val, true, stream);
}

int asx_plan_is_checked(const asx_plan *plan) { return plan && plan->checked ? 1 : 0; }

int asx_plan_refresh_if_changed(asx_plan *plan, const void *d_val, void *stream)
{
    if (!plan) return ASX_STATUS_INVALID_POINTER;
    if (!plan->checked) return ASX_STATUS_SUCCESS;  // reads the caller's values in every call, or was made unchecked
    if (plan->nnz > 0 && !d_val) return ASX_STATUS_INVALID_POINTER;
    if (((uintptr_t)d_val % 16) != 0) return ASX_STATUS_INVALID_VALUE;
    hipStream_t s = (hipStream_t)stream;
    unsigned long long *w = checksum_words(plan);
    int st = launch_checksum(d_val, (size_t)plan->nnz * vsize(plan->value_type), plan->d_checksum_parts, w, s);
    if (st) return st;
    if (plan->alg == ASX_SPMV_SLICED)
        st = plan->value_type == ASX_R_64F ? sliced_update_values<double>(&plan->sliced, (const double *)d_val, s, w)
                                           : sliced_update_values<float>(&plan->sliced, (const float *)d_val, s, w);
    else if (plan->alg == ASX_SPMV_WINDOW)
        st = plan->value_type == ASX_R_64F ? window_update_values<double>(&plan->window, (const double *)d_val, s, w)
                                           : window_update_values<float>(&plan->window, (const float *)d_val, s, w);
    if (st) return st;
    return launch_checksum_commit(w, w + 2, s);
}

int asx_plan_update_values(asx_plan *plan, const void *d_val, void *stream)
{
    if (!plan) return ASX_STATUS_INVALID_POINTER;
    if (plan->nnz > 0 && !d_val) return ASX_STATUS_INVALID_POINTER;
    hipStream_t s = (hipStream_t)stream;
    if (!plan->is_spmm && (plan->alg == ASX_SPMV_SLICED || plan->alg == ASX_SPMV_WINDOW)) {
        int st;
        if (plan->alg == ASX_SPMV_SLICED)
            st = plan->value_type == ASX_R_64F ? sliced_update_values<double>(&plan->sliced, (const double *)d_val, s)
                                               : sliced_update_values<float>(&plan->sliced, (const float *)d_val, s);
        else
            st = plan->value_type == ASX_R_64F ? window_update_values<double>(&plan->window, (const double *)d_val, s)
                                               : window_update_values<float>(&plan->window, (const float *)d_val, s);
        if (!st && plan->checked) st = ((uintptr_t)d_val % 16) == 0 ? keep_checksum(plan, d_val, s) : ASX_STATUS_INVALID_VALUE;
        return st;
    }
    if (plan->is_spmm && plan->alg == ASX_SPMM_BLOCKED)
        return plan->value_type == ASX_R_64F ? blocked_update_values<double>(&plan->blocked, (const double *)d_val, s)
                                             : blocked_update_values<float>(&plan->blocked, (const float *)d_val, s);
    return ASX_STATUS_SUCCESS;  // the other kernels read the caller's values in every call
}

int asx_plan_holds_values(const asx_plan *plan)
{
    if (!plan) return 0;
    return (!plan->is_spmm && (plan->alg == ASX_SPMV_SLICED || (plan->alg == ASX_SPMV_WINDOW && !plan->window.by_reference))) ||
           (plan->is_spmm && plan->alg == ASX_SPMM_BLOCKED);
}

int asx_plan_block_stats(const asx_plan *plan, int64_t *nblocks, double *fill)
{
    if (!plan || !nblocks || !fill) return ASX_STATUS_INVALID_POINTER;
    if (plan->alg != ASX_SPMM_BLOCKED) return ASX_STATUS_INVALID_VALUE;
    *nblocks = plan->blocked.nblocks;
    *fill = plan->blocked.nblocks > 0 ? (double)plan->nnz / (64.0 * (double)plan->blocked.nblocks) : 0.0;
    return ASX_STATUS_SUCCESS;
}

size_t asx_plan_own_scratch_bytes(const asx_plan *plan)
{
    if (!plan || plan->is_spmm) return 0;
    if (plan->alg == ASX_SPMV_SLICED && plan->sliced.partial) return sliced_scratch_bytes(&plan->sliced, vsize(plan->value_type));
    if (plan->alg == ASX_SPMV_WINDOW && plan->window.carry) return window_scratch_bytes(&plan->window, vsize(plan->value_type));
    return 0;
}

int asx_plan_release_scratch(asx_plan *plan)
{
    if (!plan) return ASX_STATUS_INVALID_POINTER;
    int st = ASX_STATUS_SUCCESS;
    if (plan->sliced.partial) {
        st = status_of(hipFree(plan->sliced.partial));
        plan->sliced.partial = nullptr;
    }
    if (plan->window.carry) {
        const int st2 = status_of(hipFree(plan->window.carry));
        plan->window.carry = nullptr;
        if (!st) st = st2;
    }
    return st;
}

// The arrays of a plan that holds a regrouped copy of A: device address and bytes.
static bool plan_array(const asx_plan *p, int what, const void **ptr, size_t *bytes)
{
    const size_t sv = vsize(p->value_type);
    *ptr = nullptr;
    *bytes = 0;
    if (!p->is_spmm && p->alg == ASX_SPMV_SLICED) {
        const SlicedMatrix &m = p->sliced;
        const size_t slots = (size_t)m.ntiles * kSlicedTile;
        switch (what) {
        case ASX_PLAN_ARRAY_VAL: *ptr = m.val, *bytes = slots * sv; return true;
        case ASX_PLAN_ARRAY_CF: *ptr = m.cf, *bytes = slots * 2; return true;
        case ASX_PLAN_ARRAY_PERM: *ptr = m.perm, *bytes = slots * 4; return true;
        case ASX_PLAN_ARRAY_TILE_WORDS: *ptr = m.tile_base, *bytes = ((size_t)m.ntiles + 1) * 4; return true;
        case ASX_PLAN_ARRAY_WORKGROUPS: *ptr = m.wg_tab, *bytes = (size_t)m.npieces * 16; return true;
        case ASX_PLAN_ARRAY_WG_PIECES: *ptr = m.wg_pieces, *bytes = (size_t)m.nwg * 32; return true;
        case ASX_PLAN_ARRAY_PARTIAL_ROWS: *ptr = m.prow, *bytes = (size_t)m.npartials * 2; return true;
        case ASX_PLAN_ARRAY_RANGES: *ptr = m.chunk_lo, *bytes = ((size_t)m.nrb + 1) * (size_t)m.nslices * 4; return true;
        case ASX_PLAN_ARRAY_STEP_PTR: *ptr = m.pstep_ptr, *bytes = ((size_t)m.nrb + 1) * 4; return true;
        case ASX_PLAN_ARRAY_STEPS: *ptr = m.psteps, *bytes = (size_t)m.npsteps * 16; return true;
        default: return false;
        }
    }
    if (!p->is_spmm && p->alg == ASX_SPMV_WINDOW) {
        const WindowMatrix &m = p->window;
        const size_t slots = (size_t)m.ntiles * kSlicedTile;
        switch (what) {
        case ASX_PLAN_ARRAY_VAL: *ptr = m.val, *bytes = slots * sv; return m.val != nullptr;
        case ASX_PLAN_ARRAY_CF: *ptr = m.cf, *bytes = slots * 2; return true;
        case ASX_PLAN_ARRAY_PERM: *ptr = m.perm, *bytes = slots * 4; return m.perm != nullptr;
        case ASX_PLAN_ARRAY_TILE_WORDS: *ptr = m.tile_info, *bytes = (size_t)m.ntiles * 16; return true;
        case ASX_PLAN_ARRAY_WORKGROUPS: *ptr = m.chains, *bytes = (size_t)m.nchains * 8; return true;
        case ASX_PLAN_ARRAY_BLOCKS: *ptr = m.blocks, *bytes = (size_t)m.nblocks * 16; return true;
        case ASX_PLAN_ARRAY_PIECES: *ptr = m.pieces, *bytes = (size_t)m.npieces * 16; return true;
        default: return false;
        }
    }
    return false;
}

int asx_plan_export(const asx_plan *plan, int what, void *h_dst, size_t cap, size_t *bytes, void *stream)
{
    if (!plan || !bytes) return ASX_STATUS_INVALID_POINTER;
    const void *src;
    if (!plan_array(plan, what, &src, bytes)) return ASX_STATUS_INVALID_VALUE;
    if (!h_dst) return ASX_STATUS_SUCCESS;  // sizing call
    if (cap < *bytes) return ASX_STATUS_INVALID_SIZE;
    if (*bytes == 0) return ASX_STATUS_SUCCESS;
    hipStream_t s = (hipStream_t)stream;
    int st = status_of(hipMemcpyAsync(h_dst, src, *bytes, hipMemcpyDeviceToHost, s));
    if (!st) st = status_of(hipStreamSynchronize(s));
    return st;
}

int asx_plan_alg(const asx_plan *plan) { return plan ? plan->alg : -1; }
const char *asx_kernel_name(int is_spmm, int kernel)
{
    if (is_spmm) {
        switch (kernel) {
        case ASX_SPMM_ROW: return "row";
        case ASX_SPMM_MERGE: return "merge";
        case ASX_SPMM_BLOCKED: return "blocked";
        default: return "?";
        }
    }
    switch (kernel) {
    case ASX_SPMV_VECTOR: return "vector";
    case ASX_SPMV_STREAM: return "stream";
    case ASX_SPMV_MERGE: return "merge";
    case ASX_SPMV_FLAT: return "flat";
    case ASX_SPMV_SLICED: return "sliced";
    case ASX_SPMV_WINDOW: return "window";
    default: return "?";
    }
}
size_t asx_plan_workspace_bytes(const asx_plan *plan) { return plan ? plan->workspace_bytes : 0; }
int64_t asx_plan_info(const asx_plan *plan, int what)
{
    if (!plan || plan->is_spmm) return -1;
    const bool sliced = plan->alg == ASX_SPMV_SLICED, window = plan->alg == ASX_SPMV_WINDOW;
    switch (what) {
    case ASX_PLAN_INFO_TILES: return sliced ? plan->sliced.ntiles : window ? plan->window.ntiles : -1;
    case ASX_PLAN_INFO_SLICES: return sliced ? plan->sliced.nslices : -1;
    case ASX_PLAN_INFO_PARTIAL_SUMS: return sliced ? plan->sliced.npartials : -1;
    case ASX_PLAN_INFO_ROWS_PER_WAVE: return sliced ? plan->sliced.rows_per_wave : -1;
    case ASX_PLAN_INFO_ROWS_PER_BLOCK: return window ? plan->window.rows_per_block : -1;
    case ASX_PLAN_INFO_BANDS: return window ? plan->window.nbands : -1;
    case ASX_PLAN_INFO_CHAINS: return window ? plan->window.nchains : -1;
    case ASX_PLAN_INFO_CARRY_PASS: return window ? plan->window.has_carry : -1;
    case ASX_PLAN_INFO_ROW_BLOCKS: return sliced ? plan->sliced.nrb : window ? plan->window.nblocks : -1;
    case ASX_PLAN_INFO_STEPS: return sliced ? plan->sliced.npsteps : -1;
    case ASX_PLAN_INFO_WIDTH: return sliced ? plan->sliced.width : window ? 16384 : -1;
    case ASX_PLAN_INFO_WORKGROUPS: return sliced ? plan->sliced.nwg : window ? plan->window.nchains : -1;
    case ASX_PLAN_INFO_PIECES: return window ? plan->window.npieces : -1;
    case ASX_PLAN_INFO_STACKED_ROWS: return window ? plan->window.stack_rows : -1;
    case ASX_PLAN_INFO_BY_REFERENCE: return window ? plan->window.by_reference : -1;
    default: return -1;
    }
}
int asx_plan_histogram(const asx_plan *plan, int64_t h_hist[33], int64_t h_stats[4])
{
    if (!plan || !h_hist || !h_stats) return ASX_STATUS_INVALID_POINTER;
    std::memcpy(h_hist, plan->hist, sizeof(plan->hist));
    std::memcpy(h_stats, plan->stats, sizeof(plan->stats));
    return ASX_STATUS_SUCCESS;
}

// ---------------------------------------------------------------- SpMV
// Reference algorithm ids (include/alphasparse/spdef.h:345-365) onto the four plan-less kernels here:
// the reference's scalar/vector/line-enhance families are one-row-per-lane-group kernels, its
// adaptive/stream families stage row blocks through LDS, its flat/acc families cut the stored
// elements into equal tiles of 1024, its merge/row-partition/load-balance families split work
// evenly whatever the row lengths.
int asx_spmv_resolve_alg(int alg, int32_t m, int32_t nnz)
{
    (void)m;
    (void)nnz;
    switch (alg) {
    case 0: return ASX_SPMV_FLAT;    /* DEFAULT without a histogram: even work per tile, no bad case */
    case 5:                          /* SCALAR */
    case 6:                          /* VECTOR */
    case 10:                         /* LINE */
    case 16: return ASX_SPMV_VECTOR; /* LINE_ENHANCE */
    case 2:                          /* CSR_ADAPTIVE */
    case 3:                          /* CSR_STREAM */
    case 8: return ASX_SPMV_STREAM;  /* ADAPTIVE */
    case 11:
    case 12:
    case 13: /* FLAT1/4/8 */
    case 14: /* ACC */
    case 15: /* FLAT */
    case 18: return ASX_SPMV_FLAT;   /* PFLAT */
    case 7:                          /* ROW_PARTITION */
    case 9:                          /* MERGE */
    case 17: return ASX_SPMV_MERGE;  /* LOAD_BALANCE */
    default: return -1;              /* COO (1), ELL (4): other formats */
    }
}

size_t asx_spmv_workspace_bytes(int alg, int value_type, int32_t m, int32_t nnz)
{
    const int kernel = asx_spmv_resolve_alg(alg, m, nnz);
    const size_t merge = spmv_merge_layout(m, nnz, vsize(value_type), true).bytes;
    const size_t flat = spmv_flat_layout(nnz, vsize(value_type), true).bytes;
    // DEFAULT: a plan may pick the merge-path kernel (hypersparse or very long rows), whose carry
    // array can exceed the flat kernel's: report what every choice fits in
    if (alg == ASX_SPMV_DEFAULT) return std::max(merge, flat);
    if (kernel == ASX_SPMV_MERGE) return merge;
    if (kernel == ASX_SPMV_FLAT) return flat;
    if (kernel == ASX_SPMV_STREAM)
        return align_up(((size_t)std::max(stream_blocks(nnz), 1) + 1) * 8, kAlign);
    return 0;
}

int asx_spmv_csr_f64(const asx_plan *plan, int alg, int32_t m, int32_t n, int32_t nnz, double alpha,
                     const int32_t *d_row_ptr, const int32_t *d_col, const double *d_val,
                     const double *d_x, double beta, double *d_y, void *d_workspace,
                     size_t workspace_bytes, void *stream)
{
    return spmv_impl<double>(plan, alg, m, n, nnz, alpha, d_row_ptr, d_col, d_val, d_x, beta, d_y,
                             d_workspace, workspace_bytes, (hipStream_t)stream);
}
int asx_spmv_csr_f32(const asx_plan *plan, int alg, int32_t m, int32_t n, int32_t nnz, float alpha,
                     const int32_t *d_row_ptr, const int32_t *d_col, const float *d_val,
                     const float *d_x, float beta, float *d_y, void *d_workspace,
                     size_t workspace_bytes, void *stream)
{
    return spmv_impl<float>(plan, alg, m, n, nnz, alpha, d_row_ptr, d_col, d_val, d_x, beta, d_y,
                            d_workspace, workspace_bytes, (hipStream_t)stream);
}

// ---------------------------------------------------------------- SpMV without any allocation
}  // extern "C"

// Split points and carries of a plan-less call, for callers that can neither allocate nor bring
// a buffer.  One copy of the array per GPU, held until the process ends; its device address is
// looked up once per device (the array's name is not a device address in host code).
static constexpr size_t kNoAllocScratchBytes = (size_t)4 << 20;
static __device__ __align__(256) unsigned char asx_noalloc_scratch[kNoAllocScratchBytes];
static constexpr int kNoAllocMaxDevices = 64;
static void *g_noalloc_ptr[kNoAllocMaxDevices];
static std::mutex g_noalloc_mutex;

// Device address of this device's copy of the scratch array; the device must be current.
static int noalloc_scratch(void **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return status_of(e);
    if (dev < 0 || dev >= kNoAllocMaxDevices) return ASX_STATUS_NOT_SUPPORTED;
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);
    if (!g_noalloc_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(asx_noalloc_scratch));
        if (e != hipSuccess) return status_of(e);
        if (!p) return ASX_STATUS_INTERNAL_ERROR;
        g_noalloc_ptr[dev] = p;
    }
    *out = g_noalloc_ptr[dev];
    return ASX_STATUS_SUCCESS;
}

extern "C" {

size_t asx_spmv_noalloc_max_workspace(void) { return kNoAllocScratchBytes; }

int asx_spmv_csr_f64_noalloc(int alg, int32_t m, int32_t n, int32_t nnz, double alpha, const int32_t *d_row_ptr,
                             const int32_t *d_col, const double *d_val, const double *d_x, double beta, double *d_y,
                             void *stream)
{
    if (m < 0 || n < 0 || nnz < 0) return ASX_STATUS_INVALID_SIZE;
    if (asx_spmv_resolve_alg(alg, m, nnz) < 0) return ASX_STATUS_NOT_SUPPORTED;
    // what the kernel this call runs would ask of a caller's buffer must fit the array (for DEFAULT
    // that is the flat kernel: without a plan nothing else is chosen)
    const size_t need = asx_spmv_workspace_bytes(asx_spmv_resolve_alg(alg, m, nnz), ASX_R_64F, m, nnz);
    if (need > kNoAllocScratchBytes) return ASX_STATUS_INVALID_SIZE;
    void *ws = nullptr;
    const int st = noalloc_scratch(&ws);
    if (st) return st;
    // every kernel writes the split points and carries it reads: nothing has to start at zero
    return spmv_impl<double>(nullptr, alg, m, n, nnz, alpha, d_row_ptr, d_col, d_val, d_x, beta, d_y, ws,
                             kNoAllocScratchBytes, (hipStream_t)stream);
}

// ---------------------------------------------------------------- SpMM
int asx_spmm_resolve_alg(int alg, int32_t m, int32_t nnz, int32_t ncols)
{
    (void)m;
    (void)nnz;
    (void)ncols;
    switch (alg) {
    case 0: return ASX_SPMM_MERGE; /* DEFAULT */
    case 5: return ASX_SPMM_ROW;   /* CSR_ALG1 row split */
    case 6:                        /* CSR_ALG2 nnz split */
    case 7:                        /* CSR_ALG3 merge */
    case 8:                        /* CSR_ALG4 adaptive */
    case 9: return ASX_SPMM_MERGE; /* CSR_ALG5 flat */
    case 10: return ASX_SPMM_BLOCKED; /* CSR_ALG6: needs a plan from asx_spmm_plan_create */
    default: return -1;            /* COO algorithms */
    }
}

size_t asx_spmm_workspace_bytes(int alg, int value_type, int32_t m, int32_t nnz, int32_t ncols)
{
    const int kernel = asx_spmm_resolve_alg(alg, m, nnz, ncols);
    if (kernel == ASX_SPMM_MERGE) return spmm_merge_layout(m, nnz, ncols, vsize(value_type), true).bytes;
    return 0;
}

int asx_spmm_csr_f32(const asx_plan *plan, int alg, int32_t m, int32_t k, int32_t nnz, int32_t ncols,
                     float alpha, const int32_t *d_row_ptr, const int32_t *d_col, const float *d_val,
                     const float *d_B, int64_t ldb, float beta, float *d_C, int64_t ldc,
                     void *d_workspace, size_t workspace_bytes, void *stream)
{
    return spmm_impl<float>(plan, alg, m, k, nnz, ncols, alpha, d_row_ptr, d_col, d_val, d_B, ldb, beta,
                            d_C, ldc, d_workspace, workspace_bytes, (hipStream_t)stream);
}
int asx_spmm_csr_f64(const asx_plan *plan, int alg, int32_t m, int32_t k, int32_t nnz, int32_t ncols,
                     double alpha, const int32_t *d_row_ptr, const int32_t *d_col, const double *d_val,
                     const double *d_B, int64_t ldb, double beta, double *d_C, int64_t ldc,
                     void *d_workspace, size_t workspace_bytes, void *stream)
{
    return spmm_impl<double>(plan, alg, m, k, nnz, ncols, alpha, d_row_ptr, d_col, d_val, d_B, ldb,
                             beta, d_C, ldc, d_workspace, workspace_bytes, (hipStream_t)stream);
}

int asx_copy_bytes(const void *d_src, void *d_dst, size_t bytes, void *stream)
{
    if (!d_src || !d_dst) return ASX_STATUS_INVALID_POINTER;
    if (bytes % 16) return ASX_STATUS_INVALID_SIZE;
    return launch_copy_bytes(d_src, d_dst, bytes, (hipStream_t)stream);
}

int asx_gather_lines(const void *d_buf, size_t bytes, int group_lanes, int loads_per_lane, void *d_out, int *nthreads,
                     void *stream)
{
    if (d_out && !d_buf) return ASX_STATUS_INVALID_POINTER;
    return launch_gather_lines(d_buf, bytes, group_lanes, loads_per_lane, d_out, nthreads, (hipStream_t)stream);
}

}  // extern "C"
