// Builds the column-panel copy of a CSR matrix for the panel SpMV kernel (device side, once per
// plan).  A stable radix sort of the stored elements by panel keeps CSR order inside each panel;
// the first element of every (panel, row) run opens a compact row of that panel.
#include <hipcub/hipcub.hpp>

#include "asx_internal.hpp"

namespace asx {

__global__ __launch_bounds__(kBlock) void k_panel_keys(const int32_t *__restrict__ col, int32_t nnz, int32_t width,
                                                       int32_t *__restrict__ keys, int32_t *__restrict__ idx)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    keys[i] = col[i] / width;
    idx[i] = (int32_t)i;
}

struct PanelOffsets {
    int32_t pstart[kPanels + 1];
    int64_t elem_off[kPanels + 1];
};

// Copies columns and values into panel order and finds the row of A of every element.
template <typename T>
__global__ __launch_bounds__(kBlock) void k_panel_gather(const int32_t *__restrict__ keys, const int32_t *__restrict__ idx,
                                                         int32_t nnz, PanelOffsets o, const int32_t *__restrict__ row_ptr,
                                                         int32_t m, const int32_t *__restrict__ col,
                                                         const T *__restrict__ val, int32_t *__restrict__ col_out,
                                                         T *__restrict__ val_out, int32_t *__restrict__ srow)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    const int j = keys[i];
    const int64_t dst = o.elem_off[j] + (i - o.pstart[j]);
    const int32_t src = idx[i];
    col_out[dst] = col[src];
    val_out[dst] = val[src];
    int32_t lo = 0, hi = m;  // largest r with row_ptr[r] <= src
    while (lo < hi) {
        const int32_t mid = lo + (hi - lo + 1) / 2;
        if (row_ptr[mid] <= src)
            lo = mid;
        else
            hi = mid - 1;
    }
    srow[i] = lo;
}

// head[i] = 1 where element i opens a (panel, row) run
__global__ __launch_bounds__(kBlock) void k_panel_heads(const int32_t *__restrict__ keys, const int32_t *__restrict__ srow,
                                                        int32_t nnz, int32_t *__restrict__ head)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    head[i] = i == 0 || keys[i] != keys[i - 1] || srow[i] != srow[i - 1];
}

// For every run head (its index among all heads is g = hscan - 1): where the run starts inside its
// panel and which row of A it belongs to.  The last element of a panel also closes the panel's
// offsets.
__global__ __launch_bounds__(kBlock) void k_panel_rows(const int32_t *__restrict__ keys, const int32_t *__restrict__ srow,
                                                       const int32_t *__restrict__ head, const int32_t *__restrict__ hscan,
                                                       int32_t nnz, PanelOffsets o, int32_t *__restrict__ crow_ptr,
                                                       int32_t *__restrict__ hrow)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    const int j = keys[i];
    if (head[i]) {
        const int32_t g = hscan[i] - 1;
        crow_ptr[g + j] = (int32_t)(i - o.pstart[j]);
        hrow[g] = srow[i];
    }
    if (i + 1 == o.pstart[j + 1]) crow_ptr[hscan[i] + j] = o.pstart[j + 1] - o.pstart[j];
}

struct PanelBases {
    int32_t kbase[kPanels + 1];
};
// blk_lo[b][j] = index (among all partial sums) of panel j's first partial sum whose row is >= b * kPanelRowBlock
__global__ __launch_bounds__(kBlock) void k_panel_block_offsets(const int32_t *__restrict__ rowid, PanelBases kb,
                                                                int32_t nrb, int32_t *__restrict__ blk_lo)
{
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int j = blockIdx.y;
    if (b > nrb) return;
    const int64_t target = b * kPanelRowBlock;
    int32_t lo = kb.kbase[j], hi = kb.kbase[j + 1];
    while (lo < hi) {
        const int32_t mid = lo + (hi - lo) / 2;
        if (rowid[mid] < target)
            lo = mid + 1;
        else
            hi = mid;
    }
    blk_lo[b * kPanels + j] = lo;
}

void free_panels(PanelMatrix *p)
{
    for (void *q : {(void *)p->col, p->val, (void *)p->row_ptr, (void *)p->seg_row, (void *)p->rowid, (void *)p->blk_lo})
        if (q) (void)hipFree(q);
    p->col = p->row_ptr = p->seg_row = p->rowid = p->blk_lo = nullptr;
    p->val = nullptr;
}

constexpr int kPanelBits = 5;  // radix bits that hold a panel index
static_assert(kPanels <= (1 << kPanelBits), "panel index must fit the sort key bits");

template <typename T>
int build_panels(int32_t m, int32_t n, int32_t nnz, int32_t npanels, const int32_t *row_ptr, const int32_t *col,
                 const T *val, PanelMatrix *out, hipStream_t s)
{
    PanelMatrix pm{};
    if (m <= 0 || nnz <= 0 || n <= 0) return ASX_STATUS_INVALID_SIZE;
    if (npanels < kXcds || npanels > kPanels || npanels % kXcds) return ASX_STATUS_INVALID_VALUE;
    pm.npanels = npanels;
    pm.width = (int32_t)(ceil_div64(ceil_div64(n, npanels), 32) * 32);
    int st = ASX_STATUS_SUCCESS;
    // a..e: five nnz-sized scratch arrays reused through the stages
    int32_t *a = nullptr, *b = nullptr, *c = nullptr, *d = nullptr, *e = nullptr, *d_small = nullptr;
    void *tmp = nullptr;
    size_t tmp_sort = 0, tmp_scan = 0, tmp_bytes = 0;
    PanelOffsets o{};
    PanelBases kb{};
    int32_t h_flag = 0, ktotal = 0;
    const int32_t nrb = (int32_t)ceil_div64(m, kPanelRowBlock);
    const unsigned grid = (unsigned)ceil_div64(nnz, kBlock);
    const size_t nb = sizeof(int32_t) * (size_t)nnz;
#define ASX_TRY(expr)             \
    do {                          \
        st = status_of(expr);     \
        if (st) goto done;        \
    } while (0)
#define ASX_TRY_ST(expr)   \
    do {                   \
        st = (expr);       \
        if (st) goto done; \
    } while (0)
    for (int32_t **q : {&a, &b, &c, &d, &e}) ASX_TRY(hipMalloc((void **)q, nb));
    ASX_TRY(hipMalloc((void **)&d_small, sizeof(int32_t) * (kPanels + 2)));
    ASX_TRY(hipcub::DeviceRadixSort::SortPairs(nullptr, tmp_sort, a, b, c, d, nnz, 0, kPanelBits, s));
    ASX_TRY(hipcub::DeviceScan::InclusiveSum(nullptr, tmp_scan, a, b, nnz, s));
    tmp_bytes = std::max(tmp_sort, tmp_scan);
    ASX_TRY(hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1));

    // 1. elements by panel: b = panel of each sorted element, d = its position in A
    hipLaunchKernelGGL(k_panel_keys, dim3(grid), dim3(kBlock), 0, s, col, nnz, pm.width, a, c);
    ASX_TRY(hipcub::DeviceRadixSort::SortPairs(tmp, tmp_bytes, a, b, c, d, nnz, 0, kPanelBits, s));
    ASX_TRY_ST(launch_offsets_from_sorted(b, nnz, kPanels, d_small, s));
    ASX_TRY(hipMemcpyAsync(o.pstart, d_small, sizeof(o.pstart), hipMemcpyDeviceToHost, s));
    ASX_TRY(hipStreamSynchronize(s));
    for (int j = 0; j < kPanels; ++j) {
        pm.count[j] = o.pstart[j + 1] - o.pstart[j];
        pm.elem_off[j + 1] = pm.elem_off[j] + (int64_t)ceil_div64(pm.count[j], 4) * 4;
        pm.tile_off[j + 1] = pm.tile_off[j] + flat_tiles(pm.count[j]);
        o.elem_off[j] = pm.elem_off[j];
    }
    pm.max_tiles = 0;
    for (int x = 0; x < kXcds; ++x) {
        int32_t tiles = 0;
        for (int j = x; j < kPanels; j += kXcds) tiles += (int32_t)ceil_div64(pm.count[j], kFlatTile);
        if (tiles > pm.max_tiles) pm.max_tiles = tiles;
    }
    o.elem_off[kPanels] = pm.elem_off[kPanels];
    ASX_TRY(hipMalloc((void **)&pm.col, sizeof(int32_t) * (size_t)(pm.elem_off[kPanels] + 4)));
    ASX_TRY(hipMalloc(&pm.val, sizeof(T) * (size_t)(pm.elem_off[kPanels] + 4)));
    // 2. columns and values in panel order; a = row of A of each sorted element
    hipLaunchKernelGGL((k_panel_gather<T>), dim3(grid), dim3(kBlock), 0, s, b, d, nnz, o, row_ptr, m, col, val, pm.col,
                       (T *)pm.val, a);
    // 3. run heads: c = flags, e = their inclusive scan
    hipLaunchKernelGGL(k_panel_heads, dim3(grid), dim3(kBlock), 0, s, b, a, nnz, c);
    ASX_TRY(hipcub::DeviceScan::InclusiveSum(tmp, tmp_bytes, c, e, nnz, s));
    ASX_TRY(hipMemcpyAsync(&ktotal, e + (nnz - 1), sizeof(int32_t), hipMemcpyDeviceToHost, s));
    for (int j = 1; j <= kPanels; ++j) {
        if (o.pstart[j] > 0)
            ASX_TRY(hipMemcpyAsync(&pm.kbase[j], e + (o.pstart[j] - 1), sizeof(int32_t), hipMemcpyDeviceToHost, s));
    }
    ASX_TRY(hipStreamSynchronize(s));
    for (int j = 0; j < kPanels; ++j) pm.krows[j] = pm.kbase[j + 1] - pm.kbase[j];
    ASX_TRY(hipMalloc((void **)&pm.row_ptr, sizeof(int32_t) * ((size_t)ktotal + kPanels)));
    ASX_TRY(hipMalloc((void **)&pm.seg_row, sizeof(int32_t) * (size_t)(pm.tile_off[kPanels] + kPanels)));
    ASX_TRY(hipMalloc((void **)&pm.rowid, sizeof(int32_t) * (size_t)ktotal));
    ASX_TRY(hipMalloc((void **)&pm.blk_lo, sizeof(int32_t) * ((size_t)nrb + 1) * kPanels));
    // panels without elements still need their single offset
    ASX_TRY(hipMemsetAsync(pm.row_ptr, 0, sizeof(int32_t) * ((size_t)ktotal + kPanels), s));
    // 4. compact row offsets per panel and the row of A of each partial sum
    hipLaunchKernelGGL(k_panel_rows, dim3(grid), dim3(kBlock), 0, s, b, a, c, e, nnz, o, pm.row_ptr, pm.rowid);
    // 5. where each block of rows of A starts in each panel's partial sums
    for (int j = 0; j <= kPanels; ++j) kb.kbase[j] = pm.kbase[j];
    hipLaunchKernelGGL(k_panel_block_offsets, dim3((unsigned)ceil_div64((int64_t)nrb + 1, kBlock), kPanels), dim3(kBlock),
                       0, s, pm.rowid, kb, nrb, pm.blk_lo);
    // 6. tiles of each panel
    ASX_TRY(hipMemsetAsync(d_small, 0, sizeof(int32_t), s));
    for (int j = 0; j < kPanels; ++j) {
        const int32_t *rp = pm.row_ptr + pm.kbase[j] + j;
        int32_t *seg = pm.seg_row + pm.tile_off[j] + j;
        ASX_TRY_ST(launch_nnz_split_rows_n(rp, pm.krows[j], flat_tiles(pm.count[j]), kFlatTile, seg, s));
        if (pm.count[j] > 0) ASX_TRY_ST(launch_flat_has_carry(rp, pm.krows[j], pm.count[j], seg, d_small, s));
    }
    ASX_TRY(hipMemcpyAsync(&h_flag, d_small, sizeof(int32_t), hipMemcpyDeviceToHost, s));
    ASX_TRY(hipStreamSynchronize(s));
    pm.carry_pass = h_flag != 0;
#undef ASX_TRY
#undef ASX_TRY_ST
done:
    for (void *p : {(void *)a, (void *)b, (void *)c, (void *)d, (void *)e, (void *)d_small, tmp})
        if (p) (void)hipFree(p);
    if (st) {
        free_panels(&pm);
        return st;
    }
    *out = pm;
    return ASX_STATUS_SUCCESS;
}

template int build_panels<float>(int32_t, int32_t, int32_t, int32_t, const int32_t *, const int32_t *, const float *,
                                 PanelMatrix *, hipStream_t);
template int build_panels<double>(int32_t, int32_t, int32_t, int32_t, const int32_t *, const int32_t *,
                                  const double *, PanelMatrix *, hipStream_t);

}  // namespace asx
