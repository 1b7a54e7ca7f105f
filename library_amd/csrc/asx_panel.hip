// Builds the column-panel copy of a CSR matrix for the panel SpMV kernel (device side, once per
// plan): a stable radix sort of the stored elements by panel keeps CSR order inside each panel,
// so every panel is itself a CSR matrix over all m rows; its row offsets come from binary
// searches of the original row offsets in the sorted element positions.
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

template <typename T>
__global__ __launch_bounds__(kBlock) void k_panel_gather(const int32_t *__restrict__ keys, const int32_t *__restrict__ idx,
                                                         int32_t nnz, PanelOffsets o, const int32_t *__restrict__ col,
                                                         const T *__restrict__ val, int32_t *__restrict__ col_out,
                                                         T *__restrict__ val_out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nnz) return;
    const int j = keys[i];
    const int64_t dst = o.elem_off[j] + (i - o.pstart[j]);
    const int32_t src = idx[i];
    col_out[dst] = col[src];
    val_out[dst] = val[src];
}

// row_ptr_out[j][r] = number of panel-j elements whose original position is below row_ptr[r]
__global__ __launch_bounds__(kBlock) void k_panel_row_ptr(const int32_t *__restrict__ idx, PanelOffsets o,
                                                          const int32_t *__restrict__ row_ptr, int32_t m,
                                                          int32_t *__restrict__ row_ptr_out)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int j = blockIdx.y;
    if (r > m) return;
    const int32_t *p = idx + o.pstart[j];
    const int32_t target = row_ptr[r];
    int32_t lo = 0, hi = o.pstart[j + 1] - o.pstart[j];
    while (lo < hi) {
        const int32_t mid = (lo + hi) / 2;
        if (p[mid] < target)
            lo = mid + 1;
        else
            hi = mid;
    }
    row_ptr_out[(int64_t)j * (m + 1) + r] = lo;
}

void free_panels(PanelMatrix *p)
{
    for (void *q : {(void *)p->col, p->val, (void *)p->row_ptr, (void *)p->seg_row})
        if (q) (void)hipFree(q);
    p->col = p->row_ptr = p->seg_row = nullptr;
    p->val = nullptr;
}

template <typename T>
int build_panels(int32_t m, int32_t n, int32_t nnz, const int32_t *row_ptr, const int32_t *col, const T *val,
                 PanelMatrix *out, hipStream_t s)
{
    PanelMatrix pm{};
    if (m <= 0 || nnz <= 0 || n < kPanels) return ASX_STATUS_INVALID_SIZE;
    pm.width = (int32_t)(ceil_div64(ceil_div64(n, kPanels), 32) * 32);
    int st = ASX_STATUS_SUCCESS;
    int32_t *keys = nullptr, *keys2 = nullptr, *idx = nullptr, *idx2 = nullptr, *d_pstart = nullptr, *d_flag = nullptr;
    void *tmp = nullptr;
    size_t tmp_bytes = 0;
    PanelOffsets o{};
    int32_t h_flag = 0;
    const unsigned grid = (unsigned)ceil_div64(nnz, kBlock);
#define ASX_TRY(expr)             \
    do {                          \
        st = status_of(expr);     \
        if (st) goto done;        \
    } while (0)
#define ASX_TRY_ST(expr) \
    do {                 \
        st = (expr);     \
        if (st) goto done; \
    } while (0)
    ASX_TRY(hipMalloc((void **)&keys, sizeof(int32_t) * (size_t)nnz));
    ASX_TRY(hipMalloc((void **)&keys2, sizeof(int32_t) * (size_t)nnz));
    ASX_TRY(hipMalloc((void **)&idx, sizeof(int32_t) * (size_t)nnz));
    ASX_TRY(hipMalloc((void **)&idx2, sizeof(int32_t) * (size_t)nnz));
    ASX_TRY(hipMalloc((void **)&d_pstart, sizeof(int32_t) * (kPanels + 1)));
    ASX_TRY(hipMalloc((void **)&d_flag, sizeof(int32_t)));
    ASX_TRY(hipcub::DeviceRadixSort::SortPairs(nullptr, tmp_bytes, keys, keys2, idx, idx2, nnz, 0, 3, s));
    ASX_TRY(hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1));
    hipLaunchKernelGGL(k_panel_keys, dim3(grid), dim3(kBlock), 0, s, col, nnz, pm.width, keys, idx);
    ASX_TRY(hipcub::DeviceRadixSort::SortPairs(tmp, tmp_bytes, keys, keys2, idx, idx2, nnz, 0, 3, s));
    ASX_TRY_ST(launch_offsets_from_sorted(keys2, nnz, kPanels, d_pstart, s));
    ASX_TRY(hipMemcpyAsync(o.pstart, d_pstart, sizeof(o.pstart), hipMemcpyDeviceToHost, s));
    ASX_TRY(hipStreamSynchronize(s));
    pm.max_tiles = 0;
    for (int j = 0; j < kPanels; ++j) {
        pm.count[j] = o.pstart[j + 1] - o.pstart[j];
        pm.elem_off[j + 1] = pm.elem_off[j] + (int64_t)ceil_div64(pm.count[j], 4) * 4;
        const int32_t tiles = flat_tiles(pm.count[j]);
        pm.tile_off[j + 1] = pm.tile_off[j] + tiles;
        if (pm.count[j] > 0 && tiles > pm.max_tiles) pm.max_tiles = tiles;
        o.elem_off[j] = pm.elem_off[j];
    }
    o.elem_off[kPanels] = pm.elem_off[kPanels];
    ASX_TRY(hipMalloc((void **)&pm.col, sizeof(int32_t) * (size_t)(pm.elem_off[kPanels] + 4)));
    ASX_TRY(hipMalloc(&pm.val, sizeof(T) * (size_t)(pm.elem_off[kPanels] + 4)));
    ASX_TRY(hipMalloc((void **)&pm.row_ptr, sizeof(int32_t) * (size_t)kPanels * ((size_t)m + 1)));
    ASX_TRY(hipMalloc((void **)&pm.seg_row, sizeof(int32_t) * (size_t)(pm.tile_off[kPanels] + kPanels)));
    hipLaunchKernelGGL((k_panel_gather<T>), dim3(grid), dim3(kBlock), 0, s, keys2, idx2, nnz, o, col, val, pm.col,
                       (T *)pm.val);
    hipLaunchKernelGGL(k_panel_row_ptr, dim3((unsigned)ceil_div64((int64_t)m + 1, kBlock), kPanels), dim3(kBlock), 0, s,
                       idx2, o, row_ptr, m, pm.row_ptr);
    ASX_TRY(hipGetLastError());
    ASX_TRY(hipMemsetAsync(d_flag, 0, sizeof(int32_t), s));
    for (int j = 0; j < kPanels; ++j) {
        const int32_t *rp = pm.row_ptr + (int64_t)j * (m + 1);
        int32_t *seg = pm.seg_row + pm.tile_off[j] + j;
        ASX_TRY_ST(launch_nnz_split_rows_n(rp, m, flat_tiles(pm.count[j]), kFlatTile, seg, s));
        if (pm.count[j] > 0) ASX_TRY_ST(launch_flat_has_carry(rp, m, pm.count[j], seg, d_flag, s));
    }
    ASX_TRY(hipMemcpyAsync(&h_flag, d_flag, sizeof(int32_t), hipMemcpyDeviceToHost, s));
    ASX_TRY(hipStreamSynchronize(s));
    pm.carry_pass = h_flag != 0;
#undef ASX_TRY
#undef ASX_TRY_ST
done:
    for (void *p : {(void *)keys, (void *)keys2, (void *)idx, (void *)idx2, (void *)d_pstart, (void *)d_flag, tmp})
        if (p) (void)hipFree(p);
    if (st) {
        free_panels(&pm);
        return st;
    }
    *out = pm;
    return ASX_STATUS_SUCCESS;
}

template int build_panels<float>(int32_t, int32_t, int32_t, const int32_t *, const int32_t *, const float *,
                                 PanelMatrix *, hipStream_t);
template int build_panels<double>(int32_t, int32_t, int32_t, const int32_t *, const int32_t *, const double *,
                                  PanelMatrix *, hipStream_t);

}  // namespace asx
