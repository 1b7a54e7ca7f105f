// Row-block CSR SpMV with the block's window of x in LDS, for matrices whose rows reach only
// nearby columns (stencils, banded and finite-element matrices).
//
// The row-ordered kernels read 4 bytes of column index per stored element, the row offsets, and
// gather x through the L2 (one request per stored element).  Here the rows are cut, once (plan
// build), into blocks of R consecutive rows whose columns all lie inside a window of at most
// 128 KiB of x; a workgroup copies its window into LDS and streams its block's stored elements as
// tiles of 256 with a 16-bit column-in-window and a "first element of a row" flag per element
// (10 instead of 12.8 bytes per stored element in fp64; no row offsets are read).  Every row owns
// at least one slot (an empty row gets a zero that points at a zero in LDS), so the runs of a
// tile are consecutive rows and a run's sum goes straight to y.  A tile that starts inside a row
// puts that first sum into a carry slot instead, and an ordered pass adds the carries to y
// afterwards (no atomics; results are bit-reproducible).
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

// first and last column of every row (cmin = kNoCol, cmax = -1 for an empty row), its emptiness
__global__ __launch_bounds__(kBlock) void k_window_row_span(const int32_t *__restrict__ row_ptr,
                                                            const int32_t *__restrict__ col, int32_t m,
                                                            int32_t *__restrict__ cmin, int32_t *__restrict__ cmax,
                                                            int32_t *__restrict__ empty)
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
    empty[r] = hi < 0 ? 1 : 0;
}

// bmin / bmax of every block of `rows` rows (bmin preset to kNoCol, bmax to -1)
__global__ __launch_bounds__(kBlock) void k_window_block_span(const int32_t *__restrict__ cmin,
                                                              const int32_t *__restrict__ cmax, int32_t m,
                                                              int32_t rows, int32_t *__restrict__ bmin,
                                                              int32_t *__restrict__ bmax)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= m || cmax[r] < 0) return;
    atomicMin(bmin + r / rows, cmin[r]);
    atomicMax(bmax + r / rows, cmax[r]);
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

// start (in slots, from the start of its block) of row r: stored elements and empty rows before it
__device__ __forceinline__ int32_t window_row_start(const int32_t *__restrict__ row_ptr,
                                                    const int32_t *__restrict__ empties_before, int32_t r0, int32_t r)
{
    return (row_ptr[r] - row_ptr[r0]) + (empties_before[r] - empties_before[r0]);
}

// tiles of every block
__global__ __launch_bounds__(kBlock) void k_window_block_tiles(const int32_t *__restrict__ row_ptr,
                                                               const int32_t *__restrict__ empties_before, int32_t m,
                                                               int32_t rows, int32_t nblocks,
                                                               int32_t *__restrict__ tiles)
{
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const int32_t r0 = (int32_t)(b * rows);
    const int32_t r1 = (int64_t)r0 + rows < m ? r0 + rows : m;
    tiles[b] = (window_row_start(row_ptr, empties_before, r0, r1) + kSlicedTile - 1) / kSlicedTile;
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
                                                         const int32_t *__restrict__ empties_before,
                                                         const int32_t *__restrict__ tile_off,
                                                         const int32_t *__restrict__ bmin, uint16_t *__restrict__ cf,
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
    const int32_t r = lo, b = r / rows, r0 = b * rows;
    const int32_t o = window_row_start(row_ptr, empties_before, r0, r) + (int32_t)(i - row_ptr[r]);
    const int64_t d = (int64_t)tile_off[b] * kSlicedTile + o;
    const bool head = i == row_ptr[r] || o % kSlicedTile == 0;
    cf[d] = (uint16_t)((col[i] - (bmin[b] & ~3)) | (head ? 0x8000 : 0));
    const int64_t phys = d / kSlicedTile * kSlicedTile + tile_val_pos<T>((int)(d % kSlicedTile));
    val_out[phys] = val[i];
    perm[phys] = (int32_t)i;
}

// per tile: the row its first slot belongs to, bit 31 set when the tile starts inside that row
__global__ __launch_bounds__(kBlock) void k_window_tile_words(const int32_t *__restrict__ row_ptr,
                                                              const int32_t *__restrict__ empties_before, int32_t m,
                                                              int32_t rows, int32_t nblocks,
                                                              const int32_t *__restrict__ tile_off, int32_t ntiles,
                                                              int32_t *__restrict__ tile_word, int32_t *__restrict__ any_cont)
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
        if (window_row_start(row_ptr, empties_before, r0, mid) <= o)
            a = mid;
        else
            z = mid - 1;
    }
    const bool cont = window_row_start(row_ptr, empties_before, r0, a) != o;
    tile_word[t] = a | (cont ? (int32_t)0x80000000 : 0);
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
// rank k of a tile is row (first row of the tile) + k; the first sum of a tile that starts inside
// a row goes to the tile's carry slot
template <typename T>
struct StoreRows {
    T *y, *carry_slot;
    int32_t row0, r1;
    bool cont;
    T alpha, beta;
    __device__ __forceinline__ void operator()(int rank, T v) const
    {
        if (rank == 0 && cont) {
            *carry_slot = v;
            return;
        }
        const int64_t r = (int64_t)row0 + rank;
        if (r < r1) y[r] = beta == T(0) ? alpha * v : fma_t<T>(alpha, v, beta * y[r]);
    }
};

template <typename T, int WIDTH, int NW, int D>
__global__ __launch_bounds__(NW *kWave) void k_spmv_window(int32_t n, T alpha, T beta, const int4 *__restrict__ wg_tab,
                                                           const uint16_t *__restrict__ cf, const T *__restrict__ val,
                                                           const int32_t *__restrict__ tile_word,
                                                           const T *__restrict__ x, T *__restrict__ y,
                                                           T *__restrict__ carry)
{
    __shared__ T xs[WIDTH];
    const int4 wg = wg_tab[blockIdx.x];  // window start, first tile, end tile, end row
    const int64_t c0 = wg.x;
    const int32_t cnt = n - c0 < WIDTH ? (int32_t)(n - c0) : WIDTH;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    // the first tiles' loads go out before the window of x is fetched (they do not need it)
    const int32_t last = wg.z - 1;
    Tile<T> tl[D];
    int32_t t = wg.y + wave;
#pragma unroll
    for (int d = 0; d < D; ++d) tile_load<T>(tl[d], t + d * NW < last ? t + d * NW : last, lane, cf, val, tile_word);
    load_x_window<T, WIDTH, NW * kWave>(xs, x, c0, cnt);
    if (threadIdx.x == NW * kWave - 1) xs[WIDTH - 1] = T(0);  // what the slots of empty rows and the padding point at
    __syncthreads();
    while (t < wg.z) {  // uniform over the wave
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int32_t td = t + d * NW;
            if (td < wg.z)
                tile_reduce<T>(tl[d], lane, xs,
                               StoreRows<T>{y, carry + td, tl[d].base & 0x7fffffff, wg.w, tl[d].base < 0, alpha, beta});
            tile_load<T>(tl[d], t + (D + d) * NW < last ? t + (D + d) * NW : last, lane, cf, val, tile_word);
        }
        t += D * NW;
    }
}

// Adds the carries to their rows, in tile order: the thread of the first tile of a run of tiles
// that start inside the same row sums the run's carries and adds the total once.
template <typename T>
__global__ __launch_bounds__(kBlock) void k_window_fixup(int32_t ntiles, T alpha, const int32_t *__restrict__ tile_word,
                                                         const T *__restrict__ carry, T *__restrict__ y)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= ntiles) return;
    const int32_t w = tile_word[t];
    if (w >= 0) return;                         // starts at a row start
    if (t > 0 && tile_word[t - 1] == w) return;  // a later tile of its run
    T s = carry[t];
    for (int64_t j = t + 1; j < ntiles && tile_word[j] == w; ++j) s += carry[j];
    const int32_t r = w & 0x7fffffff;
    y[r] = fma_t<T>(alpha, s, y[r]);
}

}  // namespace

void free_window(WindowMatrix *p)
{
    for (void *q : {p->val, p->carry, (void *)p->cf, (void *)p->perm, (void *)p->tile_word, (void *)p->wg_tab})
        if (q) (void)hipFree(q);
    p->val = p->carry = nullptr;
    p->cf = nullptr;
    p->perm = p->tile_word = p->wg_tab = nullptr;
}

template <typename T>
int build_window(int32_t m, int32_t n, int32_t nnz, int32_t width, int32_t max_rows_per_block, int32_t max_reload,
                 const int32_t *row_ptr, const int32_t *col, const T *val, WindowMatrix *out, hipStream_t s)
{
    WindowMatrix wm{};
    if (m <= 0 || nnz <= 0 || n <= 0) return ASX_STATUS_INVALID_SIZE;
    if (width < 64 || width > 32768) return ASX_STATUS_INVALID_VALUE;
    wm.width = width;
    int st = ASX_STATUS_SUCCESS;
    int32_t *cmin = nullptr, *cmax = nullptr, *empty = nullptr, *ebefore = nullptr;  // m (+1) each
    int32_t *bmin = nullptr, *bmax = nullptr, *btiles = nullptr, *tile_off = nullptr, *d_small = nullptr;
    void *tmp = nullptr;
    size_t tmp_bytes = 0, tb = 0;
    std::vector<int32_t> h_bmin, h_off, tab;
    int64_t slots = 0;
    int32_t h_small[2] = {0, 0};
    const unsigned mgrid = (unsigned)ceil_div64(m, kBlock);
    const int32_t min_blocks = 1024;  // larger blocks only while at least this many row blocks remain
    const int32_t max_nb = (int32_t)ceil_div64(m, 256);
#define ASX_TRY(expr)         \
    do {                      \
        st = status_of(expr); \
        if (st) goto done;    \
    } while (0)
    for (int32_t **q : {&cmin, &cmax, &empty, &ebefore}) ASX_TRY(hipMalloc((void **)q, sizeof(int32_t) * ((size_t)m + 1)));
    for (int32_t **q : {&bmin, &bmax, &btiles, &tile_off}) ASX_TRY(hipMalloc((void **)q, sizeof(int32_t) * ((size_t)max_nb + 1)));
    ASX_TRY(hipMalloc((void **)&d_small, sizeof(int32_t) * 2));
    ASX_TRY(hipcub::DeviceScan::ExclusiveSum(nullptr, tmp_bytes, empty, ebefore, m + 1, s));
    ASX_TRY(hipcub::DeviceScan::ExclusiveSum(nullptr, tb, btiles, tile_off, max_nb + 1, s));
    tmp_bytes = std::max(tmp_bytes, tb);
    ASX_TRY(hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1));

    // 1. column span and emptiness of every row; empty rows before each row
    hipLaunchKernelGGL(k_window_row_span, dim3(mgrid), dim3(kBlock), 0, s, row_ptr, col, m, cmin, cmax, empty);
    ASX_TRY(hipMemsetAsync(empty + m, 0, sizeof(int32_t), s));
    ASX_TRY(hipcub::DeviceScan::ExclusiveSum(tmp, tmp_bytes, empty, ebefore, m + 1, s));

    // 2. the largest block of rows (at most max_rows_per_block, a multiple of 256) whose widest
    //    window fits; the last LDS entry is kept for the zero that empty rows point at
    wm.rows_per_block = 0;
    for (int32_t rows : {8192, 6144, 4096, 3072, 2048, 1536, 1024, 768, 512, 384, 256}) {
        if (rows > max_rows_per_block) continue;
        if (rows > 256 && ceil_div64(m, rows) < min_blocks) continue;  // too few workgroups
        const int32_t nb = (int32_t)ceil_div64(m, rows);
        hipLaunchKernelGGL(k_window_fill_i32, dim3((unsigned)ceil_div64(nb, kBlock)), dim3(kBlock), 0, s, bmin, (int64_t)nb, kNoCol);
        hipLaunchKernelGGL(k_window_fill_i32, dim3((unsigned)ceil_div64(nb, kBlock)), dim3(kBlock), 0, s, bmax, (int64_t)nb, -1);
        ASX_TRY(hipMemsetAsync(d_small, 0, sizeof(int32_t) * 2, s));
        hipLaunchKernelGGL(k_window_block_span, dim3(mgrid), dim3(kBlock), 0, s, cmin, cmax, m, rows, bmin, bmax);
        hipLaunchKernelGGL(k_window_max_span, dim3((unsigned)ceil_div64(nb, kBlock)), dim3(kBlock), 0, s, bmin, bmax, nb, d_small);
        ASX_TRY(hipMemcpyAsync(h_small, d_small, sizeof(int32_t), hipMemcpyDeviceToHost, s));
        ASX_TRY(hipStreamSynchronize(s));
        if (h_small[0] <= width - 1) {
            // every workgroup fetches its whole window: with a bound on that (max_reload > 0), blocks
            // whose window is more than max_reload times their rows wide are turned down
            if (max_reload <= 0 || h_small[0] <= (int64_t)max_reload * rows) {
                wm.rows_per_block = rows;
                wm.nblocks = nb;
            }
            break;
        }
    }
    if (wm.rows_per_block == 0) {
        st = ASX_STATUS_NOT_SUPPORTED;  // some 256 rows reach further than a window: not this kernel's matrix
        goto done;
    }
    // 3. tiles of every block
    hipLaunchKernelGGL(k_window_block_tiles, dim3((unsigned)ceil_div64(wm.nblocks, kBlock)), dim3(kBlock), 0, s, row_ptr,
                       ebefore, m, wm.rows_per_block, wm.nblocks, btiles);
    ASX_TRY(hipMemsetAsync(btiles + wm.nblocks, 0, sizeof(int32_t), s));
    ASX_TRY(hipcub::DeviceScan::ExclusiveSum(tmp, tmp_bytes, btiles, tile_off, wm.nblocks + 1, s));
    h_bmin.resize((size_t)wm.nblocks);
    h_off.resize((size_t)wm.nblocks + 1);
    ASX_TRY(hipMemcpyAsync(h_bmin.data(), bmin, sizeof(int32_t) * h_bmin.size(), hipMemcpyDeviceToHost, s));
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
    ASX_TRY(hipMalloc((void **)&wm.tile_word, sizeof(int32_t) * (size_t)wm.ntiles));
    ASX_TRY(hipMalloc(&wm.carry, sizeof(T) * (size_t)wm.ntiles));
    ASX_TRY(hipMemsetAsync(wm.carry, 0, sizeof(T) * (size_t)wm.ntiles, s));
    // 4. every slot starts as a zero that points at the zero in LDS and opens a row of its own (the
    //    slots of empty rows and the padding behind a block's last row stay that way)
    hipLaunchKernelGGL((k_window_fill_pads<T>), dim3((unsigned)ceil_div64(slots, kBlock)), dim3(kBlock), 0, s, slots,
                       (uint16_t)(0x8000 | (width - 1)), wm.cf, (T *)wm.val, wm.perm);
    hipLaunchKernelGGL((k_window_place<T>), dim3((unsigned)ceil_div64(nnz, kBlock)), dim3(kBlock), 0, s, row_ptr, col, val,
                       m, nnz, wm.rows_per_block, ebefore, tile_off, bmin, wm.cf, (T *)wm.val, wm.perm);
    // 5. first row of every tile
    ASX_TRY(hipMemsetAsync(d_small, 0, sizeof(int32_t) * 2, s));
    hipLaunchKernelGGL(k_window_tile_words, dim3((unsigned)ceil_div64(wm.ntiles, kBlock)), dim3(kBlock), 0, s, row_ptr,
                       ebefore, m, wm.rows_per_block, wm.nblocks, tile_off, wm.ntiles, wm.tile_word, d_small);
    ASX_TRY(hipMemcpyAsync(h_small, d_small, sizeof(int32_t), hipMemcpyDeviceToHost, s));
    // 6. one workgroup per block: window start, tiles, end row
    tab.resize((size_t)wm.nblocks * 4);
    for (int32_t b = 0; b < wm.nblocks; ++b) {
        const int64_t r1 = std::min<int64_t>(m, ((int64_t)b + 1) * wm.rows_per_block);
        tab[(size_t)b * 4 + 0] = h_bmin[(size_t)b] == kNoCol ? 0 : (h_bmin[(size_t)b] & ~3);
        tab[(size_t)b * 4 + 1] = h_off[(size_t)b];
        tab[(size_t)b * 4 + 2] = h_off[(size_t)b + 1];
        tab[(size_t)b * 4 + 3] = (int32_t)r1;
    }
    ASX_TRY(hipMalloc((void **)&wm.wg_tab, sizeof(int32_t) * tab.size()));
    ASX_TRY(hipMemcpyAsync(wm.wg_tab, tab.data(), sizeof(int32_t) * tab.size(), hipMemcpyHostToDevice, s));
    ASX_TRY(hipStreamSynchronize(s));
    ASX_TRY(hipGetLastError());
    wm.has_carry = h_small[0] != 0;
#undef ASX_TRY
done:
    for (void *p : {(void *)cmin, (void *)cmax, (void *)empty, (void *)ebefore, (void *)bmin, (void *)bmax, (void *)btiles,
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
#define ASX_WIN(W)                                                                                                  \
    hipLaunchKernelGGL((k_spmv_window<T, W, 16, 2>), dim3((unsigned)wm->nblocks), dim3(16 * kWave), 0, s, n, alpha, beta, \
                       reinterpret_cast<const int4 *>(wm->wg_tab), wm->cf, (const T *)wm->val, wm->tile_word, x, y,     \
                       (T *)wm->carry)
    if (wm->width == (int)(131072 / sizeof(T)))
        ASX_WIN(131072 / sizeof(T));
    else if (wm->width == (int)(81920 / sizeof(T)))
        ASX_WIN(81920 / sizeof(T));
    else if (sizeof(T) == 8 && wm->width == 20480)
        ASX_WIN(20480);
    else
        return ASX_STATUS_INVALID_VALUE;
#undef ASX_WIN
    if (wm->has_carry)
        hipLaunchKernelGGL((k_window_fixup<T>), dim3((unsigned)ceil_div64(wm->ntiles, kBlock)), dim3(kBlock), 0, s,
                           wm->ntiles, alpha, wm->tile_word, (const T *)wm->carry, y);
    return check_launch();
}

#define ASX_INST(T)                                                                                               \
    template int build_window<T>(int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, const int32_t *,         \
                                 const int32_t *, const T *, WindowMatrix *, hipStream_t);                                        \
    template int window_update_values<T>(const WindowMatrix *, const T *, hipStream_t);                           \
    template int launch_spmv_window<T>(int32_t, int32_t, T, const WindowMatrix *, const T *, T, T *, hipStream_t);
ASX_INST(float)
ASX_INST(double)
#undef ASX_INST

}  // namespace asx
