// Measurement probes: the memory-side work of a CSR SpMV without the reduction and without
// the write, to find what the chip can sustain for a given matrix (used by `bench.py --probe`).
//   mode 0: stream col and val only (read-only streaming rate)
//   mode 1: stream col and val and gather x[col] (adds the gather cost of this column pattern)
//   asx_probe_sliced_gather: as mode 1, but every workgroup's gathers are folded into one slice
//   of x, chosen from the workgroup id: shows what a column-panel layout can gain on this chip.
// The result is folded into one value per thread and stored only if it equals an impossible
// constant, so the loads cannot be optimised away and nothing is written.
#include "asx_internal.hpp"

namespace asx {

template <typename T, int MODE>
__global__ __launch_bounds__(kBlock) void k_probe(int64_t nnz, const int32_t *__restrict__ col,
                                                  const T *__restrict__ val, const T *__restrict__ x,
                                                  T *__restrict__ sink)
{
    constexpr int IPT = 8;
    const int64_t base = (int64_t)blockIdx.x * (kBlock * IPT);
    int32_t c[IPT];
    T v[IPT];
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
        const int64_t j = base + threadIdx.x + i * kBlock;
        c[i] = j < nnz ? col[j] : 0;
    }
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
        const int64_t j = base + threadIdx.x + i * kBlock;
        v[i] = j < nnz ? val[j] : T(0);
    }
    T s = T(0);
#pragma unroll
    for (int i = 0; i < IPT; ++i) s += MODE == 1 ? v[i] * x[c[i]] : v[i] * (T)c[i];
    if (s == T(123456.789)) sink[0] = s;
}

// slicing 0: slice = workgroup id mod 8 (8 slices: each XCD gathers from one slice all the time)
//         1: 16 slices, workgroup id mod 8 in the first half of the grid, + 8 in the second half
//         2: 8 slices, slice = (workgroup id / 8) mod 8 (control: every XCD sees every slice)
template <typename T>
__global__ __launch_bounds__(kBlock) void k_probe_sliced(int64_t nnz, int32_t n, int slicing,
                                                         const int32_t *__restrict__ col, const T *__restrict__ val,
                                                         const T *__restrict__ x, T *__restrict__ sink)
{
    constexpr int IPT = 8;
    const int64_t base = (int64_t)blockIdx.x * (kBlock * IPT);
    const int nslices = slicing == 1 ? 16 : 8;
    const int32_t width = n / nslices;
    int slice;
    if (slicing == 0)
        slice = blockIdx.x % 8;
    else if (slicing == 1)
        slice = blockIdx.x % 8 + (blockIdx.x >= gridDim.x / 2 ? 8 : 0);
    else
        slice = (blockIdx.x / 8) % 8;
    int32_t c[IPT];
    T v[IPT];
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
        const int64_t j = base + threadIdx.x + i * kBlock;
        c[i] = j < nnz ? col[j] : 0;
    }
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
        const int64_t j = base + threadIdx.x + i * kBlock;
        v[i] = j < nnz ? val[j] : T(0);
    }
    T s = T(0);
#pragma unroll
    for (int i = 0; i < IPT; ++i) s += v[i] * x[(int64_t)slice * width + c[i] % width];
    if (s == T(123456.789)) sink[0] = s;
}

template <typename T>
int launch_probe(int mode, int64_t nnz, const int32_t *col, const T *val, const T *x, T *sink,
                 hipStream_t s)
{
    if (nnz <= 0) return ASX_STATUS_SUCCESS;
    const unsigned grid = (unsigned)ceil_div64(nnz, kBlock * 8);
    if (mode == 0)
        hipLaunchKernelGGL((k_probe<T, 0>), dim3(grid), dim3(kBlock), 0, s, nnz, col, val, x, sink);
    else
        hipLaunchKernelGGL((k_probe<T, 1>), dim3(grid), dim3(kBlock), 0, s, nnz, col, val, x, sink);
    return check_launch();
}

}  // namespace asx

extern "C" int asx_probe_stream_gather(int value_type, int mode, int64_t nnz, const int32_t *d_col,
                                       const void *d_val, const void *d_x, void *d_sink, void *stream)
{
    if (mode != 0 && mode != 1) return ASX_STATUS_INVALID_VALUE;
    if (nnz < 0) return ASX_STATUS_INVALID_SIZE;
    if (nnz > 0 && (!d_col || !d_val || !d_x || !d_sink)) return ASX_STATUS_INVALID_POINTER;
    if (value_type == ASX_R_64F)
        return asx::launch_probe<double>(mode, nnz, d_col, (const double *)d_val, (const double *)d_x,
                                         (double *)d_sink, (hipStream_t)stream);
    if (value_type == ASX_R_32F)
        return asx::launch_probe<float>(mode, nnz, d_col, (const float *)d_val, (const float *)d_x,
                                        (float *)d_sink, (hipStream_t)stream);
    return ASX_STATUS_NOT_SUPPORTED;
}

extern "C" int asx_probe_sliced_gather(int value_type, int slicing, int64_t nnz, int32_t n, const int32_t *d_col,
                                       const void *d_val, const void *d_x, void *d_sink, void *stream)
{
    if (slicing < 0 || slicing > 2) return ASX_STATUS_INVALID_VALUE;
    if (nnz < 0 || n < 16) return ASX_STATUS_INVALID_SIZE;
    if (nnz > 0 && (!d_col || !d_val || !d_x || !d_sink)) return ASX_STATUS_INVALID_POINTER;
    if (nnz == 0) return ASX_STATUS_SUCCESS;
    const unsigned grid = (unsigned)asx::ceil_div64(nnz, asx::kBlock * 8);
    if (value_type == ASX_R_64F)
        hipLaunchKernelGGL((asx::k_probe_sliced<double>), dim3(grid), dim3(asx::kBlock), 0, (hipStream_t)stream, nnz, n,
                           slicing, d_col, (const double *)d_val, (const double *)d_x, (double *)d_sink);
    else if (value_type == ASX_R_32F)
        hipLaunchKernelGGL((asx::k_probe_sliced<float>), dim3(grid), dim3(asx::kBlock), 0, (hipStream_t)stream, nnz, n,
                           slicing, d_col, (const float *)d_val, (const float *)d_x, (float *)d_sink);
    else
        return ASX_STATUS_NOT_SUPPORTED;
    return asx::check_launch();
}
