// Exclusive prefix sum of int32 arrays on the device, for the plan builders: three launches (sums
// of blocks of 4096, scan of those sums by one workgroup, scan inside every block plus its
// offset).  The arrays scanned here are per-tile, per-block or per-(slice, block) counts, a few MB
// at most: two passes over them cost microseconds.
#pragma once
#include "asx_internal.hpp"

namespace asx {

constexpr int kScanThreads = 256;
constexpr int kScanPerThread = 16;
constexpr int kScanBlock = kScanThreads * kScanPerThread;

// sum over the workgroup; every thread receives the total (barriers inside)
__device__ __forceinline__ int32_t scan_block_total(int32_t v, int32_t *wave_tot)
{
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) v += __shfl_xor(v, d, kWave);
    if (lane == 0) wave_tot[wave] = v;
    __syncthreads();
    int32_t t = 0;
    for (int w = 0; w < kScanThreads / kWave; ++w) t += wave_tot[w];
    __syncthreads();
    return t;
}

// exclusive sum of one value per thread over the workgroup (barriers inside)
__device__ __forceinline__ int32_t scan_block_exclusive(int32_t v, int32_t *wave_tot, int32_t *total)
{
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    int32_t incl = v;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int32_t t = __shfl_up(incl, d, kWave);
        if (lane >= d) incl += t;
    }
    if (lane == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    int32_t before = 0, all = 0;
    for (int w = 0; w < kScanThreads / kWave; ++w) {
        const int32_t t = wave_tot[w];
        before += w < wave ? t : 0;
        all += t;
    }
    __syncthreads();
    *total = all;
    return before + incl - v;
}

static __global__ __launch_bounds__(kScanThreads) void k_scan_block_sums(const int32_t *__restrict__ in, int64_t n,
                                                                          int32_t *__restrict__ sums)
{
    __shared__ int32_t wave_tot[kScanThreads / kWave];
    const int64_t base = (int64_t)blockIdx.x * kScanBlock;
    int32_t v = 0;
#pragma unroll
    for (int k = 0; k < kScanPerThread; ++k) {
        const int64_t i = base + k * kScanThreads + threadIdx.x;
        v += i < n ? in[i] : 0;
    }
    const int32_t t = scan_block_total(v, wave_tot);
    if (threadIdx.x == 0) sums[blockIdx.x] = t;
}

// in-place exclusive scan of sums[0 .. nb) by one workgroup, kScanThreads at a time
static __global__ __launch_bounds__(kScanThreads) void k_scan_sums(int32_t *__restrict__ sums, int32_t nb)
{
    __shared__ int32_t wave_tot[kScanThreads / kWave];
    int32_t carry = 0;
    for (int32_t i0 = 0; i0 < nb; i0 += kScanThreads) {  // uniform
        const int32_t i = i0 + threadIdx.x;
        const int32_t v = i < nb ? sums[i] : 0;
        int32_t total;
        const int32_t e = scan_block_exclusive(v, wave_tot, &total);
        if (i < nb) sums[i] = carry + e;
        carry += total;
    }
}

// out[i] = sums[block] + sum of in[block start .. i); a thread owns kScanPerThread consecutive items
static __global__ __launch_bounds__(kScanThreads) void k_scan_apply(const int32_t *__restrict__ in, int64_t n,
                                                                     const int32_t *__restrict__ sums,
                                                                     int32_t *__restrict__ out)
{
    __shared__ int32_t wave_tot[kScanThreads / kWave];
    const int64_t base = (int64_t)blockIdx.x * kScanBlock + (int64_t)threadIdx.x * kScanPerThread;
    int32_t v[kScanPerThread];
    int32_t mine = 0;
#pragma unroll
    for (int k = 0; k < kScanPerThread; ++k) {
        v[k] = base + k < n ? in[base + k] : 0;
        mine += v[k];
    }
    int32_t total;
    int32_t run = sums[blockIdx.x] + scan_block_exclusive(mine, wave_tot, &total);
#pragma unroll
    for (int k = 0; k < kScanPerThread; ++k) {
        if (base + k < n) out[base + k] = run;
        run += v[k];
    }
}

// ints of scratch the scan of n items needs
inline size_t scan_scratch_ints(int64_t n) { return (size_t)ceil_div64(n > 0 ? n : 1, kScanBlock); }

// out[i] = in[0] + ... + in[i - 1], i in [0, n); in == out is allowed; `scratch`: scan_scratch_ints(n) ints
inline int launch_exclusive_scan_i32(const int32_t *in, int32_t *out, int64_t n, int32_t *scratch, hipStream_t s)
{
    if (n <= 0) return ASX_STATUS_SUCCESS;
    const int64_t nb = ceil_div64(n, kScanBlock);
    if (nb > 0x7fffffff) return ASX_STATUS_INVALID_SIZE;
    hipLaunchKernelGGL(k_scan_block_sums, dim3((unsigned)nb), dim3(kScanThreads), 0, s, in, n, scratch);
    hipLaunchKernelGGL(k_scan_sums, dim3(1), dim3(kScanThreads), 0, s, scratch, (int32_t)nb);
    hipLaunchKernelGGL(k_scan_apply, dim3((unsigned)nb), dim3(kScanThreads), 0, s, in, n, scratch, out);
    return check_launch();
}

}  // namespace asx
