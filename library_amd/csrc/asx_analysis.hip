// CSR analysis kernels for gfx950: row-length histogram, row partitions, nnz-split rows,
// merge-path split points.  All outputs are integers and are defined to be bit-identical to
// the reference functions cited at each launcher (and in include/alphasparse_amd.h).
// One thread per output element; every search is a binary search over row_ptr in global
// memory (row_ptr is small next to the matrix and stays in L2 across the searches).
#include <algorithm>

#include "asx_internal.hpp"

namespace asx {

// -------------------------------------------------------------------------------------------
// Row-length histogram: 33 log2 bins + max + the three find_rows bins
// (hip/kernel/level2/alphasparse_spmv_csr_adaptive2.h:5-47: len < 2, len < 1024, else).
// -------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_zero_i64(int64_t *p, int n)
{
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

__global__ __launch_bounds__(256) void k_row_histogram(const int32_t *__restrict__ row_ptr, int32_t m,
                                                       unsigned long long *hist /*33*/,
                                                       unsigned long long *stats /*4*/)
{
    __shared__ unsigned int s_hist[33];
    __shared__ unsigned int s_bins[3];
    __shared__ int s_max;
    if (threadIdx.x < 33) s_hist[threadIdx.x] = 0;
    if (threadIdx.x < 3) s_bins[threadIdx.x] = 0;
    if (threadIdx.x == 0) s_max = 0;
    __syncthreads();
    int local_max = 0;
    const int lane = threadIdx.x & (kWave - 1);
    for (int64_t r0 = (int64_t)blockIdx.x * blockDim.x; r0 < m; r0 += (int64_t)gridDim.x * blockDim.x) {  // uniform
        const int64_t r = r0 + threadIdx.x;
        const bool valid = r < m;
        const int len = valid ? row_ptr[r + 1] - row_ptr[r] : 0;
        const int bin = len <= 0 ? 0 : 32 - __clz(len);
        // one LDS atomic per distinct bin among the wave's 64 rows (rows of one length would
        // otherwise serialise 64 atomics on one address)
        unsigned long long todo = __ballot(valid);
        while (todo) {  // uniform
            const int first = __builtin_ctzll(todo);
            const int b = __builtin_amdgcn_readlane(bin, first);
            const unsigned long long same = __ballot(valid && bin == b);
            if (lane == first) atomicAdd(&s_hist[b], (unsigned int)__popcll(same));
            todo &= ~same;
        }
        const unsigned int c0 = __popcll(__ballot(valid && len < 2)), c1 = __popcll(__ballot(valid && len >= 2 && len < 1024));
        const unsigned int c2 = __popcll(__ballot(valid && len >= 1024));
        if (lane == 0) {
            if (c0) atomicAdd(&s_bins[0], c0);
            if (c1) atomicAdd(&s_bins[1], c1);
            if (c2) atomicAdd(&s_bins[2], c2);
        }
        local_max = len > local_max ? len : local_max;
    }
    atomicMax(&s_max, local_max);
    __syncthreads();
    if (threadIdx.x < 33 && s_hist[threadIdx.x])
        atomicAdd(&hist[threadIdx.x], (unsigned long long)s_hist[threadIdx.x]);
    if (threadIdx.x < 3 && s_bins[threadIdx.x])
        atomicAdd(&stats[1 + threadIdx.x], (unsigned long long)s_bins[threadIdx.x]);
    if (threadIdx.x == 0) atomicMax(&stats[0], (unsigned long long)s_max);
}

int launch_row_histogram(const int32_t *d_row_ptr, int32_t m, int64_t *d_hist, int64_t *d_stats,
                         hipStream_t s)
{
    // counters are cleared with a kernel (not a memset node) so the call can sit in a graph
    hipLaunchKernelGGL(k_zero_i64, dim3(1), dim3(256), 0, s, d_hist, 33);
    hipLaunchKernelGGL(k_zero_i64, dim3(1), dim3(256), 0, s, d_stats, 4);
    if (m > 0) {
        int grid = (int)ceil_div64(m, 256 * 8);
        if (grid > 4096) grid = 4096;
        hipLaunchKernelGGL(k_row_histogram, dim3(grid), dim3(256), 0, s, d_row_ptr, m,
                           (unsigned long long *)d_hist, (unsigned long long *)d_stats);
    }
    return check_launch();
}

// -------------------------------------------------------------------------------------------
// hygon/util/partition.cpp:83-96: partition[i] = first p in [0, m-1) with row_end[p] >= ave*i,
// or m-1 when there is none; ave = nnz / nparts in 32-bit integer arithmetic.
// -------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_partition_rows_by_nnz(const int32_t *__restrict__ row_ptr,
                                                               int32_t m, int32_t nparts,
                                                               int32_t *__restrict__ out)
{
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i > nparts) return;
    if (i == 0) {
        out[0] = 0;
        return;
    }
    if (i == nparts) {
        out[nparts] = m;
        return;
    }
    const int32_t *row_end = row_ptr + 1;
    int32_t nnz = row_end[m - 1];
    int32_t ave = nnz / nparts;
    int32_t target = (int32_t)((uint32_t)ave * (uint32_t)i);  // wraps as the 32-bit product does
    int32_t lo = 0, hi = m - 1;
    while (lo < hi) {
        int32_t mid = (lo + hi) / 2;
        if (row_end[mid] < target)
            lo = mid + 1;
        else
            hi = mid;
    }
    out[i] = lo;
}

int launch_partition_rows_by_nnz(const int32_t *d_row_ptr, int32_t m, int32_t nparts, int32_t *d_out,
                                 hipStream_t s)
{
    int grid = (int)ceil_div64((int64_t)nparts + 1, 256);
    hipLaunchKernelGGL(k_partition_rows_by_nnz, dim3(grid), dim3(256), 0, s, d_row_ptr, m, nparts,
                       d_out);
    return check_launch();
}

// -------------------------------------------------------------------------------------------
// Row holding stored element t*items (largest r with row_ptr[r] <= t*items); out[nseg] = m.
// hip/kernel/level3/alphasparse_spmm_csr_nnz_split.h:7-47 reaches the same row through a
// two-level search; hip/kernel/level2/alphasparse_spmv_csr_flat.h:7-38 through one.
// -------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_nnz_split_rows(const int32_t *__restrict__ row_ptr, int32_t m,
                                                        int32_t nseg, int32_t items,
                                                        int32_t *__restrict__ out)
{
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t > nseg) return;
    if (t == nseg) {
        out[nseg] = m;
        return;
    }
    int64_t e = t * items;
    int32_t lo = 0, hi = m;  // invariant row_ptr[lo] <= e
    while (lo < hi) {
        int32_t mid = lo + (hi - lo + 1) / 2;
        if ((int64_t)row_ptr[mid] <= e)
            lo = mid;
        else
            hi = mid - 1;
    }
    out[t] = lo;
}

// same kernel for a caller-chosen segment count (nseg >= ceil(nnz/items))
int launch_nnz_split_rows_n(const int32_t *d_row_ptr, int32_t m, int32_t nseg, int32_t items, int32_t *d_out,
                            hipStream_t s)
{
    int grid = (int)ceil_div64((int64_t)nseg + 1, 256);
    hipLaunchKernelGGL(k_nnz_split_rows, dim3(grid), dim3(256), 0, s, d_row_ptr, m, nseg, items, d_out);
    return check_launch();
}

int launch_nnz_split_rows(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t items,
                          int32_t *d_out, hipStream_t s)
{
    int32_t nseg = (int32_t)ceil_div64(nnz, items);
    int grid = (int)ceil_div64((int64_t)nseg + 1, 256);
    hipLaunchKernelGGL(k_nnz_split_rows, dim3(grid), dim3(256), 0, s, d_row_ptr, m, nseg, items, d_out);
    return check_launch();
}

// -------------------------------------------------------------------------------------------
// Merge-path split points (hip/kernel/level2/alphasparse_spmv_csr_merge_ginkgo.h:10-33,132-157):
// diagonal d = min(g*items, m+nnz); x = least p in [max(d-nnz,0), min(d,m)] with
// row_end[p] >= d-p (else the window's upper end); y = d-x.
// -------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_merge_path_search(const int32_t *__restrict__ row_ptr,
                                                           int32_t m, int32_t nnz, int32_t items,
                                                           int32_t nblk, int32_t *__restrict__ xs,
                                                           int32_t *__restrict__ ys)
{
    int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g > nblk) return;
    const int32_t *row_end = row_ptr + 1;
    int64_t total = (int64_t)m + nnz;
    int64_t d = g * items;
    if (d > total) d = total;
    int64_t lo = d - nnz > 0 ? d - nnz : 0;
    int64_t hi = d < m ? d : m;
    while (lo < hi) {
        int64_t p = (lo + hi) / 2;
        if ((int64_t)row_end[p] < d - p)
            lo = p + 1;
        else
            hi = p;
    }
    xs[g] = (int32_t)lo;
    ys[g] = (int32_t)(d - lo);
}

int launch_merge_path_search(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t items,
                             int32_t *d_xs, int32_t *d_ys, hipStream_t s)
{
    int32_t nblk = (int32_t)ceil_div64((int64_t)m + nnz, items);
    int grid = (int)ceil_div64((int64_t)nblk + 1, 256);
    hipLaunchKernelGGL(k_merge_path_search, dim3(grid), dim3(256), 0, s, d_row_ptr, m, nnz, items, nblk,
                       d_xs, d_ys);
    return check_launch();
}

// -------------------------------------------------------------------------------------------
// hip/kernel/level2/alphasparse_spmv_csr_row_partition_ginkgo.h:15-42 as launched at :419-424:
// closed-range search over acc = row_ptr+1, indices [0, m-1]; the answer may be m.
// -------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_loadbalance_partition(const int32_t *__restrict__ row_ptr,
                                                               int32_t m, int64_t ave,
                                                               int32_t warp_size, int32_t nwarps,
                                                               int32_t *__restrict__ out)
{
    int g = blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= nwarps) return;
    const int32_t *acc = row_ptr + 1;
    int64_t target = ave * g;
    int32_t l = 0, r = m - 1;
    while (l <= r) {
        int32_t mid = (l + r) / 2;
        int64_t chunks = ((int64_t)acc[mid] + warp_size - 1) / warp_size;
        if (chunks * nwarps < target)
            l = mid + 1;
        else
            r = mid - 1;
    }
    out[g] = l;
}

int launch_loadbalance_partition(const int32_t *d_row_ptr, int32_t m, int32_t nnz, int32_t warp_size,
                                 int32_t nwarps, int32_t *d_out, hipStream_t s)
{
    if (nwarps <= 0) return ASX_STATUS_SUCCESS;
    int64_t ave = ceil_div64(nnz, warp_size);
    int grid = (int)ceil_div64(nwarps, 256);
    hipLaunchKernelGGL(k_loadbalance_partition, dim3(grid), dim3(256), 0, s, d_row_ptr, m, ave,
                       warp_size, nwarps, d_out);
    return check_launch();
}

// -------------------------------------------------------------------------------------------
// Calibration copy: four 16-byte non-temporal loads in flight per lane, then four non-temporal
// stores, grid-stride.
// -------------------------------------------------------------------------------------------
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void k_copy16(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, size_t n16)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i + 3 * stride < n16; i += 4 * stride) {
        const u32x4 a = __builtin_nontemporal_load(src + i), b = __builtin_nontemporal_load(src + i + stride),
                    c = __builtin_nontemporal_load(src + i + 2 * stride),
                    d = __builtin_nontemporal_load(src + i + 3 * stride);
        __builtin_nontemporal_store(a, dst + i);
        __builtin_nontemporal_store(b, dst + i + stride);
        __builtin_nontemporal_store(c, dst + i + 2 * stride);
        __builtin_nontemporal_store(d, dst + i + 3 * stride);
    }
    for (; i < n16; i += stride) dst[i] = src[i];
}

// A sample of the columns: `samples` tiles of 1024 consecutive stored elements, `stride` elements
// apart, one workgroup each.  out[t] = number of distinct 128-byte lines of x the tile's columns
// touch (col >> shift entered into a hash table in LDS: 4096 slots, linear probing).  With
// row_ptr given also out[64 + t] = number of (row, slice) pairs among the tile's elements, slices
// of `width` columns: an element opens a pair when it is the first of its row (or of the tile) or
// lies in another slice than the element before it (columns ascend inside a row).
__global__ __launch_bounds__(kBlock) void k_sample_columns(const int32_t *__restrict__ col, int64_t stride, int shift,
                                                           const int32_t *__restrict__ row_ptr, int32_t m, int32_t width,
                                                           int32_t *__restrict__ out)
{
    constexpr int kSlots = 4096;
    __shared__ int32_t table[kSlots];
    __shared__ int32_t count, pairs;
    for (int i = threadIdx.x; i < kSlots; i += kBlock) table[i] = -1;
    if (threadIdx.x == 0) count = 0, pairs = 0;
    __syncthreads();
    const int64_t first = (int64_t)blockIdx.x * stride;
    const int32_t *from = col + first;
    int32_t mine = 0, mine_pairs = 0;
    for (int i = threadIdx.x; i < kFlatTile; i += kBlock) {
        const int32_t c = from[i];
        const int32_t v = c >> shift;
        uint32_t h = ((uint32_t)v * 2654435761u) >> 20;
        for (;;) {
            const int32_t old = atomicCAS(&table[h], -1, v);
            if (old == -1) {
                ++mine;
                break;
            }
            if (old == v) break;
            h = (h + 1) & (kSlots - 1);
        }
        if (row_ptr) {
            bool opens = i == 0 || c / width != from[i - 1] / width;
            if (!opens) {  // first element of its row?
                const int64_t e = first + i;
                int32_t lo = 0, hi = m;  // largest r with row_ptr[r] <= e
                while (lo < hi) {
                    const int32_t mid = lo + (hi - lo + 1) / 2;
                    if ((int64_t)row_ptr[mid] <= e)
                        lo = mid;
                    else
                        hi = mid - 1;
                }
                opens = row_ptr[lo] == e;
            }
            mine_pairs += opens;
        }
    }
    if (mine) atomicAdd(&count, mine);
    if (mine_pairs) atomicAdd(&pairs, mine_pairs);
    __syncthreads();
    if (threadIdx.x == 0) {
        out[blockIdx.x] = count;
        if (row_ptr) out[64 + blockIdx.x] = pairs;
    }
}
int launch_sample_columns(const int32_t *d_col, int64_t stride, int shift, const int32_t *d_row_ptr, int32_t m,
                          int32_t width, int32_t samples, int32_t *d_out, hipStream_t s)
{
    if (samples <= 0 || samples > 64) return samples > 64 ? ASX_STATUS_INVALID_VALUE : ASX_STATUS_SUCCESS;
    hipLaunchKernelGGL(k_sample_columns, dim3((unsigned)samples), dim3(kBlock), 0, s, d_col, stride, shift, d_row_ptr, m, width,
                       d_out);
    return check_launch();
}

__global__ __launch_bounds__(kBlock) void k_fill_i32(int32_t *__restrict__ p, int64_t n, int32_t v)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}
int launch_fill_i32(int32_t *d_dst, int64_t n, int32_t value, hipStream_t s)
{
    if (n <= 0) return ASX_STATUS_SUCCESS;
    hipLaunchKernelGGL(k_fill_i32, dim3((unsigned)ceil_div64(n, kBlock)), dim3(kBlock), 0, s, d_dst, n, value);
    return check_launch();
}

int launch_copy_bytes(const void *d_src, void *d_dst, size_t bytes, hipStream_t s)
{
    size_t n16 = bytes / 16;
    if (n16 == 0) return ASX_STATUS_SUCCESS;
    size_t grid = (n16 + 256 * 4 - 1) / (256 * 4);
    if (grid > 256 * 64) grid = 256 * 64;
    hipLaunchKernelGGL(k_copy16, dim3((unsigned)grid), dim3(256), 0, s, (const u32x4 *)d_src, (u32x4 *)d_dst, n16);
    return check_launch();
}

// -------------------------------------------------------------------------------------------
// Calibration gather: groups of G consecutive lanes read G consecutive 32-bit words at pseudo-
// random places of a buffer (G = 1: every lane its own 128-byte line; G = 64: the wave reads a
// 256-byte row, the access of an N = 64 fp32 SpMM), 8 loads in flight per lane.  Measures how many
// independent lines per second the memory system delivers past the L2s.
// -------------------------------------------------------------------------------------------
template <int G>
__global__ __launch_bounds__(256) void k_gather_lines(const uint32_t *__restrict__ buf, uint64_t units, int per_lane,
                                                      uint32_t *__restrict__ out)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t state = (tid / G) * 0x9E3779B97F4A7C15ull + 0x2545F4914F6CDD1Dull;
    const uint32_t in_group = (uint32_t)(tid % G);
    uint32_t sum = 0;
    for (int i = 0; i < per_lane; i += 8) {
        uint32_t v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            state = state * 6364136223846793005ull + 1442695040888963407ull;
            const uint64_t u = __umul64hi(state, units);  // uniform in [0, units)
            // a unit is G words for G >= 32, else a 128-byte line of which the lane reads one word
            v[j] = buf[G >= 32 ? u * G + in_group : u * 32 + in_group];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) sum += v[j];
    }
    out[tid] = sum;
}

int launch_gather_lines(const void *d_buf, size_t bytes, int group_lanes, int per_lane, void *d_out, int *nthreads,
                        hipStream_t s)
{
    const int grid = 256 * 8, threads = grid * 256;
    if (nthreads) *nthreads = threads;
    if (!d_out) return ASX_STATUS_SUCCESS;  // size query
    if (per_lane < 8 || per_lane % 8) return ASX_STATUS_INVALID_VALUE;
    if (group_lanes == 1) {
        if (bytes < 128) return ASX_STATUS_INVALID_SIZE;
        hipLaunchKernelGGL(k_gather_lines<1>, dim3(grid), dim3(256), 0, s, (const uint32_t *)d_buf, (uint64_t)(bytes / 128),
                           per_lane, (uint32_t *)d_out);
    } else if (group_lanes == 64) {
        if (bytes < 256) return ASX_STATUS_INVALID_SIZE;
        hipLaunchKernelGGL(k_gather_lines<64>, dim3(grid), dim3(256), 0, s, (const uint32_t *)d_buf, (uint64_t)(bytes / 256),
                           per_lane, (uint32_t *)d_out);
    } else {
        return ASX_STATUS_INVALID_VALUE;
    }
    return check_launch();
}


// ---- a checksum of the caller's values ------------------------------------------------------
// Two 64-bit sums over the 32-bit words of an array, each word mixed with its position (a
// changed word always changes the first sum: its term is the product of two non-zero 32-bit
// numbers; swapped words change it unless the mixed values collide).  Sums of terms: any order of
// accumulation gives the same pair.  Every workgroup leaves its two sums in partials[2 * blockIdx.x]
// (no atomics: thousands of them on one address take longer than reading the values).
constexpr int kChecksumThreads = 256;
__global__ __launch_bounds__(kChecksumThreads) void k_checksum_words(const uint32_t *__restrict__ data, int64_t nwords,
                                                                     unsigned long long *__restrict__ partials)
{
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    __shared__ unsigned long long s_sum[2 * kChecksumThreads / kWave];
    unsigned long long h1 = 0, h2 = 0;
    const int64_t nvec = nwords / 4;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const auto mix = [&](uint32_t w, int64_t j) {
        const uint32_t jj = (uint32_t)j, a = w + 0x9E3779B9u * jj;
        h1 += (unsigned long long)a * ((0x85EBCA6Bu ^ jj) | 1u) + (unsigned long long)(j >> 32);
        h2 += (unsigned long long)(a ^ (a >> 15)) * (0xC2B2AE35u + 2u * jj + 1u);
    };
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += stride) {
        const u32x4 q = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(data) + v);
        mix(q.x, 4 * v);
        mix(q.y, 4 * v + 1);
        mix(q.z, 4 * v + 2);
        mix(q.w, 4 * v + 3);
    }
    if (blockIdx.x == 0 && threadIdx.x < (int)(nwords - 4 * nvec)) mix(data[4 * nvec + threadIdx.x], 4 * nvec + threadIdx.x);
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        h1 += __shfl_xor(h1, d, kWave);
        h2 += __shfl_xor(h2, d, kWave);
    }
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) s_sum[2 * wave] = h1, s_sum[2 * wave + 1] = h2;
    __syncthreads();
    if (threadIdx.x < 2) {
        unsigned long long t = 0;
        for (int k = 0; k < kChecksumThreads / kWave; ++k) t += s_sum[2 * k + threadIdx.x];
        partials[2 * (int64_t)blockIdx.x + threadIdx.x] = t;
    }
}
// now[0..1] = the sums over the workgroups' partial sums (one workgroup)
__global__ __launch_bounds__(kChecksumThreads) void k_checksum_finish(const unsigned long long *__restrict__ partials,
                                                                      int32_t nparts, unsigned long long *__restrict__ now)
{
    __shared__ unsigned long long s_sum[2 * kChecksumThreads / kWave];
    unsigned long long h1 = 0, h2 = 0;
    for (int32_t i = threadIdx.x; i < nparts; i += kChecksumThreads) h1 += partials[2 * i], h2 += partials[2 * i + 1];
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        h1 += __shfl_xor(h1, d, kWave);
        h2 += __shfl_xor(h2, d, kWave);
    }
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) s_sum[2 * wave] = h1, s_sum[2 * wave + 1] = h2;
    __syncthreads();
    if (threadIdx.x < 2) {
        unsigned long long t = 0;
        for (int k = 0; k < kChecksumThreads / kWave; ++k) t += s_sum[2 * k + threadIdx.x];
        now[threadIdx.x] = t;
    }
}
// kept = now (after the copy was brought up to the values the sums were taken from)
__global__ void k_checksum_commit(const unsigned long long *now, unsigned long long *kept)
{
    if (threadIdx.x < 2 && blockIdx.x == 0) kept[threadIdx.x] = now[threadIdx.x];
}

int checksum_parts()
{
    int cus = 256;
    (void)asx_device_info(&cus, nullptr);
    return cus * 8;
}
int launch_checksum(const void *d_data, size_t bytes, unsigned long long *d_partials, unsigned long long *d_now, hipStream_t s)
{
    if (((uintptr_t)d_data % 16) != 0 || bytes % 4 != 0) return ASX_STATUS_INVALID_VALUE;
    const int64_t nwords = (int64_t)(bytes / 4);
    const int64_t want = ceil_div64(nwords / 4 + 1, kChecksumThreads * 4);  // about four 16-byte loads a thread
    const int parts = (int)std::max<int64_t>(1, std::min<int64_t>(want, checksum_parts()));
    hipLaunchKernelGGL(k_checksum_words, dim3((unsigned)parts), dim3(kChecksumThreads), 0, s, (const uint32_t *)d_data, nwords,
                       d_partials);
    hipLaunchKernelGGL(k_checksum_finish, dim3(1), dim3(kChecksumThreads), 0, s, d_partials, parts, d_now);
    return check_launch();
}
int launch_checksum_commit(const unsigned long long *d_now, unsigned long long *d_kept, hipStream_t s)
{
    hipLaunchKernelGGL(k_checksum_commit, dim3(1), dim3(64), 0, s, d_now, d_kept);
    return check_launch();
}

}  // namespace asx
