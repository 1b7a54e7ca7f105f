/*
 * CPU oracle for the CSR SpMV / SpMM hot path.  TEST INFRASTRUCTURE ONLY: the shipped
 * library never links or loads this file; tests, the smoke check and the CPU-baseline
 * leg of the benchmark are its only callers.
 *
 * Build: gcc -O2 -mfma -mavx2 -ffp-contract=off -fopenmp -shared -fPIC.
 * -ffp-contract=off matters: every rounding below is written out (fma()/fmaf() where
 * the reference fuses, separate * and + where it does not).
 */
#include "alphasparse_oracle.h"

#include <math.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- hygon/util/partition.cpp:50-65 : first index in [lo,hi) with t[idx] >= v, else hi ---- */
static int32_t first_not_less(const int32_t *t, int32_t lo, int32_t hi, int32_t v)
{
    while (lo < hi) {
        int32_t mid = (lo + hi) / 2;
        if (t[mid] < v)
            lo = mid + 1;
        else
            hi = mid;
    }
    return lo;
}

/* ---- hygon/util/partition.cpp:83-96 ----
 * The search window is [0, rows-1): an index that would land past it sticks at rows-1.
 * ave*i is a 32-bit product in the reference (ALPHA_INT); kept 32-bit here. */
void orc_partition_rows_by_nnz(const int32_t *row_end, int32_t rows, int32_t nthreads,
                               int32_t *partition)
{
    int32_t nnz = row_end[rows - 1];
    int32_t ave = nnz / nthreads;
    partition[0] = 0;
    for (int32_t i = 1; i < nthreads; ++i)
        partition[i] = first_not_less(row_end, 0, rows - 1, (int32_t)(ave * i));
    partition[nthreads] = rows;
}

/* ---- gemv_csr_serial_fma_fp64_u4.S:70-151 : one row ----
 * Four running sums (the two lanes of two 128-bit accumulators) over groups of four
 * stored entries, folded as (s2+s0) and (s3+s1), then high+low; up to three left-over
 * entries by scalar fma in order; y = fma(alpha, sum, beta*y). */
static inline double row_dot_f64(const int32_t *col, const double *val, const double *x,
                                 int32_t s, int32_t e)
{
    double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0, sum = 0.0;
    int32_t k = s;
    if (k < e - 3) {
        for (; k < e - 3; k += 4) {
            s0 = fma(val[k], x[col[k]], s0);
            s1 = fma(val[k + 1], x[col[k + 1]], s1);
            s2 = fma(val[k + 2], x[col[k + 2]], s2);
            s3 = fma(val[k + 3], x[col[k + 3]], s3);
        }
        double lo = s2 + s0;
        double hi = s3 + s1;
        sum = hi + lo;
    }
    for (; k < e; ++k)
        sum = fma(val[k], x[col[k]], sum);
    return sum;
}

/* ---- gemv_sload_shuffle_shuffle_reduce_128.S:61-169 : one row ----
 * One 4-lane accumulator; fold = pairwise swap-add (l0+l1, l2+l3) then lane2 + lane0. */
static inline float row_dot_f32(const int32_t *col, const float *val, const float *x, int32_t s,
                                int32_t e)
{
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f, sum = 0.f;
    int32_t k = s;
    if (k < e - 3) {
        for (; k < e - 3; k += 4) {
            a0 = fmaf(val[k], x[col[k]], a0);
            a1 = fmaf(val[k + 1], x[col[k + 1]], a1);
            a2 = fmaf(val[k + 2], x[col[k + 2]], a2);
            a3 = fmaf(val[k + 3], x[col[k + 3]], a3);
        }
        float p01 = a0 + a1; /* shufps 0xb1 + addps, lane 0 */
        float p23 = a2 + a3; /* lane 2 */
        sum = p23 + p01;     /* unpckhps + addss */
    }
    for (; k < e; ++k)
        sum = fmaf(val[k], x[col[k]], sum);
    return sum;
}

static int at_least_one(int nthreads) { return nthreads < 1 ? 1 : nthreads; }

/* ---- gemv_csr.hpp:48-78 : rows are dealt to threads by orc_partition_rows_by_nnz ---- */
void orc_spmv_csr_f64(int32_t m, const int32_t *row_ptr, const int32_t *col, const double *val,
                      const double *x, double alpha, double beta, double *y, int nthreads)
{
    if (m <= 0)
        return;
    nthreads = at_least_one(nthreads);
    int32_t *part = (int32_t *)malloc(sizeof(int32_t) * (size_t)(nthreads + 1));
    orc_partition_rows_by_nnz(row_ptr + 1, m, nthreads, part);
#pragma omp parallel num_threads(nthreads)
    {
#ifdef _OPENMP
        int tid = omp_get_thread_num();
#else
        int tid = 0;
#endif
        int t0 = tid, t1 = tid + 1;
#ifndef _OPENMP
        t0 = 0;
        t1 = nthreads;
#endif
        for (int t = t0; t < t1; ++t)
            for (int32_t r = part[t]; r < part[t + 1]; ++r) {
                double sum = row_dot_f64(col, val, x, row_ptr[r], row_ptr[r + 1]);
                double by = beta * y[r];
                y[r] = fma(sum, alpha, by);
            }
    }
    free(part);
}

/* ---- gemv_csr.hpp:14-46 ---- */
void orc_spmv_csr_f32(int32_t m, const int32_t *row_ptr, const int32_t *col, const float *val,
                      const float *x, float alpha, float beta, float *y, int nthreads)
{
    if (m <= 0)
        return;
    nthreads = at_least_one(nthreads);
    int32_t *part = (int32_t *)malloc(sizeof(int32_t) * (size_t)(nthreads + 1));
    orc_partition_rows_by_nnz(row_ptr + 1, m, nthreads, part);
#pragma omp parallel num_threads(nthreads)
    {
#ifdef _OPENMP
        int tid = omp_get_thread_num();
#else
        int tid = 0;
#endif
        int t0 = tid, t1 = tid + 1;
#ifndef _OPENMP
        t0 = 0;
        t1 = nthreads;
#endif
        for (int t = t0; t < t1; ++t)
            for (int32_t r = part[t]; r < part[t + 1]; ++r) {
                float sum = row_dot_f32(col, val, x, row_ptr[r], row_ptr[r + 1]);
                float by = beta * y[r];
                y[r] = fmaf(sum, alpha, by);
            }
    }
    free(part);
}

/* ---- gemm_csr_row.hpp:15-73 ----
 * C[r,:] *= beta, then for every stored entry of the row in CSR order: v = alpha*a
 * (rounded), C[r,c] = fma(v, B[col,c], C[r,c]).  The reference's K-blocking visits the
 * entries of one row in stored order (its column-block table is built by a forward walk
 * over the row, hygon/util/partition.cpp:178-201), and its N tile (512 for fp32, 1024
 * otherwise) only changes when the beta scaling of later column tiles happens, not the
 * per-element sequence of operations.  Both the 8-lane body and the scalar tail round
 * as one fused multiply-add (the tail is `a*b+c` compiled with -mfma and GCC's default
 * contraction). */
void orc_spmm_csr_row_f32(int32_t m, const int32_t *row_ptr, const int32_t *col, const float *val,
                          const float *B, int32_t n, int32_t ldb, float alpha, float beta,
                          float *C, int32_t ldc, int nthreads)
{
    if (m <= 0)
        return;
    nthreads = at_least_one(nthreads);
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 64)
    for (int32_t r = 0; r < m; ++r) {
        float *c = C + (size_t)r * (size_t)ldc;
        for (int32_t j = 0; j < n; ++j)
            c[j] = c[j] * beta;
        for (int32_t k = row_ptr[r]; k < row_ptr[r + 1]; ++k) {
            float v = alpha * val[k];
            const float *b = B + (size_t)col[k] * (size_t)ldb;
            for (int32_t j = 0; j < n; ++j)
                c[j] = fmaf(v, b[j], c[j]);
        }
    }
}

void orc_spmm_csr_row_f64(int32_t m, const int32_t *row_ptr, const int32_t *col, const double *val,
                          const double *B, int32_t n, int32_t ldb, double alpha, double beta,
                          double *C, int32_t ldc, int nthreads)
{
    if (m <= 0)
        return;
    nthreads = at_least_one(nthreads);
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 64)
    for (int32_t r = 0; r < m; ++r) {
        double *c = C + (size_t)r * (size_t)ldc;
        for (int32_t j = 0; j < n; ++j)
            c[j] = c[j] * beta;
        for (int32_t k = row_ptr[r]; k < row_ptr[r + 1]; ++k) {
            double v = alpha * val[k];
            const double *b = B + (size_t)col[k] * (size_t)ldb;
            for (int32_t j = 0; j < n; ++j)
                c[j] = fma(b[j], v, c[j]);
        }
    }
}

/* ---- alphasparse_spmm_utils.h:22-36 + alphasparse_spmm_csr_nnz_split.h:7-47 ----
 * Largest r with row_ptr[r] <= e.  For e < nnz that r is < m and is the row holding
 * stored element e (empty rows that share the offset are skipped). */
static int32_t last_row_not_after(const int32_t *row_ptr, int32_t m, int64_t e)
{
    int32_t lo = 0, hi = m; /* invariant: row_ptr[lo] <= e */
    while (lo < hi) {
        int32_t mid = lo + (hi - lo + 1) / 2;
        if ((int64_t)row_ptr[mid] <= e)
            lo = mid;
        else
            hi = mid - 1;
    }
    return lo;
}

void orc_nnz_split_rows(const int32_t *row_ptr, int32_t m, int32_t nnz, int32_t items, int32_t *out)
{
    int32_t nseg = (int32_t)(((int64_t)nnz + items - 1) / items);
    for (int32_t t = 0; t < nseg; ++t)
        out[t] = last_row_not_after(row_ptr, m, (int64_t)t * items);
    out[nseg] = m;
}

/* ---- alphasparse_spmv_csr_merge_ginkgo.h:10-33,132-157 ----
 * Diagonal d = min(items*g, m+nnz).  x = least p in [max(d-nnz,0), min(d,m)] such that
 * row_end[p] >= d - p (or the upper end of the window), y = d - x. */
void orc_merge_path_search(const int32_t *row_ptr, int32_t m, int32_t nnz, int32_t items,
                           int32_t *xs, int32_t *ys)
{
    const int32_t *row_end = row_ptr + 1;
    int64_t total = (int64_t)m + nnz;
    int32_t nblk = (int32_t)((total + items - 1) / items);
    for (int32_t g = 0; g <= nblk; ++g) {
        int64_t d = (int64_t)items * g;
        if (d > total)
            d = total;
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
}

/* ---- alphasparse_spmv_csr_row_partition_ginkgo.h:93-122 ----
 * The thresholds are the float literals 2e5..2e8 converted to the integer type. */
int64_t orc_loadbalance_nwarps(int64_t nnz, int64_t warp_size, int64_t nwarps_base)
{
    if (warp_size <= 0)
        return 0;
    int64_t mult = 8;
    if (nnz >= 200000000)
        mult = 2048;
    else if (nnz >= 20000000)
        mult = 512;
    else if (nnz >= 2000000)
        mult = 128;
    else if (nnz >= 200000)
        mult = 32;
    int64_t cap = nwarps_base * mult;
    int64_t need = (nnz + warp_size - 1) / warp_size;
    return need < cap ? need : cap;
}

/* ---- alphasparse_spmv_csr_row_partition_ginkgo.h:15-42 with the host call at :419-424 ----
 * acc = row_ptr+1 searched over the closed index range [0, m-1]; the answer may be m. */
void orc_loadbalance_partition(const int32_t *row_ptr, int32_t m, int32_t nnz, int32_t warp_size,
                               int32_t nwarps, int32_t *out)
{
    const int32_t *acc = row_ptr + 1;
    int64_t ave = ((int64_t)nnz + warp_size - 1) / warp_size;
    for (int32_t g = 0; g < nwarps; ++g) {
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
}

/* ---- alphasparse_spmv_csr_adaptive2.h:5-47 ---- */
void orc_find_rows_counts(const int32_t *row_ptr, int32_t m, int32_t thr1, int32_t thr2,
                          int32_t counts[3], int64_t *nnz_mid)
{
    counts[0] = counts[1] = counts[2] = 0;
    *nnz_mid = 0;
    for (int32_t r = 0; r < m; ++r) {
        int32_t len = row_ptr[r + 1] - row_ptr[r];
        if (len < thr1)
            counts[0]++;
        else if (len < thr2) {
            counts[1]++;
            *nnz_mid += len;
        } else
            counts[2]++;
    }
}

/* ---- include/alphasparse/common.h:12-20 : largest power of two <= v (0 for 0) ---- */
static uint32_t pow2_floor(uint32_t v)
{
    uint32_t p = 0;
    for (int b = 31; b >= 0; --b)
        if (v & (1u << b)) {
            p = 1u << b;
            break;
        }
    return p;
}

/* include/alphasparse/common.h:192-200 with WG_SIZE 256 */
static uint64_t reduction_threads(uint64_t nrows) { return pow2_floor((uint32_t)(256 / nrows)); }

/* ---- alphasparse_spmv_csr_adaptive.h:354-568 ----
 * Greedy scan over rows producing packed entries (first_row << 32 | low bits).  Constants
 * at :6-11: 1024 entries per block, long rows get one entry per 3*1024 entries, a block
 * of more than one row carries the reduction thread count in its low bits (ORed into the
 * block's opening entry when the block is closed).  Rows longer than 128 open a "long"
 * run; the run ends at the first row shorter than 32. */
size_t orc_csr_adaptive_row_blocks(const int32_t *row_ptr, int32_t m, uint64_t *out, size_t cap)
{
    const uint64_t BLK = 1024, MULT = 3, VEC_ROWS = 1;
    size_t n = 0;
#define PUT(v)                                                                                     \
    do {                                                                                           \
        if (n < cap)                                                                               \
            out[n] = (v);                                                                          \
        ++n;                                                                                       \
    } while (0)
#define TAG_PREV(cnt)                                                                              \
    do {                                                                                           \
        if ((cnt) > VEC_ROWS && n >= 2 && n - 2 < cap)                                             \
            out[n - 2] |= reduction_threads(cnt);                                                  \
    } while (0)
    PUT(0);
    uint64_t sum = 0, i, last = 0;
    int32_t long_run = 0;
    for (i = 1; i <= (uint64_t)m; ++i) {
        int32_t len = row_ptr[i] - row_ptr[i - 1];
        sum += (uint64_t)len;
        if (len > 128)
            ++long_run;
        else if (long_run > 0)
            long_run = (len < 32) ? -1 : long_run + 1;

        if (long_run == 1) {
            /* first long row after short ones: close the short rows' block */
            if (i - last > 1) {
                PUT((i - 1) << 32);
                TAG_PREV((i - 1) - last);
                last = i - 1;
                sum = (uint64_t)len;
            }
        } else if (long_run == -1) {
            /* first short row after long ones that had not filled a block */
            PUT((i - 1) << 32);
            TAG_PREV((i - 1) - last);
            last = i - 1;
            sum = (uint64_t)len;
            long_run = 0;
        }

        if (i - last == 1 && sum > BLK) {
            /* one row alone exceeds a block: several workgroups share it */
            int32_t nwg = (int32_t)ceil((double)len / (double)(MULT * BLK));
            if (nwg > (1 << 24))
                nwg = 1 << 24;
            for (int32_t w = 1; w < nwg; ++w)
                PUT(((i - 1) << 32) | (uint64_t)w);
            PUT(i << 32);
            last = i;
            sum = 0;
            long_run = 0;
        } else if (i - last > 1 && sum > BLK) {
            /* this row does not fit: close before it and visit it again */
            --i;
            PUT(i << 32);
            TAG_PREV(i - last);
            last = i;
            sum = 0;
            long_run = 0;
        } else if (sum == BLK) {
            PUT(i << 32);
            TAG_PREV(i - last);
            last = i;
            sum = 0;
            long_run = 0;
        }
    }
    /* trailing rows that did not fill a block; the thread count uses the loop index as it
     * stands after the loop (m+1), as the reference does */
    uint64_t tail_row = (n - 1 < cap) ? (out[n - 1] >> 32) : (uint64_t)m;
    if (tail_row != (uint64_t)m) {
        PUT(((uint64_t)m) << 32);
        if (((uint64_t)m - last) > VEC_ROWS && n >= 2 && n - 2 < cap)
            out[n - 2] |= reduction_threads(i - last);
    }
#undef PUT
#undef TAG_PREV
    return n;
}

/* ---- hip/format/coo2csr.h:7-16 -> hipsparseXcoo2csr: counting form of the contract ---- */
void orc_coo2csr(const int32_t *row_ind, int32_t nnz, int32_t m, int32_t *row_ptr)
{
    for (int32_t r = 0; r <= m; ++r)
        row_ptr[r] = 0;
    for (int32_t i = 0; i < nnz; ++i)
        if (row_ind[i] >= 0 && row_ind[i] < m)
            row_ptr[row_ind[i] + 1]++;
    for (int32_t r = 0; r < m; ++r)
        row_ptr[r + 1] += row_ptr[r];
}
